"""Runs a zoo.GraphSpec on the CPU oracle, node by node.  TEST INFRASTRUCTURE ONLY (see espdl_oracle.h).

It mirrors what dl::Model does with the same spec: per node, read attributes the way the reference's
Module::deserialize does (pads arrive in ONNX order [t,l,b,r] and are re-ordered to [t,b,l,r],
esp-dl/dl/module/include/dl_module_conv.hpp:186-190), derive shift[c] = out_exp - w_exp[c] - in_exp
(esp-dl/dl/base/dl_base.hpp:243-261) and call the oracle function of the operator.
"""
import numpy as np

import espdl_oracle as oracle

INT8, INT16 = 3, 5


def _shift(spec, node, x_name, w_name, y_name):
    w_exps = np.array(spec.initializers[w_name][3], dtype=np.int64)
    return (spec.exponent(y_name) - w_exps - spec.exponent(x_name)).astype(np.int32)


def run(spec, inputs, round_mode=oracle.ROUND_HALF_UP, keep_all=True, state=None):
    """inputs: {name: ndarray for the whole batch}.  Returns {tensor name: ndarray}.  `state` (a dict the
    caller keeps between calls) holds the frames StreamingCache nodes carry from one call to the next."""
    t = dict(inputs)
    state = {} if state is None else state

    def operand(name):
        """An activation, or a constant operand (initializer) as stored."""
        if name in t:
            return t[name]
        dims, _, data, _ = spec.initializers[name]
        return np.asarray(data).reshape(dims)

    def exponent_of(name):
        return spec.exponent(name) if name in spec.value_info else int(spec.initializers[name][3][0])

    for node in spec.nodes:
        op, a = node["op_type"], node["attrs"]
        ins, outs = node["inputs"], node["outputs"]
        x = operand(ins[0])
        y_name = outs[0]
        if op == "Conv":
            dims, wdt, w, _ = spec.initializers[ins[1]]
            bias = spec.initializers[ins[2]][2] if len(ins) > 2 else None
            shift = _shift(spec, node, ins[0], ins[1], y_name)
            act = oracle.RELU if a.get("activation", "Linear") == "Relu" else oracle.LINEAR
            depthwise = a.get("group", 1) != 1
            s16 = a.get("quant_type") == "S16"
            fn = {(False, False): oracle.conv2d_s8, (True, False): oracle.depthwise_s8,
                  (False, True): oracle.conv2d_s16, (True, True): oracle.depthwise_s16}[(depthwise, s16)]
            if x.ndim == 3:  # Conv1d on NWC runs as one image row (dl_module_conv.hpp: 3-D inputs)
                pl, pr = a["pads"]
                y = fn(x[:, None], w, bias, shift, (1, dims[0]), (1, a["strides"][0]), (1, a["dilations"][0]),
                       (0, 0, pl, pr), act, round_mode)[:, 0]
            else:
                pt, pl, pb, pr = a["pads"]
                y = fn(x, w, bias, shift, (dims[0], dims[1]), tuple(a["strides"]), tuple(a["dilations"]),
                       (pt, pb, pl, pr), act, round_mode)
        elif op == "MatMul" and ins[1] in t:
            # two activations: per matrix pair a 1x1 convolution with one shift
            shift = spec.exponent(y_name) - spec.exponent(ins[0]) - spec.exponent(ins[1])
            act = oracle.RELU if a.get("activation", "Linear") == "Relu" else oracle.LINEAR
            y = oracle.matmul_s8(x, t[ins[1]], shift, act, round_mode)
        elif op == "Softmax":
            if x.dtype != np.int8:
                raise NotImplementedError("Softmax on " + str(x.dtype))
            y = oracle.softmax_s8(x, a.get("axis", -1), spec.exponent(ins[0]))
        elif op in ("QuantizeLinear", "DequantizeLinear") or (op == "RequantizeLinear" and x.dtype == np.float32):
            if x.dtype == np.float32:
                y = oracle.quantize_f32(x, spec.exponent(y_name), np.int16 if spec.dtype(y_name) == INT16 else np.int8)
            else:
                y = oracle.dequantize_f32(x, spec.exponent(ins[0]))
        elif op in ("Gemm", "MatMul"):
            w = spec.initializers[ins[1]][2]
            bias = spec.initializers[ins[2]][2] if len(ins) > 2 else None
            shift = _shift(spec, node, ins[0], ins[1], y_name)
            act = oracle.RELU if a.get("activation", "Linear") == "Relu" else oracle.LINEAR
            if x.dtype == np.int16:  # the same 1x1 convolution view, int16 x int16 -> int64
                k = x.shape[-1]
                y = oracle.conv2d_s16(x.reshape(1, 1, x.size // k, k), w, bias, shift, (1, 1), activation=act,
                                      round_mode=round_mode)
                y = y.reshape(x.shape[:-1] + (y.shape[-1],))
            else:
                y = oracle.gemm_s8(x, w, bias, shift, activation=act, round_mode=round_mode)
        elif "lut" in a:
            if x.dtype == np.int16:
                y = oracle.lut_s16(x, spec.initializers[a["lut"]][2], p4_ties=(round_mode == oracle.ROUND_HALF_EVEN))
            else:
                y = oracle.lut_s8(x, spec.initializers[a["lut"]][2])
        elif op == "Relu":
            y = oracle.relu_s8(x, spec.exponent(ins[0]), spec.exponent(y_name))
        elif op == "PRelu":
            alpha_dims, _, alpha, alpha_exp = spec.initializers[ins[1]]
            shift = spec.exponent(y_name) - spec.exponent(ins[0]) - alpha_exp[0]
            y = oracle.prelu_s8(x, alpha, shift)
        elif op == "Clip":
            lo = int(spec.initializers[ins[1]][2].ravel()[0]) if len(ins) > 1 else -128
            hi = int(spec.initializers[ins[2]][2].ravel()[0]) if len(ins) > 2 else 127
            y = oracle.clip_s8(x, lo, hi, spec.exponent(ins[0]), spec.exponent(y_name))
        elif op == "Add":
            # the C path adds the stored integers and saturates, whatever the exponents say
            # (esp-dl/dl/base/dl_base_add.cpp:35-44); the exporter gives all three the same exponent
            b = operand(ins[1])
            if x.shape != b.shape:
                x, b = np.broadcast_arrays(x, b)
            add = oracle.add_s16 if x.dtype == np.int16 else oracle.add_s8
            y = add(np.ascontiguousarray(x), np.ascontiguousarray(b))
        elif op in oracle.UNARY_KINDS:
            y = oracle.unary(op, x, exponent_of(ins[0]), spec.exponent(y_name), a.get("alpha"), a.get("beta"), round_mode)
        elif op == "Identity":  # output->assign(input): a requantize when the exponents differ
            y = requantize(x, spec.exponent(ins[0]), spec.exponent(y_name), spec.dtype(y_name))
        elif op == "SpaceToDepth":
            y = oracle.space_to_depth(x, a.get("blocksize", 2))
        elif op == "DepthToSpace":
            y = oracle.depth_to_space(x, a.get("blocksize", 2), a.get("mode", "DCR"))
        elif op == "Gather":
            dims, _, data, _ = spec.initializers[ins[1]]
            y = oracle.gather(x, np.asarray(data).reshape(dims), a.get("axis", 0))
        elif op == "Pad":
            pads = [int(v) for v in spec.initializers[ins[1]][2].ravel()]
            value = int(spec.initializers[ins[2]][2].ravel()[0]) if len(ins) > 2 and ins[2] else 0
            y = oracle.pad(x, pads, a.get("mode", "constant"), value)
        elif op == "Sub":
            b = operand(ins[1])
            if x.shape != b.shape:
                x, b = np.broadcast_arrays(x, b)
            sub = oracle.sub_s16 if x.dtype == np.int16 else oracle.sub_s8
            y = sub(np.ascontiguousarray(x), np.ascontiguousarray(b))
        elif op == "Div":
            b = operand(ins[1])
            div = oracle.div_s16 if x.dtype == np.int16 else oracle.div_s8
            y = div(x, b, spec.exponent(y_name) - exponent_of(ins[0]) + exponent_of(ins[1]))
        elif op == "Mul":
            b = operand(ins[1])
            shift = spec.exponent(y_name) - exponent_of(ins[0]) - exponent_of(ins[1])
            if x.shape != b.shape:  # broadcast explicitly: the oracle takes equal sizes or a scalar
                x, b = np.broadcast_arrays(x, b)
            mul = oracle.mul_s16 if x.dtype == np.int16 else oracle.mul_s8
            y = mul(np.ascontiguousarray(x), np.ascontiguousarray(b), shift, round_mode)
        elif op == "GlobalAveragePool":
            y = oracle.global_avg_pool_s8(x, spec.exponent(ins[0]), spec.exponent(y_name))
        elif op == "RequantizeLinear":
            y = requantize(x, spec.exponent(ins[0]), spec.exponent(y_name), spec.dtype(y_name))
        elif op == "Flatten":
            y = x.reshape(x.shape[0], -1)
        elif op in ("Squeeze", "Unsqueeze"):
            axes = a["axes"] if "axes" in a else [int(v) for v in spec.initializers[ins[1]][2].ravel()]
            y = np.squeeze(x, axis=tuple(axes)) if op == "Squeeze" else np.expand_dims(x, tuple(axes))
        elif op == "Reshape":
            # exported target shapes are per image (leading 1); a batch keeps its own leading extent
            shape = [int(v) for v in spec.initializers[ins[1]][2].ravel()]
            per_image = x.size // x.shape[0]
            rest = [d if d != 0 else x.shape[i] for i, d in enumerate(shape)][1:]
            if -1 in rest:
                known = int(np.prod([d for d in rest if d != -1]))
                rest[rest.index(-1)] = per_image // max(1, known)
            y = x.reshape([x.shape[0]] + rest)
        elif op == "AveragePool":
            k, st, pads = list(a["kernel_shape"]), list(a.get("strides") or [1] * len(a["kernel_shape"])), list(a.get("pads") or [])
            avg_pool = oracle.avg_pool_s16 if x.dtype == np.int16 else oracle.avg_pool_s8
            if x.ndim == 3:  # NWC runs as one row
                pl, pr = pads if pads else (0, 0)
                y = avg_pool(x[:, None], (1, k[0]), (1, st[0]), (0, 0, pl, pr), spec.exponent(ins[0]),
                                       spec.exponent(y_name))[:, 0]
            else:
                pt, pl, pb, pr = pads if pads else (0, 0, 0, 0)
                y = avg_pool(x, tuple(k), tuple(st), (pt, pb, pl, pr), spec.exponent(ins[0]), spec.exponent(y_name))
        elif op == "ReduceMean":
            axes = spec.initializers[ins[1]][2].ravel() if len(ins) > 1 and ins[1] in spec.initializers else a.get("axes", [])
            if len(axes) == 0 and a.get("noop_with_empty_axes", 0):
                y = x
            else:
                reduce_mean = oracle.reduce_mean_s16 if x.dtype == np.int16 else oracle.reduce_mean_s8
                y = reduce_mean(x, [int(v) for v in axes], bool(a.get("keepdims", 1)), spec.exponent(ins[0]),
                                spec.exponent(y_name))
        elif op in oracle.REDUCE_OPS:
            axes = spec.initializers[ins[1]][2].ravel() if len(ins) > 1 and ins[1] in spec.initializers else a.get("axes", [])
            if len(axes) == 0 and a.get("noop_with_empty_axes", 0):
                y = x
            else:
                y = oracle.reduce_int(op, x, [int(v) for v in axes], bool(a.get("keepdims", 1)),
                                      spec.exponent(y_name) - spec.exponent(ins[0]) * (2 if op == "ReduceSumSquare" else 1),
                                      round_mode)
        elif op == "Slice":
            par = [spec.initializers[n][2].ravel() if n in spec.initializers else None for n in (ins[1:5] + [None] * 4)[:4]]
            y = oracle.slice_(x, par[0], par[1], par[2], par[3])
        elif op == "MaxPool":
            pt, pl, pb, pr = a["pads"]
            y = oracle.max_pool(x, tuple(a["kernel_shape"]), tuple(a["strides"]), (pt, pb, pl, pr))
        elif op == "Concat":
            y = oracle.concat([t[n] for n in ins], a["axis"])
        elif op == "Split":
            sizes = [int(v) for v in spec.initializers[ins[1]][2].ravel()]
            for name, piece in zip(outs, oracle.split(x, a["axis"], sizes)):
                t[name] = piece
            continue
        elif op == "Resize":
            scales = spec.initializers[ins[2]][2].ravel()
            y = oracle.resize_nearest_s8(x, scales[2], scales[3], spec.exponent(ins[0]), spec.exponent(y_name))
        elif op == "StreamingCache":
            # esp-dl/dl/module/include/dl_module_streaming_cache.hpp: [previous window_size - 1 frames | input]
            # along axis 1, zeros before the first call; the last frames of the result are kept
            keep = a.get("window_size", 1) - 1
            if a.get("frame_axis", 1) % x.ndim != 1:
                raise NotImplementedError("StreamingCache along axis %d" % a.get("frame_axis", 1))
            prev = state.get(node["name"])
            if prev is None:
                prev = np.zeros((x.shape[0], keep) + x.shape[2:], dtype=x.dtype)
            y = np.concatenate([prev, x], axis=1)
            state[node["name"]] = y[:, y.shape[1] - keep:].copy()
        elif op == "InsertZeros":
            st, op_pad = list(a["stride"]), list(a.get("output_padding") or [0])
            if x.ndim == 3:
                y = oracle.insert_zeros(x[:, :, None], (st[0], 1), (op_pad[0], 0))[:, :, 0]
            else:
                st = st * 2 if len(st) == 1 else st
                op_pad = op_pad * 2 if len(op_pad) == 1 else op_pad
                y = oracle.insert_zeros(x, st, op_pad)
        elif op == "Transpose":
            y = oracle.transpose(x, list(a["perm"]))
        else:
            raise NotImplementedError(op)
        t[y_name] = y
    return t if keep_all else {k: t[k] for k in spec.outputs}


def requantize(x, in_exp, out_exp, out_dtype_code):
    """TensorBase::assign across exponents / widths (esp-dl/dl/tensor/src/dl_tensor_base.cpp:321-392):
    same exponent -> widen or saturate; otherwise quantize(dequantize(x)) in float32 with round-half-up."""
    out_np = np.int16 if out_dtype_code == INT16 else np.int8
    lo, hi = (-32768, 32767) if out_dtype_code == INT16 else (-128, 127)
    if x.dtype == np.int8 and out_np == np.int8:
        return oracle.requantize_s8(x, in_exp, out_exp)
    if in_exp == out_exp:
        return np.clip(x.astype(np.int32), lo, hi).astype(out_np)
    src_scale = np.float32(2.0 ** in_exp)
    inv_scale = np.float32(1.0 / np.float32(2.0 ** out_exp))
    tmp = x.astype(np.float32) * src_scale
    q = np.floor((tmp * inv_scale).astype(np.float64) + 0.5).astype(np.float32)
    return np.clip(q.astype(np.int64), lo, hi).astype(out_np)
