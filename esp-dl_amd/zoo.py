"""Seeded synthetic graphs in ESP-DL's exported form (what an `.espdl` file holds), for the five
benchmark configurations: nodes with ONNX-style attributes, int8/int16 initializers with per-tensor
or per-channel exponents, int32/int64 biases with exponent in_exp + w_exp[c], 8-bit LUT tables,
value_info exponents.  There are no datasets or trained weights: everything is drawn from
numpy's PCG64 with the seeds given here.

A GraphSpec is plain data.  `espdl.model.Graph.from_spec` turns it into the native fbs::FbsModel;
the CPU oracle's graph runner executes the same spec, so both sides see identical bytes.

Layouts follow the reference's `c` target: dense filter initializer dims [kH,kW,Cin,Cout] over
[Cout][kH][kW][Cin] bytes, depthwise dims [kH,kW,C,1] over [kH][kW][C] bytes, Gemm dims [1,1,K,N]
over [N][K] bytes (esp-dl/dl/base/dl_base_conv2d.cpp:23,64,140; dl_base_depthwise_conv2d.cpp:46-65).
"""
import math

import numpy as np

FLOAT, INT8, INT16, INT32, INT64 = 1, 3, 5, 6, 7
_NP = {FLOAT: np.float32, INT8: np.int8, INT16: np.int16, INT32: np.int32, INT64: np.int64}


class GraphSpec:
    def __init__(self, name):
        self.name = name
        self.initializers = {}  # name -> (dims, dtype_code, ndarray (bytes as stored), exponents list)
        self.value_info = {}    # name -> (per-image dims with leading 1, dtype_code, exponent)
        self.nodes = []         # dicts: name, op_type, inputs, outputs, attrs
        self.inputs = []
        self.outputs = []
        self.macs_per_image = 0
        self.conv_macs_per_image = 0

    # -- construction helpers ------------------------------------------------------------------
    def add_init(self, name, dims, dtype, data, exponents):
        data = np.ascontiguousarray(data, dtype=_NP[dtype])
        assert data.size == int(np.prod(dims)), (name, dims, data.shape)
        self.initializers[name] = (list(dims), dtype, data, [int(e) for e in exponents])

    def add_value(self, name, dims, exponent, dtype=INT8):
        self.value_info[name] = (list(dims), dtype, int(exponent))

    def add_node(self, name, op_type, inputs, outputs, **attrs):
        assert all(n["name"] != name for n in self.nodes), "duplicate node name " + name
        self.nodes.append({"name": name, "op_type": op_type, "inputs": list(inputs), "outputs": list(outputs),
                           "attrs": attrs})

    def shape(self, name):
        return self.value_info[name][0]

    def exponent(self, name):
        return self.value_info[name][2]

    def dtype(self, name):
        return self.value_info[name][1]

    def make_input(self, rng, batch, name=None):
        """Seeded uniform input for the (single) graph input, whole batch."""
        name = name or self.inputs[0]
        dims, dtype, _ = self.value_info[name]
        shape = [batch * dims[0]] + dims[1:]
        if dtype == INT16:
            return rng.integers(-32768, 32768, size=shape, dtype=np.int64).astype(np.int16)
        return rng.integers(-128, 128, size=shape, dtype=np.int64).astype(np.int8)


def typical_shift(k_total):
    """Shift that maps the accumulator of K uniform-int8 products to a std of about 40."""
    return max(1, int(round(math.log2(5461.0 * math.sqrt(k_total) / 40.0))))


class Builder:
    """Adds layers to a GraphSpec, tracking the current tensor name."""

    def __init__(self, spec, seed, per_channel=True, w_exp_range=(-10, -6), bits=8):
        self.g = spec
        self.rng = np.random.default_rng(seed)
        self.per_channel = per_channel
        self.w_exp_range = w_exp_range
        self.n = 0

    def _name(self, prefix):
        self.n += 1
        return "%s_%d" % (prefix, self.n)

    def _w_exps(self, oc, k_total=64):
        """Per-channel filter exponents.  With an explicit range they are drawn from it; otherwise from
        [-s-2, -s+2] with s = typical_shift(k_total), so that a layer neither amplifies nor shrinks its
        input scale (trained networks behave the same way: the shipped MobileNetV2 has filter exponents
        between -7 and -12 and activations that stay within a few exponents of each other)."""
        if self.w_exp_range is None:
            s = typical_shift(k_total)
            lo, hi = -s - 2, -s + 2
        else:
            lo, hi = self.w_exp_range
        if self.per_channel:
            return self.rng.integers(lo, hi + 1, size=oc).astype(np.int64)
        return np.array([(lo + hi) // 2], dtype=np.int64)

    def input(self, name, dims, exponent, dtype=INT8):
        self.g.add_value(name, dims, exponent, dtype)
        self.g.inputs.append(name)
        return name

    def conv(self, x, out_c, k=1, stride=1, pad=None, dilation=1, depthwise=False, relu=False, bias=True,
             out_exp=None, name=None, s16=False, gain=0):
        """Conv2D (dense or depthwise).  `gain` lowers the output exponent (finer scale, more saturation)."""
        g = self.g
        _, h, w, c = g.shape(x)
        kh, kw = (k, k) if isinstance(k, int) else k
        sh, sw = (stride, stride) if isinstance(stride, int) else stride
        dh, dw = (dilation, dilation) if isinstance(dilation, int) else dilation
        if pad is None:
            pad = (dh * (kh - 1) // 2, dh * (kh - 1) // 2, dw * (kw - 1) // 2, dw * (kw - 1) // 2)
        pt, pb, pl, pr = pad
        oc = c if depthwise else out_c
        oh = (h + pt + pb - dh * (kh - 1) - 1) // sh + 1
        ow = (w + pl + pr - dw * (kw - 1) - 1) // sw + 1
        name = name or self._name("dwconv" if depthwise else "conv")
        wdt = INT16 if s16 else INT8
        lim = 32768 if s16 else 128
        if depthwise:
            wt = self.rng.integers(-lim, lim, size=(kh, kw, c))
            dims = [kh, kw, c, 1]
            k_total = kh * kw
        else:
            wt = self.rng.integers(-lim, lim, size=(oc, kh, kw, c))
            dims = [kh, kw, c, oc]
            k_total = kh * kw * c
        w_exps = self._w_exps(oc, k_total) - (8 if s16 else 0)
        in_exp = g.exponent(x)
        if out_exp is None:
            med = int(np.median(w_exps))
            out_exp = typical_shift(k_total) + (8 if s16 else 0) + in_exp + med - gain
        g.add_init(name + ".weight", dims, wdt, wt, w_exps)
        inputs = [x, name + ".weight"]
        if bias:
            if s16:
                b = self.rng.integers(-2 ** 26, 2 ** 26, size=oc)
                g.add_init(name + ".bias", [oc], INT64, b, in_exp + w_exps)
            else:
                b = self.rng.integers(-4096, 4097, size=oc)
                g.add_init(name + ".bias", [oc], INT32, b, in_exp + w_exps)
            inputs.append(name + ".bias")
        y = name + "_out"
        g.add_value(y, [1, oh, ow, oc], out_exp, INT16 if s16 else INT8)
        # pads attribute in ONNX order [t, l, b, r] (Conv::deserialize re-orders it)
        g.add_node(name, "Conv", inputs, [y], pads=[pt, pl, pb, pr], strides=[sh, sw], dilations=[dh, dw],
                   group=(c if depthwise else 1), activation=("Relu" if relu else "Linear"),
                   quant_type=("S16" if s16 else "S8"))
        macs = oh * ow * oc * k_total
        g.macs_per_image += macs
        g.conv_macs_per_image += macs
        return y

    def gemm(self, x, out_f, relu=False, bias=True, out_exp=None, name=None, matmul=False):
        g = self.g
        dims = g.shape(x)
        k = dims[-1]
        name = name or self._name("matmul" if matmul else "gemm")
        wt = self.rng.integers(-128, 128, size=(out_f, k))
        w_exps = self._w_exps(out_f, k)
        in_exp = g.exponent(x)
        if out_exp is None:
            out_exp = typical_shift(k) + in_exp + int(np.median(w_exps))
        g.add_init(name + ".weight", [1, 1, k, out_f], INT8, wt, w_exps)
        inputs = [x, name + ".weight"]
        if bias and not matmul:
            b = self.rng.integers(-4096, 4097, size=out_f)
            g.add_init(name + ".bias", [out_f], INT32, b, in_exp + w_exps)
            inputs.append(name + ".bias")
        y = name + "_out"
        g.add_value(y, dims[:-1] + [out_f], out_exp)
        g.add_node(name, "MatMul" if matmul else "Gemm", inputs, [y], activation=("Relu" if relu else "Linear"),
                   quant_type="S8")
        g.macs_per_image += int(np.prod(dims[1:-1])) * k * out_f if len(dims) > 2 else k * out_f
        return y

    def lut(self, x, fn, op_type="LUT", out_exp=None, name=None):
        """8-bit table activation: table[i] = clip(round(fn((i-128) * 2^in_exp) / 2^out_exp))."""
        g = self.g
        name = name or self._name(op_type.lower())
        in_exp = g.exponent(x)
        out_exp = in_exp if out_exp is None else out_exp
        table = make_lut(fn, in_exp, out_exp)
        g.add_init(name + ".lut", [256], INT8, table, [out_exp])
        y = name + "_out"
        g.add_value(y, g.shape(x), out_exp)
        g.add_node(name, op_type, [x], [y], lut=name + ".lut", quant_type="S8")
        return y

    def lut_s16(self, x, fn, points=2048, op_type="LUT", out_exp=None, name=None):
        """16-bit table activation: `points` + 1 samples of fn, one every 65536 / points input steps;
        the operator takes the nearest sample."""
        g = self.g
        name = name or self._name(op_type.lower())
        in_exp = g.exponent(x)
        out_exp = in_exp if out_exp is None else out_exp
        step = 65536 // points
        q = (np.arange(points + 1, dtype=np.int64) * step - 32768).astype(np.float64)
        table = np.clip(np.floor(fn(q * 2.0 ** in_exp) / 2.0 ** out_exp + 0.5), -32768, 32767).astype(np.int16)
        g.add_init(name + ".lut", [points + 1], INT16, table, [out_exp])
        y = name + "_out"
        g.add_value(y, g.shape(x), out_exp, INT16)
        g.add_node(name, op_type, [x], [y], lut=name + ".lut", quant_type="S16")
        return y

    def clip(self, x, lo_q, hi_q, out_exp=None, name=None):
        g = self.g
        name = name or self._name("clip")
        e = g.exponent(x)
        g.add_init(name + ".min", [1], INT8, [lo_q], [e])
        g.add_init(name + ".max", [1], INT8, [hi_q], [e])
        y = name + "_out"
        g.add_value(y, g.shape(x), e if out_exp is None else out_exp)
        g.add_node(name, "Clip", [x, name + ".min", name + ".max"], [y], quant_type="S8")
        return y

    def relu(self, x, name=None):
        g = self.g
        name = name or self._name("relu")
        y = name + "_out"
        g.add_value(y, g.shape(x), g.exponent(x))
        g.add_node(name, "Relu", [x], [y], quant_type="S8")
        return y

    def prelu(self, x, name=None, alpha_exp=-7, out_exp=None):
        g = self.g
        name = name or self._name("prelu")
        c = g.shape(x)[-1]
        alpha = self.rng.integers(-128, 128, size=c)
        g.add_init(name + ".slope", [c, 1, 1], INT8, alpha, [alpha_exp])
        y = name + "_out"
        g.add_value(y, g.shape(x), g.exponent(x) if out_exp is None else out_exp)
        g.add_node(name, "PRelu", [x, name + ".slope"], [y], quant_type="S8")
        return y

    def requantize(self, x, out_exp, name=None, with_scale_input=False):
        """with_scale_input: the node carries its scale as a second, constant input, as exported files do (the
        operator itself works from the two tensors' exponents)."""
        g = self.g
        name = name or self._name("requant")
        y = name + "_out"
        g.add_value(y, g.shape(x), out_exp, g.dtype(x))
        inputs = [x]
        if with_scale_input:
            sname = name + ".scale"
            g.add_init(sname, [1], FLOAT, [2.0 ** out_exp], [0])
            inputs.append(sname)
        g.add_node(name, "RequantizeLinear", inputs, [y], quant_type="S8")
        return y

    def add(self, a, b, name=None, out_exp=None):
        """Residual add at matched exponents: the operand with the other exponent is requantized first,
        which is what the exporter does by inserting RequantizeLinear.  `out_exp` labels the result with
        another exponent, as some exported graphs do; the operator still sums the stored integers."""
        g = self.g
        name = name or self._name("add")
        ea, eb = g.exponent(a), g.exponent(b)
        if ea != eb:
            a = self.requantize(a, eb)
        y = name + "_out"
        g.add_value(y, g.shape(b), eb if out_exp is None else out_exp)
        g.add_node(name, "Add", [a, b], [y], quant_type="S8")
        return y

    def mul(self, a, b, out_exp=None, name=None):
        """Element-wise product (numpy broadcasting).  Default output exponent keeps the larger operand's
        scale when the other one is a gate in [0, 1)."""
        g = self.g
        name = name or self._name("mul")
        y = name + "_out"
        sa, sb = g.shape(a), g.shape(b)
        rank = max(len(sa), len(sb))
        pa, pb = [1] * (rank - len(sa)) + sa, [1] * (rank - len(sb)) + sb
        g.add_value(y, [max(u, v) for u, v in zip(pa, pb)], g.exponent(a) if out_exp is None else out_exp)
        g.add_node(name, "Mul", [a, b], [y], quant_type="S8")
        return y

    def global_avg_pool(self, x, out_exp=None, name=None):
        g = self.g
        name = name or self._name("gap")
        n, h, w, c = g.shape(x)
        y = name + "_out"
        # the mean of roughly uniform values shrinks by about sqrt(area): keep resolution
        e = g.exponent(x) - max(0, int(round(math.log2(math.sqrt(h * w))))) + 1 if out_exp is None else out_exp
        g.add_value(y, [1, 1, 1, c], e)
        g.add_node(name, "GlobalAveragePool", [x], [y], quant_type="S8")
        return y

    def flatten(self, x, name=None):
        g = self.g
        name = name or self._name("flatten")
        dims = g.shape(x)
        y = name + "_out"
        g.add_value(y, [1, int(np.prod(dims[1:]))], g.exponent(x))
        g.add_node(name, "Flatten", [x], [y], axis=1, quant_type="S8")
        return y

    def reduce_mean(self, x, axes, keepdims=True, out_exp=None, name=None):
        """ReduceMean with the axes as an INT64 initializer operand, as exported graphs carry them."""
        g = self.g
        name = name or self._name("mean")
        dims = g.shape(x)
        norm = [a % len(dims) for a in axes]
        count = int(np.prod([dims[a] for a in norm]))
        out = [1 if i in norm else d for i, d in enumerate(dims)] if keepdims else \
            [d for i, d in enumerate(dims) if i not in norm]
        e = g.exponent(x) - max(0, int(round(math.log2(math.sqrt(count))))) + 1 if out_exp is None else out_exp
        g.add_init(name + ".axes", [len(axes)], INT64, list(axes), [0])
        y = name + "_out"
        g.add_value(y, out, e)
        g.add_node(name, "ReduceMean", [x, name + ".axes"], [y], keepdims=1 if keepdims else 0, noop_with_empty_axes=0,
                   quant_type="S8")
        return y

    def avg_pool(self, x, k, stride=1, pad=0, out_exp=None, name=None):
        g = self.g
        name = name or self._name("avgpool")
        _, h, w, c = g.shape(x)
        oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        y = name + "_out"
        g.add_value(y, [1, oh, ow, c], g.exponent(x) if out_exp is None else out_exp)
        g.add_node(name, "AveragePool", [x], [y], kernel_shape=[k, k], strides=[stride, stride],
                   pads=[pad, pad, pad, pad], quant_type="S8")
        return y

    def reshape(self, x, shape, name=None):
        """Reshape with the per-image target shape (leading 1, one -1 allowed) as an INT64 initializer operand."""
        g = self.g
        name = name or self._name("reshape")
        total = int(np.prod(g.shape(x)))
        known = int(np.prod([d for d in shape if d != -1]))
        out = [total // known if d == -1 else d for d in shape]
        g.add_init(name + ".shape", [len(shape)], INT64, list(shape), [0])
        y = name + "_out"
        g.add_value(y, out, g.exponent(x), g.dtype(x))
        g.add_node(name, "Reshape", [x, name + ".shape"], [y], allowzero=0, quant_type="S8")
        return y

    def insert_zeros(self, x, stride=2, name=None):
        """The zero-stuffing half of a transposed convolution; a Conv follows."""
        g = self.g
        name = name or self._name("insert_zeros")
        _, h, w, c = g.shape(x)
        y = name + "_out"
        g.add_value(y, [1, h + (stride - 1) * (h - 1), w + (stride - 1) * (w - 1), c], g.exponent(x), g.dtype(x))
        g.add_node(name, "InsertZeros", [x], [y], stride=[stride, stride], output_padding=[0, 0], quant_type="S8")
        return y

    def softmax(self, x, axis=-1, name=None):
        """Softmax with a float32 result, as the exporter leaves it (QuantizeLinear follows)."""
        g = self.g
        name = name or self._name("softmax")
        y = name + "_out"
        g.add_value(y, g.shape(x), 0, FLOAT)
        g.add_node(name, "Softmax", [x], [y], axis=axis, quant_type="S8")
        return y

    def quantize(self, x, out_exp, name=None):
        g = self.g
        name = name or self._name("quantize")
        y = name + "_out"
        g.add_value(y, g.shape(x), out_exp, INT8)
        g.add_node(name, "QuantizeLinear", [x], [y], quant_type="S8")
        return y

    def matmul_act(self, a, b, out_exp=None, name=None):
        """MatMul of two activations (rank 3 or 4, equal leading dims or 1)."""
        g = self.g
        name = name or self._name("matmul")
        sa, sb = g.shape(a), g.shape(b)
        assert sa[-1] == sb[-2]
        lead = [max(p, q) for p, q in zip(sa[:-2], sb[:-2])]
        if out_exp is None:
            out_exp = typical_shift(sa[-1]) + g.exponent(a) + g.exponent(b)
        y = name + "_out"
        g.add_value(y, lead + [sa[-2], sb[-1]], out_exp)
        g.add_node(name, "MatMul", [a, b], [y], activation="Linear", quant_type="S8")
        g.macs_per_image += int(np.prod(lead[1:])) * sa[-2] * sa[-1] * sb[-1]
        return y

    def max_pool(self, x, k, stride=1, pad=None, name=None):
        g = self.g
        name = name or self._name("maxpool")
        _, h, w, c = g.shape(x)
        pad = k // 2 if pad is None else pad
        oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        y = name + "_out"
        g.add_value(y, [1, oh, ow, c], g.exponent(x), g.dtype(x))
        g.add_node(name, "MaxPool", [x], [y], kernel_shape=[k, k], pads=[pad, pad, pad, pad], strides=[stride, stride],
                   quant_type="S8")
        return y

    def concat(self, xs, axis=3, name=None):
        """Concat at one exponent: inputs at another exponent are requantized to the coarsest one first,
        as the exporter does."""
        g = self.g
        name = name or self._name("concat")
        e = max(g.exponent(x) for x in xs)
        xs = [x if g.exponent(x) == e else self.requantize(x, e, name="%s_rq%d" % (name, i)) for i, x in enumerate(xs)]
        dims = list(g.shape(xs[0]))
        dims[axis] = sum(g.shape(x)[axis] for x in xs)
        y = name + "_out"
        g.add_value(y, dims, e, g.dtype(xs[0]))
        g.add_node(name, "Concat", xs, [y], axis=axis, quant_type="S8")
        return y

    def split(self, x, sizes, axis=3, name=None):
        g = self.g
        name = name or self._name("split")
        g.add_init(name + ".split", [len(sizes)], INT64, sizes, [0])
        outs = []
        for i, sz in enumerate(sizes):
            dims = list(g.shape(x))
            dims[axis] = int(sz)
            y = "%s_out%d" % (name, i)
            g.add_value(y, dims, g.exponent(x), g.dtype(x))
            outs.append(y)
        g.add_node(name, "Split", [x, name + ".split"], outs, axis=axis, quant_type="S8")
        return outs

    def resize_nearest(self, x, scale=2, out_exp=None, name=None):
        g = self.g
        name = name or self._name("resize")
        _, h, w, c = g.shape(x)
        g.add_init(name + ".scales", [4], FLOAT, [1.0, 1.0, float(scale), float(scale)], [0])
        y = name + "_out"
        g.add_value(y, [1, int(h * np.float32(scale)), int(w * np.float32(scale)), c],
                    g.exponent(x) if out_exp is None else out_exp, g.dtype(x))
        # ONNX inputs: X, roi (absent), scales
        g.add_node(name, "Resize", [x, "", name + ".scales"], [y], mode="nearest",
                   coordinate_transformation_mode="asymmetric", quant_type="S8")
        return y

    def transpose(self, x, perm, name=None):
        g = self.g
        name = name or self._name("transpose")
        dims = g.shape(x)
        y = name + "_out"
        g.add_value(y, [dims[p] for p in perm], g.exponent(x), g.dtype(x))
        g.add_node(name, "Transpose", [x], [y], perm=list(perm), quant_type="S8")
        return y

    def output(self, x):
        self.g.outputs.append(x)
        return x


def make_lut(fn, in_exp, out_exp):
    """Closed form of the exporter's 8-bit tables: entry i is fn at real input (i - 128) * 2^in_exp,
    divided by 2^out_exp, rounded to nearest and clipped to int8."""
    x = (np.arange(256, dtype=np.float64) - 128.0) * (2.0 ** in_exp)
    y = np.asarray(fn(x), dtype=np.float64) / (2.0 ** out_exp)
    return np.clip(np.rint(y), -128, 127).astype(np.int8)


def silu(x):
    with np.errstate(over="ignore"):
        return x / (1.0 + np.exp(-x))


def hardswish(x):
    return x * np.clip(x + 3.0, 0.0, 6.0) / 6.0


def relu6(x):
    return np.clip(x, 0.0, 6.0)


# ------------------------------------------------------------------------------------------------
# The five benchmark configurations
# ------------------------------------------------------------------------------------------------
def config1_single_conv(seed=0xE5D1):
    """int8 Conv2D 1x56x56x64 -> 64, 3x3, s1, p1, per-tensor exponents in -7 / w -8 / out -6, bias, ReLU."""
    g = GraphSpec("config1_single_conv")
    b = Builder(g, seed, per_channel=False, w_exp_range=(-8, -8))
    x = b.input("input", [1, 56, 56, 64], -7)
    y = b.conv(x, 64, k=3, stride=1, relu=True, out_exp=-6, name="conv")
    b.output(y)
    return g


def config2_mbv2_block(seed=0xE5D2):
    """MobileNetV2 inverted residual, 56x56x24: 1x1 -> 144, ReLU6 as Clip, dw 3x3 s1, 1x1 -> 24, residual Add."""
    g = GraphSpec("config2_mbv2_block")
    b = Builder(g, seed, per_channel=True)
    x = b.input("input", [1, 56, 56, 24], -5)
    e = b.conv(x, 144, k=1, name="expand")
    six = min(127, int(round(6.0 / 2.0 ** g.exponent(e)))) if g.exponent(e) < 0 else 6
    e = b.clip(e, 0, max(1, six), name="relu6_a")
    d = b.conv(e, 144, k=3, depthwise=True, name="dw")
    six = min(127, int(round(6.0 / 2.0 ** g.exponent(d)))) if g.exponent(d) < 0 else 6
    d = b.clip(d, 0, max(1, six), name="relu6_b")
    p = b.conv(d, 24, k=1, name="project")
    y = b.add(x, p, name="residual")
    b.output(y)
    return g


MBV2_TABLE = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]


def config3_mobilenetv2(seed=0xE5D3, resolution=224, num_classes=1000, width=1.0, relabel_residual=False):
    """MobileNetV2-1.0 as ESP-DL runs it: ReLU fused into Conv (ReLU6 was replaced by ReLU before
    quantization), project convs Linear, residual Adds, GlobalAveragePool, Flatten, Gemm head.
    relabel_residual: as in the exported files of the reference, some residual operands pass through a
    RequantizeLinear (with its scale as a second, constant input) to an exponent that is NOT the project
    convolution's; the Add sums the stored integers whatever the exponents say."""
    g = GraphSpec("config3_mobilenetv2_%d" % resolution)
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, resolution, resolution, 3], -6)
    x = b.conv(x, int(32 * width), k=3, stride=2, relu=True, name="stem")
    cin = int(32 * width)
    blk = 0
    for t, c, n, s in MBV2_TABLE:
        c = int(c * width)
        for i in range(n):
            stride = s if i == 0 else 1
            blk += 1
            skip = x
            h = x
            if t != 1:
                h = b.conv(h, cin * t, k=1, relu=True, name="b%d_expand" % blk)
            h = b.conv(h, cin * t, k=3, stride=stride, depthwise=True, relu=True, name="b%d_dw" % blk)
            h = b.conv(h, c, k=1, relu=False, name="b%d_project" % blk)
            if stride == 1 and cin == c:
                if relabel_residual and blk % 2 == 0:
                    # exponent one or two off the project output's, never equal to it
                    e = g.exponent(h) + (1 if blk % 4 == 0 else -2)
                    if e == g.exponent(skip):
                        e += 1
                    skip = b.requantize(skip, e, name="b%d_skip_requant" % blk, with_scale_input=True)
                    y = "b%d_add_out" % blk
                    g.add_value(y, g.shape(h), g.exponent(h))
                    g.add_node("b%d_add" % blk, "Add", [skip, h], [y], quant_type="S8")
                    h = y
                else:
                    h = b.add(skip, h, name="b%d_add" % blk)
            x = h
            cin = c
    x = b.conv(x, int(1280 * max(1.0, width)), k=1, relu=True, name="head_conv")
    x = b.global_avg_pool(x, name="gap")
    x = b.flatten(x, name="flatten")
    x = b.gemm(x, num_classes, name="classifier")
    b.output(x)
    return g


def c3k2_like(b, x, c_out, name):
    """YOLO11-style C3k2 / C2f block: 1x1 conv, Split into two halves, a bottleneck (two 3x3 convs with
    SiLU tables and a residual Add) on the second half, Concat of both halves and the bottleneck output,
    1x1 fuse."""
    h = b.conv(x, c_out, k=1, name=name + "_cv1")
    h = b.lut(h, silu, "Swish", name=name + "_cv1_act")
    a, c = b.split(h, [c_out // 2, c_out // 2], name=name + "_split")
    m = b.conv(c, c_out // 2, k=3, name=name + "_m1")
    m = b.lut(m, silu, "Swish", name=name + "_m1_act")
    m = b.conv(m, c_out // 2, k=3, name=name + "_m2")
    m = b.lut(m, silu, "Swish", name=name + "_m2_act")
    m = b.add(c, m, name=name + "_add")
    cat = b.concat([a, c, m], name=name + "_cat")
    y = b.conv(cat, c_out, k=1, name=name + "_cv2")
    return b.lut(y, silu, "Swish", name=name + "_cv2_act")


def sppf_like(b, x, c_out, name):
    """SPPF: 1x1 reduce, three chained 5x5 stride-1 max pools, Concat of all four, 1x1 fuse."""
    c = b.g.shape(x)[3] // 2
    h = b.conv(x, c, k=1, name=name + "_cv1")
    h = b.lut(h, silu, "Swish", name=name + "_cv1_act")
    m1 = b.max_pool(h, 5, name=name + "_m1")
    m2 = b.max_pool(m1, 5, name=name + "_m2")
    m3 = b.max_pool(m2, 5, name=name + "_m3")
    cat = b.concat([h, m1, m2, m3], name=name + "_cat")
    y = b.conv(cat, c_out, k=1, name=name + "_cv2")
    return b.lut(y, silu, "Swish", name=name + "_cv2_act")


def config4_yolo_style(seed=0xE5D4, resolution=640):
    """YOLO11n-style detector trunk: int8 Conv backbone with SiLU as 8-bit LUT after every conv
    (conv -> LUT pairs, as in the exported YOLO11n), strided 3x3 downsampling, bottleneck blocks
    (Split -> bottleneck with residual Add -> Concat), SPPF (chained 5x5 max pools + Concat), an FPN
    top-down path (nearest Resize x2 + Concat with the skip), an NCHW Transpose of one class output,
    and an int16 detection head (int16 weights and activations, int64 bias).  Channel widths follow
    YOLO11n (16-32-64-128-256)."""
    g = GraphSpec("config4_yolo_style_%d" % resolution)
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, resolution, resolution, 3], -6)

    def cbs(x, c, k, s, name):
        y = b.conv(x, c, k=k, stride=s, name=name)
        return b.lut(y, silu, "Swish", name=name + "_act")

    x = cbs(x, 16, 3, 2, "p1")     # 320
    x = cbs(x, 32, 3, 2, "p2")     # 160
    x = c3k2_like(b, x, 64, "c2")
    x = cbs(x, 64, 3, 2, "p3")     # 80
    x = c3k2_like(b, x, 128, "c3")
    p3 = x
    x = cbs(x, 128, 3, 2, "p4")    # 40
    x = c3k2_like(b, x, 128, "c4")
    p4 = x
    x = cbs(x, 256, 3, 2, "p5")    # 20
    x = c3k2_like(b, x, 256, "c5")
    p5 = sppf_like(b, x, 256, "sppf")
    # FPN top-down: upsample, concatenate with the skip, fuse
    up = b.resize_nearest(p5, 2, name="up5")
    p4 = c3k2_like(b, b.concat([up, p4], name="fpn4_join"), 128, "fpn4")
    up = b.resize_nearest(p4, 2, name="up4")
    p3 = c3k2_like(b, b.concat([up, p3], name="fpn3_join"), 64, "fpn3")
    # detection head per scale: int8 3x3 conv + SiLU, then int16 box branch (requantize to int16,
    # int16 3x3 conv, SiLU through a 2049-entry int16 table, int16 1x1 conv) and an int8 class branch
    for i, (p, c) in enumerate(((p3, 64), (p4, 64), (p5, 64))):
        h = cbs(p, c, 3, 1, "head%d_cv" % i)
        h16 = "head%d_s16_in" % i
        g.add_value(h16, g.shape(h), g.exponent(h) - 8, INT16)
        g.add_node("head%d_to_s16" % i, "RequantizeLinear", [h], [h16], quant_type="S16")
        box = b.conv(h16, c, k=3, s16=True, name="head%d_box1" % i)
        box = b.lut_s16(box, silu, name="head%d_box1_silu" % i)
        box = b.conv(box, 64, k=1, s16=True, name="head%d_box2" % i)
        b.output(box)
        cls = cbs(h, 80, 1, 1, "head%d_cls1" % i)
        cls = b.conv(cls, 80, k=1, name="head%d_cls2" % i)
        if i == 2:  # one output in the NCHW layout detection post-processing reads
            cls = b.transpose(cls, (0, 3, 1, 2), name="head%d_cls_nchw" % i)
        b.output(cls)
    return g


def config5_ocr_style(seed=0xE5D5):
    """PP-OCR-style text-line recognizer on 48x320x3 crops: conv backbone (3x3 and depthwise-separable
    stages, hardswish tables) down to a 1x40x120 sequence, two int8 Gemm/MatMul layers
    120 -> 480 -> 120 with LUT activation, and a 120 -> 6625 int8 Gemm classifier."""
    g = GraphSpec("config5_ocr_style")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 48, 320, 3], -6)

    def cbh(x, c, k, s, name, depthwise=False):
        y = b.conv(x, c, k=k, stride=s, depthwise=depthwise, name=name)
        return b.lut(y, hardswish, "HardSwish", name=name + "_act")

    x = cbh(x, 16, 3, (2, 2), "stem")                  # 24 x 160
    for i, (c, s) in enumerate(((32, (2, 2)), (64, (2, 2)), (120, (2, 1)), (120, (3, 1)))):
        x = cbh(x, None, 3, s, "s%d_dw" % i, depthwise=True)
        x = cbh(x, c, 1, 1, "s%d_pw" % i)
    # now [1, 1, 40, 120]: a sequence of 40 steps of 120 features
    _, h, w, c = g.shape(x)
    assert (h, w, c) == (1, 40, 120), (h, w, c)
    seq = "sequence"
    g.add_value(seq, [1, 40, 120], g.exponent(x))
    g.add_node("to_sequence", "Squeeze", [x], [seq], axes=[1], quant_type="S8")
    y = b.gemm(seq, 480, name="fc1")
    y = b.lut(y, hardswish, "HardSwish", name="fc1_act")
    y = b.gemm(y, 120, name="fc2", matmul=True)
    y = b.lut(y, hardswish, "HardSwish", name="fc2_act")
    y = b.gemm(y, 6625, name="classifier")
    b.output(y)
    return g


CONFIGS = {
    1: config1_single_conv,
    2: config2_mbv2_block,
    3: config3_mobilenetv2,
    4: config4_yolo_style,
    5: config5_ocr_style,
}


def gated_block(seed=0xE5D6):
    """Conv blocks with x * sigmoid(x) written as Sigmoid (8-bit LUT) + Mul, a squeeze-and-excitation
    gate (GlobalAveragePool -> 1x1 Conv -> Sigmoid LUT -> Mul broadcast over H x W) and a residual Add:
    the operator mix of the reference's exported streaming / SE models."""
    g = GraphSpec("gated_block")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 20, 20, 32], -5)
    h = b.conv(x, 64, k=3, name="c1")
    s = b.lut(h, lambda v: 1.0 / (1.0 + np.exp(-v)), "Sigmoid", out_exp=-7, name="c1_sig")
    h = b.mul(h, s, name="c1_gate")                      # same shape
    sq = b.global_avg_pool(h, name="se_pool")
    sq = b.conv(sq, 64, k=1, name="se_fc")
    sq = b.lut(sq, lambda v: 1.0 / (1.0 + np.exp(-v)), "Sigmoid", out_exp=-7, name="se_sig")
    h = b.mul(h, sq, name="se_scale")                    # [1,20,20,64] * [1,1,1,64]
    y = b.conv(h, 32, k=1, name="c2")
    y = b.add(x, y, name="res")
    b.output(y)
    # transposed convolution as exported: InsertZeros, then a Conv whose padding restores 2x the size
    up = b.conv(b.insert_zeros(h, 2, name="up_zeros"), 16, k=2, pad=(1, 1, 1, 1), name="up_conv")
    b.output(up)
    # detection-style score head: two single-channel Conv -> Sigmoid branches multiplied together (each
    # Conv's only reader is its LUT, and each LUT's only reader is the Mul)
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    p = b.lut(b.conv(h, 1, k=1, name="score_cls"), sig, "Sigmoid", out_exp=-7, name="score_cls_sig")
    q = b.lut(b.conv(h, 1, k=5, name="score_obj"), sig, "Sigmoid", out_exp=-7, name="score_obj_sig")
    b.output(b.mul(p, q, name="score"))
    return g


def channel_slices(seed=0xE5E7):
    """Splits and Concats along channels in every combination a model has to tell apart when it leaves Split
    outputs inside the Split's input and lets Convs write into Concat outputs: pieces of 16 / 20 / 12
    channels (rows that are not multiples of 16 bytes), a piece read by a module that takes no channel
    pitch (Relu), a residual Add on a piece, a Concat of all pieces of a Split plus more (the C2f pattern),
    one tensor twice in a Concat, one tensor in two Concats, a Concat input that is a graph output, a Concat
    with the graph input, a strided 3x3 Conv on a piece and a depthwise Conv (no pitches) on another, a
    RequantizeLinear and a Resize that write their places in a Concat."""
    g = GraphSpec("channel_slices")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 14, 18, 24], -5)
    e = -4
    h = b.conv(x, 48, k=1, out_exp=e, name="s1_cv1")
    a, c, d = b.split(h, [16, 20, 12], name="s1_split")
    m = b.conv(c, 20, k=3, out_exp=e, relu=True, name="s1_m1")
    m = b.conv(m, 20, k=3, out_exp=e, name="s1_m2")
    m = b.add(c, m, name="s1_add")
    r = b.relu(d, name="s1_relu")                       # d must stay dense
    cat1 = b.concat([a, c, m, r], name="s1_cat")        # 16 + 20 + 20 + 12 = 68
    h2 = b.conv(cat1, 32, k=1, out_exp=e, name="s2_cv1")
    p, q = b.split(h2, [16, 16], name="s2_split")
    m2 = b.conv(q, 16, k=3, out_exp=e, name="s2_m")
    cat2 = b.concat([p, q, m2], name="s2_cat")          # h2 itself moves into this one
    y = b.conv(cat2, 8, k=1, out_exp=e, name="s3_y")
    cat3 = b.concat([y, y], name="s3_twice")
    z = b.conv(cat3, 24, k=3, out_exp=-5, name="s3_z")
    cat4 = b.concat([z, x], name="s4_with_input")       # z in place, the graph input copied
    out1 = b.conv(cat4, 16, k=1, out_exp=e, name="s4_out")
    b.output(out1)
    cat5 = b.concat([out1, y], name="s5_cat")           # out1 is a graph output: copied; y read with a pitch
    t, u = b.split(cat5, [8, 16], name="s5_split")
    t2 = b.conv(t, 8, k=3, stride=2, out_exp=e, name="s5_strided")
    u2 = b.conv(u, 16, k=3, stride=2, depthwise=True, out_exp=e, name="s5_dw")
    b.output(b.concat([t2, u2], name="s5_out"))
    # a Concat input at a finer exponent (requantized straight into its place), an upsampled one (the Resize
    # writes its place, reading a tensor that itself lives in another Concat) and a graph output (copied)
    fine = b.conv(out1, 16, k=1, out_exp=e - 1, name="s6_fine")
    up = b.resize_nearest(t2, 2, name="s6_up")
    cat6 = b.concat([fine, up, out1], name="s6_cat")    # 16 + 8 + 16 = 40
    b.output(b.conv(cat6, 8, k=1, out_exp=e, name="s6_out"))
    return g


def activation_modules(seed=0xE5E0):
    """The activation operators as graph nodes of their own rather than fused into a Conv: Conv (Linear) ->
    PRelu with a per-channel int8 slope -> Conv (Linear) -> standalone Relu -> Conv -> PRelu whose result
    is requantized to another exponent -> Add with the Relu branch.  This is how the reference's face /
    landmark models carry PReLU (esp-dl/dl/module/include/dl_module_prelu.hpp:109-121, dl_module_relu.hpp:65-93)."""
    g = GraphSpec("activation_modules")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 18, 22, 16], -5)
    h = b.conv(x, 48, k=3, name="c1")
    h = b.prelu(h, name="c1_prelu")
    h = b.conv(h, 32, k=1, name="c2")
    r = b.relu(h, name="c2_relu")
    h = b.conv(r, 32, k=3, depthwise=True, name="c3")
    h = b.prelu(h, name="c3_prelu", alpha_exp=-6, out_exp=g.exponent(h) + 1)
    r2 = b.requantize(r, g.exponent(h), name="r_align")
    y = b.add(r2, h, name="join")
    b.output(y)
    return g


def pooled_embedding(seed=0xE5D7):
    """Conv -> AveragePool -> Conv -> ReduceMean over H x W (axes as an initializer operand) -> Transpose to
    N,C,1,1 -> Reshape [1,-1] (shape as an initializer operand) -> Gemm: the tail of the reference's exported
    re-identification / embedding models."""
    g = GraphSpec("pooled_embedding")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 24, 12, 16], -5)
    h = b.conv(x, 32, k=3, relu=True, name="c1")
    h = b.avg_pool(h, 2, stride=2, name="pool")
    h = b.conv(h, 128, k=1, relu=True, name="c2")
    r = b.conv(h, 128, k=1, out_exp=g.exponent(h), name="c3")
    h = b.add(h, r, out_exp=g.exponent(h) - 1, name="res")   # the Add's result carries its own exponent
    h = b.reduce_mean(h, [1, 2], keepdims=True, name="mean")
    h = b.transpose(h, [0, 3, 1, 2], name="to_nchw")
    h = b.reshape(h, [1, -1], name="view")
    y = b.gemm(h, 64, relu=True, name="fc")
    b.output(y)
    return g


def attention_block(seed=0xE5D8, hw=10, heads=2, key_dim=16, head_dim=32):
    """The position-sensitive attention block of the reference's exported YOLO11n graphs: a 1x1 Conv makes
    q, k and v, Reshape / Split / Transpose bring them to [1, heads, ., hw*hw], q^T x k is scaled (Mul by a
    constant), Softmax leaves a float32 tensor that QuantizeLinear turns back into int8, v x attn^T is
    reshaped to the feature map, a depthwise positional Conv of v is added and a 1x1 Conv projects."""
    g = GraphSpec("attention_block")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    c = heads * head_dim
    per_head = 2 * key_dim + head_dim
    n = hw * hw
    x = b.input("input", [1, hw, hw, c], -4)
    qkv = b.conv(x, heads * per_head, k=1, name="qkv")                  # [1, hw, hw, heads*per_head]
    qkv = b.transpose(qkv, [0, 3, 1, 2], name="qkv_nchw")               # [1, heads*per_head, hw, hw]
    qkv = b.reshape(qkv, [1, heads, per_head, n], name="qkv_heads")     # [1, heads, per_head, n]
    q, k, v = b.split(qkv, [key_dim, key_dim, head_dim], axis=2, name="qkv_split")
    qt = b.transpose(q, [0, 1, 3, 2], name="q_t")                        # [1, heads, n, key_dim]
    attn = b.matmul_act(qt, k, name="qk")                                # [1, heads, n, n]
    g.add_init("attn_scale", [1], INT8, [91], [-9])                      # ~ key_dim ** -0.5 at exponent -9
    y = "attn_scaled_out"
    g.add_value(y, g.shape(attn), -3)
    g.add_node("attn_scaled", "Mul", [attn, "attn_scale"], [y], quant_type="S8")
    attn = b.quantize(b.softmax(y, axis=-1, name="attn_softmax"), -8, name="attn_q")
    attn_t = b.transpose(attn, [0, 1, 3, 2], name="attn_t")              # [1, heads, n, n]
    o = b.matmul_act(v, attn_t, out_exp=g.exponent(v), name="av")                               # [1, heads, head_dim, n]
    o = b.reshape(o, [1, c, hw, hw], name="o_map")
    o = b.transpose(o, [0, 2, 3, 1], name="o_nhwc")                      # [1, hw, hw, c]
    vmap = b.transpose(b.reshape(v, [1, c, hw, hw], name="v_map"), [0, 2, 3, 1], name="v_nhwc")
    pe = b.conv(vmap, c, k=3, depthwise=True, name="pe")
    o = b.add(o, pe, name="o_pe")
    b.output(b.conv(o, c, k=1, name="proj"))
    return g


def centered_ratio(seed=0xE5DA):
    """int8 Sub and Div in all of the reference's forms: features minus their spatial mean (broadcast Sub), the
    result over a one-element constant (divisor table), over a second feature map (element by element, zeros
    from its ReLU included) and a one-element constant over that map (dividend table)."""
    g = GraphSpec("centered_ratio")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 14, 14, 16], -5)
    f = b.conv(x, 32, k=3, name="features")
    m = b.reduce_mean(f, [1, 2], out_exp=g.exponent(f), name="spatial_mean")
    ctr = "centered_out"
    g.add_value(ctr, g.shape(f), g.exponent(f))
    g.add_node("centered", "Sub", [f, m], [ctr], quant_type="S8")
    g.add_init("three", [1], INT8, [3], [0])
    third = "third_out"
    g.add_value(third, g.shape(f), g.exponent(ctr) - 1)
    g.add_node("third", "Div", [ctr, "three"], [third], quant_type="S8")
    d = b.conv(x, 32, k=3, relu=True, name="denominator")
    ratio = "ratio_out"
    g.add_value(ratio, g.shape(f), -4)
    g.add_node("ratio", "Div", [third, d], [ratio], quant_type="S8")
    g.add_init("numerator", [1], INT8, [100], [-6])
    inv = "inverse_out"
    g.add_value(inv, g.shape(f), -4)
    g.add_node("inverse", "Div", ["numerator", d], [inv], quant_type="S8")
    g.outputs.append(ratio)
    g.outputs.append(inv)
    return g


def activation_chain(seed=0xE5DB, s16=False):
    """Every activation module that the reference evaluates in float32 per element, without tables in the file:
    Conv -> Sigmoid / Tanh / HardSwish / Elu / LeakyRelu / Swish / HardSigmoid / Neg branches summed pairwise,
    then Exp, Sqrt and Log on tensors whose sign suits them, and an Identity that changes the exponent."""
    g = GraphSpec("activation_chain_s16" if s16 else "activation_chain")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    qt, dt = ("S16", INT16) if s16 else ("S8", INT8)
    bits = 15 if s16 else 7
    x = b.input("input", [1, 10, 10, 16], -5)
    f = b.conv(x, 32, k=3, name="features")              # spans roughly [-4, 4) at its exponent
    fe = g.exponent(f)
    if s16:
        f16 = "features_s16"
        g.add_value(f16, g.shape(f), fe - 8, INT16)
        g.add_node("to_s16", "RequantizeLinear", [f], [f16], quant_type="S16")
        f = b.conv(f16, 32, k=1, s16=True, out_exp=fe - 8, name="mixed")   # int16 values, not multiples of 256
        fe = fe - 8
    span = fe + bits                                      # the input covers [-2^span, 2^span)

    def unary(op, src, out_exp, name, **attrs):
        y = name + "_out"
        g.add_value(y, g.shape(src), out_exp, dt)
        g.add_node(name, op, [src], [y], quant_type=qt, **attrs)
        return y

    outs = [unary("Sigmoid", f, -bits, "sigmoid"),
            unary("Tanh", f, -bits, "tanh"),
            unary("HardSwish", f, span - bits, "hard_swish"),
            unary("Elu", f, span - bits, "elu", alpha=0.75),
            unary("LeakyRelu", f, span - bits, "leaky_relu", alpha=0.1),
            unary("Swish", f, span - bits, "swish"),
            unary("HardSigmoid", f, -bits, "hard_sigmoid", alpha=0.25, beta=0.5),
            unary("HardSigmoid", f, -bits, "hard_sigmoid_default"),
            unary("Neg", f, fe, "neg")]
    small = unary("Identity", f, fe + 2, "quarter")       # a requantize by assign
    outs.append(unary("Exp", outs[1], 2 - bits, "exp"))   # exp(tanh) in (0.36, 2.72)
    pos = unary("Sigmoid", small, -bits, "gate")
    outs.append(unary("Sqrt", pos, -bits, "sqrt"))
    outs.append(unary("Log", pos, 3 - bits, "log"))       # log(sigmoid) in (-4.1, 0)
    g.outputs.extend(outs)
    return g


def padded_convs(seed=0xE5DC):
    """Explicit Pad nodes in the three modes of the reference in front of unpadded convolutions: reflect (H, W by
    2), edge (1 and 2, unequal sides) and constant with a non-zero value (also along channels)."""
    g = GraphSpec("padded_convs")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 12, 12, 16], -5)

    def pad(src, pads, mode, name, value=None):
        dims = g.shape(src)
        nd = len(dims)
        y = name + "_out"
        g.add_init(name + ".pads", [2 * nd], INT64, pads, [0])
        ins = [src, name + ".pads"]
        if value is not None:
            g.add_init(name + ".value", [1], INT8, [value], [g.exponent(src)])
            ins.append(name + ".value")
        g.add_value(y, [dims[i] + pads[i] + pads[i + nd] for i in range(nd)], g.exponent(src))
        g.add_node(name, "Pad", ins, [y], mode=mode, quant_type="S8")
        return y

    h = pad(x, [0, 2, 2, 0, 0, 2, 2, 0], "reflect", "mirror")
    h = b.conv(h, 32, k=5, pad=(0, 0, 0, 0), relu=True, name="c1")
    h = pad(h, [0, 1, 2, 0, 0, 2, 1, 0], "edge", "border")
    h = b.conv(h, 32, k=3, pad=(0, 0, 0, 0), depthwise=True, name="dw")
    h = pad(h, [0, 1, 1, 3, 0, 1, 1, 5], "constant", "frame", value=-3)
    b.output(b.conv(h, 24, k=3, pad=(0, 0, 0, 0), name="c2"))
    return g


def reduce_heads(seed=0xE5DD, s16=False):
    """ReduceMax over the image, ReduceMin over channels, ReduceSum and ReduceSumSquare over the image and ReduceL1
    over channels (coarser output exponents for the sums) on one feature map, int8 or int16."""
    g = GraphSpec("reduce_heads_s16" if s16 else "reduce_heads")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    qt, dt = ("S16", INT16) if s16 else ("S8", INT8)
    x = b.input("input", [1, 10, 12, 16], -5)
    f = b.conv(x, 32, k=3, name="features")
    if s16:
        f16 = "features_s16"
        g.add_value(f16, g.shape(f), g.exponent(f) - 8, INT16)
        g.add_node("to_s16", "RequantizeLinear", [f], [f16], quant_type="S16")
        f = b.conv(f16, 32, k=1, s16=True, out_exp=g.exponent(f16), name="mixed")
    n, h, w, c = g.shape(f)

    def reduce(op, axes, out_shape, out_exp, name, keepdims=1):
        y = name + "_out"
        g.add_init(name + ".axes", [len(axes)], INT64, axes, [0])
        g.add_value(y, out_shape, out_exp, dt)
        g.add_node(name, op, [f, name + ".axes"], [y], keepdims=keepdims, noop_with_empty_axes=0, quant_type=qt)
        g.outputs.append(y)

    reduce("ReduceMax", [1, 2], [1, 1, 1, c], g.exponent(f), "image_max")
    reduce("ReduceMin", [-1], [1, h, w], g.exponent(f), "channel_min", keepdims=0)
    reduce("ReduceSum", [1, 2], [1, 1, 1, c], g.exponent(f) + 5, "image_sum")
    reduce("ReduceL1", [-1], [1, h, w, 1], g.exponent(f) + 4, "channel_l1")
    reduce("ReduceSumSquare", [1, 2], [1, 1, 1, c], 2 * g.exponent(f) + (20 if s16 else 12), "image_energy")
    return g


def pixel_shuffle(seed=0xE5DE):
    """SpaceToDepth in front of a convolution (a stride-2 stem without losing pixels), then DepthToSpace in both
    channel orders as sub-pixel upsampling heads."""
    g = GraphSpec("pixel_shuffle")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 12, 16, 8], -5)

    def shuffle(op, src, out_shape, name, **attrs):
        y = name + "_out"
        g.add_value(y, out_shape, g.exponent(src))
        g.add_node(name, op, [src], [y], quant_type="S8", **attrs)
        return y

    s = shuffle("SpaceToDepth", x, [1, 6, 8, 32], "fold", blocksize=2)
    f = b.conv(s, 48, k=3, relu=True, name="features")
    up_crd = shuffle("DepthToSpace", f, [1, 12, 16, 12], "unfold_crd", blocksize=2, mode="CRD")
    up_dcr = shuffle("DepthToSpace", f, [1, 12, 16, 12], "unfold_dcr", blocksize=2, mode="DCR")
    b.output(b.conv(up_crd, 8, k=3, name="head_crd"))
    b.output(b.conv(up_dcr, 8, k=3, name="head_dcr"))
    return g


def gathered_rows(seed=0xE5DF):
    """Gather with constant indices along three axes: one time step of a sequence (the usual exported form), a
    reordering with repeats along channels, and a 2-D index tensor along the width."""
    g = GraphSpec("gathered_rows")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 8, 10, 16], -5)
    f = b.conv(x, 24, k=3, name="features")

    def gather(src, indices, idx_shape, axis, out_shape, name):
        y = name + "_out"
        g.add_init(name + ".indices", idx_shape, INT64, indices, [0])
        g.add_value(y, out_shape, g.exponent(src))
        g.add_node(name, "Gather", [src, name + ".indices"], [y], axis=axis, quant_type="S8")
        g.outputs.append(y)
        return y

    gather(f, [7], [1], 1, [1, 1, 10, 24], "last_row")
    gather(f, [5, 6, 7, 0, 0, 23, 1, 2, 3], [9], -1, [1, 8, 10, 9], "channels")
    gather(f, [0, 9, 4, 5, 6, 2], [2, 3], 2, [1, 8, 2, 3, 24], "columns")
    return g


def int16_tail(seed=0xE5D9):
    """int8 Conv -> RequantizeLinear to int16 -> int16 Conv -> int16 table (SiLU) -> int16 Add (residual) ->
    int16 Mul by a constant -> int16 AveragePool -> int16 ReduceMean -> int16 Gemm: the operator mix of the
    reference's int16 text recognizer."""
    g = GraphSpec("int16_tail")
    b = Builder(g, seed, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 12, 16, 16], -5)
    h = b.conv(x, 32, k=3, relu=True, name="c1")
    h16 = "to_s16_out"
    g.add_value(h16, g.shape(h), g.exponent(h) - 8, INT16)
    g.add_node("to_s16", "RequantizeLinear", [h], [h16], quant_type="S16")
    c2 = b.conv(h16, 32, k=1, s16=True, out_exp=g.exponent(h16) + 3, name="c2")
    act = b.lut_s16(c2, silu, name="c2_silu")
    res = "res_out"
    g.add_value(res, g.shape(act), g.exponent(act), INT16)
    g.add_node("res", "Add", [act, c2], [res], quant_type="S16")
    g.add_init("gain", [1], INT16, [23170], [-15])       # ~ 0.707 at exponent -15
    sc = "scaled_out"
    g.add_value(sc, g.shape(res), g.exponent(res), INT16)
    g.add_node("scaled", "Mul", [res, "gain"], [sc], quant_type="S16")
    ap = "pool_out"
    g.add_value(ap, [1, 6, 8, 32], g.exponent(sc), INT16)
    g.add_node("pool", "AveragePool", [sc], [ap], kernel_shape=[2, 2], strides=[2, 2], pads=[0, 0, 0, 0], quant_type="S16")
    g.add_init("mean.axes", [1], INT64, [1], [0])
    mn = "mean_out"
    g.add_value(mn, [1, 1, 8, 32], g.exponent(ap) - 1, INT16)
    g.add_node("mean", "ReduceMean", [ap, "mean.axes"], [mn], keepdims=1, noop_with_empty_axes=0, quant_type="S16")
    g.outputs.append(mn)
    return g
