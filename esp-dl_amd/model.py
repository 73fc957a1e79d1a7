"""ctypes binding of include/espdl_model.h (lib/libespdl_dl.so): native graph + dl::Model handles."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libespdl_dl.so")

_lib = None


class EspdlModelError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EspdlModelError(f"{LIB_PATH} is missing: build it with `python esp-dl_amd/build.py`")
        # libespdl_dl.so links libespdl_hip.so through $ORIGIN
        from . import capi
        capi.torch_device_first()
        L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        vp, cp, i32, i64 = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int32, ctypes.c_int64
        pi32 = ctypes.POINTER(i32)
        L.espdl_graph_create.restype = vp
        L.espdl_graph_create.argtypes = [cp]
        L.espdl_graph_destroy.argtypes = [vp]
        L.espdl_graph_destroy.restype = None
        L.espdl_graph_add_initializer.argtypes = [vp, cp, pi32, i32, i32, vp, pi32, i32]
        L.espdl_graph_add_value_info.argtypes = [vp, cp, pi32, i32, i32, i32]
        L.espdl_graph_add_input.argtypes = [vp, cp]
        L.espdl_graph_add_output.argtypes = [vp, cp]
        L.espdl_graph_add_node.argtypes = [vp, cp, cp, ctypes.POINTER(cp), i32, ctypes.POINTER(cp), i32]
        L.espdl_graph_node_set_int.argtypes = [vp, cp, cp, i64]
        L.espdl_graph_node_set_float.argtypes = [vp, cp, cp, ctypes.c_float]
        L.espdl_graph_node_set_ints.argtypes = [vp, cp, cp, ctypes.POINTER(i64), i32]
        L.espdl_graph_node_set_string.argtypes = [vp, cp, cp, cp]
        L.espdl_graph_add_test_input.argtypes = [vp, cp, pi32, i32, i32, vp, i32]
        L.espdl_graph_add_test_output.argtypes = [vp, cp, pi32, i32, i32, vp, i32]
        L.espdl_model_create.restype = vp
        L.espdl_model_create.argtypes = [vp, i32, i32, vp, i32]
        L.espdl_model_destroy.argtypes = [vp]
        L.espdl_model_destroy.restype = None
        for name in ("run", "run_async", "synchronize", "enable_graph", "disable_graph", "test", "module_count"):
            getattr(L, "espdl_model_" + name).argtypes = [vp]
        L.espdl_model_profile.argtypes = [vp, i32, i32, ctypes.POINTER(cp), ctypes.POINTER(cp),
                                          ctypes.POINTER(ctypes.c_float), ctypes.POINTER(i64), ctypes.POINTER(i64)]
        L.espdl_model_print_profile.argtypes = [vp]
        L.espdl_model_print_profile.restype = None
        L.espdl_model_tensor_channel_pitch.argtypes = [vp, cp]
        L.espdl_model_tensor_device_ptr.restype = vp
        L.espdl_model_tensor_device_ptr.argtypes = [vp, cp]
        L.espdl_model_tensor_bytes.restype = i64
        L.espdl_model_tensor_bytes.argtypes = [vp, cp]
        L.espdl_model_tensor_shape.argtypes = [vp, cp, pi32, i32]
        L.espdl_model_tensor_exponent.argtypes = [vp, cp, pi32]
        L.espdl_model_set_input.argtypes = [vp, cp, vp, i64]
        L.espdl_model_get_tensor.argtypes = [vp, cp, vp, i64]
        L.espdl_model_device_bytes.restype = i64
        L.espdl_model_device_bytes.argtypes = [vp]
        L.espdl_graph_load_file.restype = vp
        L.espdl_graph_load_file.argtypes = [cp, i32]
        L.espdl_graph_load_memory.restype = vp
        L.espdl_graph_load_memory.argtypes = [vp, ctypes.c_int64, i32]
        L.espdl_graph_load_error.restype = cp
        for nm in ("input", "output"):
            getattr(L, "espdl_graph_%s_count" % nm).argtypes = [vp]
            getattr(L, "espdl_graph_%s_name" % nm).argtypes = [vp, i32]
            getattr(L, "espdl_graph_%s_name" % nm).restype = cp
        L.espdl_graph_initializer_bytes.restype = ctypes.c_int64
        L.espdl_graph_initializer_bytes.argtypes = [vp, cp, vp, ctypes.c_int64]
        L.espdl_graph_node_count.argtypes = [vp]
        L.espdl_graph_node_op_type.argtypes = [vp, i32]
        L.espdl_graph_node_op_type.restype = cp
        L.espdl_module_is_registered.argtypes = [cp]
        L.espdl_model_stream.restype = vp
        L.espdl_model_stream.argtypes = [vp]
        _lib = L
    return _lib


def _dims(d):
    return (ctypes.c_int32 * len(d))(*[int(v) for v in d]), len(d)


_NP_OF = {1: np.float32, 3: np.int8, 5: np.int16, 6: np.int32, 7: np.int64}


class Graph:
    """Native fbs::FbsModel built from a zoo.GraphSpec."""

    def __init__(self, name):
        self.h = lib().espdl_graph_create(name.encode())

    @classmethod
    def from_spec(cls, spec, test_input=None, test_outputs=None):
        L = lib()
        g = cls(spec.name)
        for name, (dims, dtype, data, exps) in spec.initializers.items():
            d, nd = _dims(dims)
            e, ne = _dims(exps)
            arr = np.ascontiguousarray(data, dtype=_NP_OF[dtype])
            rc = L.espdl_graph_add_initializer(g.h, name.encode(), d, nd, dtype, arr.ctypes.data_as(ctypes.c_void_p),
                                               e, ne)
            assert rc == 0, name
        for name, (dims, dtype, exp) in spec.value_info.items():
            d, nd = _dims(dims)
            assert L.espdl_graph_add_value_info(g.h, name.encode(), d, nd, dtype, exp) == 0
        for name in spec.inputs:
            L.espdl_graph_add_input(g.h, name.encode())
        for name in spec.outputs:
            L.espdl_graph_add_output(g.h, name.encode())
        for node in spec.nodes:
            ins = (ctypes.c_char_p * len(node["inputs"]))(*[s.encode() for s in node["inputs"]])
            outs = (ctypes.c_char_p * len(node["outputs"]))(*[s.encode() for s in node["outputs"]])
            nm = node["name"].encode()
            assert L.espdl_graph_add_node(g.h, nm, node["op_type"].encode(), ins, len(node["inputs"]), outs,
                                          len(node["outputs"])) == 0
            for key, val in node["attrs"].items():
                if isinstance(val, str):
                    L.espdl_graph_node_set_string(g.h, nm, key.encode(), val.encode())
                elif isinstance(val, (list, tuple)):
                    arr = (ctypes.c_int64 * len(val))(*[int(v) for v in val])
                    L.espdl_graph_node_set_ints(g.h, nm, key.encode(), arr, len(val))
                elif isinstance(val, float):
                    L.espdl_graph_node_set_float(g.h, nm, key.encode(), val)
                else:
                    L.espdl_graph_node_set_int(g.h, nm, key.encode(), int(val))
        if test_input is not None:
            for name, arr in test_input.items():
                _, dtype, exp = spec.value_info[name]
                d, nd = _dims(arr.shape)
                arr = np.ascontiguousarray(arr)
                L.espdl_graph_add_test_input(g.h, name.encode(), d, nd, dtype, arr.ctypes.data_as(ctypes.c_void_p), exp)
        if test_outputs is not None:
            for name, arr in test_outputs.items():
                _, dtype, exp = spec.value_info[name]
                d, nd = _dims(arr.shape)
                arr = np.ascontiguousarray(arr)
                L.espdl_graph_add_test_output(g.h, name.encode(), d, nd, dtype, arr.ctypes.data_as(ctypes.c_void_p),
                                              exp)
        return g

    @classmethod
    def from_file(cls, path, model_index=0):
        """Read an `.espdl` container with the native loader (no GPU needed)."""
        g = cls.__new__(cls)
        g.h = lib().espdl_graph_load_file(os.fsencode(path), model_index)
        if not g.h:
            raise EspdlModelError("%s: %s" % (path, lib().espdl_graph_load_error().decode("utf-8", "replace")))
        return g

    @classmethod
    def from_bytes(cls, blob, model_index=0):
        g = cls.__new__(cls)
        g.h = lib().espdl_graph_load_memory(blob, len(blob), model_index)
        if not g.h:
            raise EspdlModelError(lib().espdl_graph_load_error().decode("utf-8", "replace"))
        return g

    def initializer(self, name, dtype=np.int8):
        """Bytes of a constant tensor as the kernels will read it (flat array of dtype)."""
        n = lib().espdl_graph_initializer_bytes(self.h, name.encode(), None, 0)
        if n < 0:
            raise KeyError(name)
        out = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        lib().espdl_graph_initializer_bytes(self.h, name.encode(), out.ctypes.data_as(ctypes.c_void_p), n)
        return out

    def op_types(self):
        L = lib()
        return [L.espdl_graph_node_op_type(self.h, i).decode() for i in range(L.espdl_graph_node_count(self.h))]

    def input_names(self):
        L = lib()
        return [L.espdl_graph_input_name(self.h, i).decode() for i in range(L.espdl_graph_input_count(self.h))]

    def output_names(self):
        L = lib()
        return [L.espdl_graph_output_name(self.h, i).decode() for i in range(L.espdl_graph_output_count(self.h))]

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            _lib.espdl_graph_destroy(self.h)
            self.h = None


def is_registered(op_type):
    return bool(lib().espdl_module_is_registered(op_type.encode()))


class Model:
    """dl::Model handle.  `stream` is a raw hipStream_t value (e.g. torch.cuda.Stream().cuda_stream) or None."""

    def __init__(self, graph, batch, round_mode=0, stream=None, fuse_lut=True, fuse_blocks=True, fuse_add=True,
                 fuse_gap=True, channel_slices=True):
        self.graph = graph  # keep alive: the native model references it
        self.h = lib().espdl_model_create(graph.h, batch, round_mode, ctypes.c_void_p(stream) if stream else None,
                                          (1 if fuse_lut else 0) | (2 if fuse_blocks else 0) | (4 if fuse_add else 0) |
                                          (8 if fuse_gap else 0) | (16 if channel_slices else 0))
        if not self.h:
            raise EspdlModelError("espdl_model_create failed (see stderr)")
        self.batch = batch

    def close(self):
        if getattr(self, "h", None):
            lib().espdl_model_destroy(self.h)
            self.h = None

    def __del__(self):
        if _lib is not None:
            self.close()

    def run(self):
        if lib().espdl_model_run(self.h) != 0:
            raise EspdlModelError("run failed: a module rejected its launch or a HIP call failed (see stderr)")

    def run_async(self):
        if lib().espdl_model_run_async(self.h) != 0:
            raise EspdlModelError("run_async failed: a module rejected its launch (see stderr)")

    def synchronize(self):
        if lib().espdl_model_synchronize(self.h) != 0:
            raise EspdlModelError("the pass failed: a module rejected its launch or a HIP call failed (see stderr)")

    def enable_graph(self):
        return lib().espdl_model_enable_graph(self.h) == 0

    def disable_graph(self):
        lib().espdl_model_disable_graph(self.h)

    def test(self):
        return lib().espdl_model_test(self.h) == 0

    def channel_pitch(self, name):
        """Elements between consecutive positions of the last axis in device memory (the last dim when dense)."""
        return lib().espdl_model_tensor_channel_pitch(self.h, name.encode())

    def module_count(self):
        return lib().espdl_model_module_count(self.h)

    def stream(self):
        return lib().espdl_model_stream(self.h)

    def device_bytes(self):
        return lib().espdl_model_device_bytes(self.h)

    def shape(self, name):
        dims = (ctypes.c_int32 * 8)()
        r = lib().espdl_model_tensor_shape(self.h, name.encode(), dims, 8)
        if r < 0:
            raise KeyError(name)
        return [dims[i] for i in range(r)]

    def exponent(self, name):
        e = ctypes.c_int32()
        if lib().espdl_model_tensor_exponent(self.h, name.encode(), ctypes.byref(e)) != 0:
            raise KeyError(name)
        return e.value

    def set_input(self, name, array):
        array = np.ascontiguousarray(array)
        if lib().espdl_model_set_input(self.h, name.encode(), array.ctypes.data_as(ctypes.c_void_p), array.nbytes) != 0:
            raise EspdlModelError(f"set_input({name}) failed: wrong name or byte size")

    def get_tensor(self, name, dtype=np.int8):
        nbytes = lib().espdl_model_tensor_bytes(self.h, name.encode())
        if nbytes < 0:
            raise KeyError(name)
        shape = self.shape(name)
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes == nbytes, (name, out.nbytes, nbytes)
        if lib().espdl_model_get_tensor(self.h, name.encode(), out.ctypes.data_as(ctypes.c_void_p), nbytes) != 0:
            raise EspdlModelError(f"get_tensor({name}) failed")
        return out

    def profile(self, repeats=3):
        n = self.module_count()
        names = (ctypes.c_char_p * n)()
        types = (ctypes.c_char_p * n)()
        lat = (ctypes.c_float * n)()
        macs = (ctypes.c_int64 * n)()
        byts = (ctypes.c_int64 * n)()
        got = lib().espdl_model_profile(self.h, repeats, n, names, types, lat, macs, byts)
        return [{"name": names[i].decode(), "type": types[i].decode(), "latency_us": lat[i], "macs": macs[i],
                 "bytes": byts[i]} for i in range(min(n, got))]
