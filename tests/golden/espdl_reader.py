"""Minimal reader for `.espdl` model containers (EDL2 header + FlatBuffers payload).

Used only to turn the reference's own fixture files (data, not code) into the small JSON
vectors kept beside this file.  It executes nothing from the file: it walks FlatBuffers
vtables by hand.  Container layout: esp-dl/fbs_loader/include/fbs_loader.hpp:41-49; schema
field numbers: esp-dl/fbs_loader/espdl.fbs:73-145.
"""
import struct

import numpy as np

# TensorDataType (espdl.fbs:24-39) -> numpy dtype
_DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32,
           7: np.int64, 9: np.bool_, 11: np.float64, 12: np.uint32, 13: np.uint64}


class _Buf:
    def __init__(self, data):
        self.d = data

    def u8(self, p):
        return self.d[p]

    def u16(self, p):
        return struct.unpack_from("<H", self.d, p)[0]

    def u32(self, p):
        return struct.unpack_from("<I", self.d, p)[0]

    def i32(self, p):
        return struct.unpack_from("<i", self.d, p)[0]

    def i64(self, p):
        return struct.unpack_from("<q", self.d, p)[0]

    def f32(self, p):
        return struct.unpack_from("<f", self.d, p)[0]


class _Table:
    """One FlatBuffers table: resolves field number -> absolute position (or None)."""

    def __init__(self, buf, pos):
        self.b = buf
        self.pos = pos
        self.vt = pos - buf.i32(pos)
        self.vt_size = buf.u16(self.vt)

    def field(self, idx):
        off = 4 + 2 * idx
        if off >= self.vt_size:
            return None
        rel = self.b.u16(self.vt + off)
        return self.pos + rel if rel else None

    def indirect(self, idx):
        p = self.field(idx)
        return None if p is None else p + self.b.u32(p)

    def table(self, idx):
        p = self.indirect(idx)
        return None if p is None else _Table(self.b, p)

    def string(self, idx):
        p = self.indirect(idx)
        if p is None:
            return None
        n = self.b.u32(p)
        return bytes(self.b.d[p + 4:p + 4 + n]).decode("utf-8", "replace")

    def scalar_i32(self, idx, default=0):
        p = self.field(idx)
        return default if p is None else self.b.i32(p)

    def vector(self, idx):
        """(start position of element 0, length) or (None, 0)."""
        p = self.indirect(idx)
        if p is None:
            return None, 0
        return p + 4, self.b.u32(p)

    def vector_i64(self, idx):
        p, n = self.vector(idx)
        return [self.b.i64(p + 8 * i) for i in range(n)]

    def vector_tables(self, idx):
        p, n = self.vector(idx)
        out = []
        for i in range(n):
            e = p + 4 * i
            out.append(_Table(self.b, e + self.b.u32(e)))
        return out

    def vector_strings(self, idx):
        p, n = self.vector(idx)
        out = []
        for i in range(n):
            e = p + 4 * i
            s = e + self.b.u32(e)
            ln = self.b.u32(s)
            out.append(bytes(self.b.d[s + 4:s + 4 + ln]).decode("utf-8", "replace"))
        return out


def _tensor(t):
    dims = t.vector_i64(0)
    dtype = t.scalar_i32(1)
    name = t.string(6)
    doc = t.string(7)
    exps = t.vector_i64(13)
    data = None
    p, n = t.vector(8)  # raw_data: [AlignedBytes], 16 bytes each
    np_dtype = _DTYPES.get(dtype)
    count = int(np.prod(dims)) if dims else 1
    if p is not None and np_dtype is not None:
        raw = bytes(t.b.d[p:p + 16 * n])
        data = np.frombuffer(raw, dtype=np_dtype, count=count).reshape(dims if dims else ())
    elif np_dtype is not None:
        # small tensors may be written as typed arrays: 2 float_data, 3 int32_data, 5 int64_data
        field = {1: 2, 6: 3, 7: 5}.get(dtype)
        if field is not None:
            q, m = t.vector(field)
            if q is not None and m >= count:
                raw = bytes(t.b.d[q:q + np.dtype(np_dtype).itemsize * count])
                data = np.frombuffer(raw, dtype=np_dtype, count=count).reshape(dims if dims else ())
    return {"name": name, "dims": dims, "dtype": dtype, "doc": doc, "exponents": exps, "data": data}


def _attribute(a):
    name = a.string(0)
    atype = a.scalar_i32(3)
    val = None
    if atype == 1:  # FLOAT, struct inline
        p = a.field(4)
        val = None if p is None else a.b.f32(p)
    elif atype == 2:  # INT
        p = a.field(5)
        val = None if p is None else a.b.i64(p)
    elif atype == 3:  # STRING stored as [uint8]
        p, n = a.vector(6)
        val = bytes(a.b.d[p:p + n]).decode("utf-8", "replace") if p is not None else ""
    elif atype == 7:  # INTS
        val = a.vector_i64(11)
    elif atype == 6:  # FLOATS
        p, n = a.vector(10)
        val = [a.b.f32(p + 4 * i) for i in range(n)]
    return name, atype, val


def _value_info(v):
    """ValueInfo: 0 name, 1 value_info_type (TypeInfo: 0 union tag, 1 value -> TensorTypeAndShape:
    0 elem_type, 1 shape -> TensorShape.dim[] -> Dimension.value -> DimensionValue.dim_value), 3 exponents."""
    out = {"name": v.string(0), "exponents": v.vector_i64(3), "dtype": 0, "dims": []}
    p = v.field(1)
    ti = v.table(1)
    if p is None or ti is None:
        return out
    tag = ti.field(0)
    if tag is None or ti.b.u8(tag) != 1:
        return out
    tts = ti.table(1)
    if tts is None:
        return out
    out["dtype"] = tts.scalar_i32(0)
    shape = tts.table(1)
    if shape is not None:
        for dim in shape.vector_tables(0):
            dv = dim.table(0)
            p = None if dv is None else dv.field(1)
            out["dims"].append(int(dv.b.i64(p)) if p is not None else 1)
    return out


def read_espdl(path):
    """Parse one plain (unencrypted) EDL2 file into plain Python / numpy objects."""
    with open(path, "rb") as f:
        blob = f.read()
    if blob[:4] != b"EDL2":
        raise ValueError(f"{path}: not an EDL2 container (magic {blob[:4]!r})")
    mode, size, _pad = struct.unpack_from("<III", blob, 4)
    if mode != 0:
        raise ValueError(f"{path}: encrypted container (mode {mode}) is not supported")
    buf = _Buf(memoryview(blob)[16:16 + size])
    model = _Table(buf, buf.u32(0))
    graph = model.table(7)
    meta = {}
    for e in model.vector_tables(8):
        meta[e.string(0)] = e.string(1)
    nodes = []
    for n in graph.vector_tables(0):
        attrs = {}
        for a in n.vector_tables(5):
            nm, _t, v = _attribute(a)
            attrs[nm] = v
        nodes.append({"name": n.string(2), "op_type": n.string(3), "input": n.vector_strings(0),
                      "output": n.vector_strings(1), "attrs": attrs})
    return {
        "meta": meta,
        "nodes": nodes,
        "initializers": {t["name"]: t for t in map(_tensor, graph.vector_tables(2))},
        "inputs": [_value_info(v) for v in graph.vector_tables(4)],
        "outputs": [_value_info(v) for v in graph.vector_tables(5)],
        "value_info": [_value_info(v) for v in graph.vector_tables(6)],
        "test_inputs": {t["name"]: t for t in map(_tensor, graph.vector_tables(8))},
        "test_outputs": {t["name"]: t for t in map(_tensor, graph.vector_tables(9))},
    }
