"""GGUF files from Python: a writer (numpy, for synthetic models and tests) and a reader that wraps the
library's parser (wd_gguf_* of the C ABI) and exposes tensors as zero-copy numpy views of the mapping.

Container layout written here (GGUF version 3, little endian): magic "GGUF", version u32, tensor count u64,
key/value count u64, the key/value pairs, the tensor directory (name, n_dims, dims u64 each, ggml type u32,
offset u64 relative to the data section), padding to `general.alignment`, then every tensor's bytes, each
padded to the alignment.
"""
import ctypes as C
import struct

import numpy as np

from . import capi

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}
_NP = {U8: np.uint8, I8: np.int8, U16: np.uint16, I16: np.int16, U32: np.uint32, I32: np.int32, F32: np.float32,
       BOOL: np.uint8, U64: np.uint64, I64: np.int64, F64: np.float64}


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STRING:
        return _s(v)
    if vtype == ARRAY:
        etype, items = v
        out = struct.pack("<IQ", etype, len(items))
        if etype == STRING:
            return out + b"".join(_s(i) for i in items)
        return out + np.asarray(items, dtype=_NP[etype]).tobytes()
    return struct.pack(_FMT[vtype], v)


def write_gguf(path, tensors, meta=(), alignment=32, version=3):
    """tensors: list of (name, dims in GGUF order, ggml type id, numpy array holding the raw bytes);
    meta: list of (key, value type, value) - arrays as (ARRAY, (element type, items))."""
    meta = list(meta)
    if alignment != 32:
        meta.append(("general.alignment", U32, alignment))
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(meta))
    for key, vtype, v in meta:
        head += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    pad = lambda n: (-n) % alignment
    offsets, at = [], 0
    for _, _, _, data in tensors:
        offsets.append(at)
        at += data.nbytes + pad(data.nbytes)
    for (name, dims, ttype, _), off in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", ttype, off)
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * pad(len(head)))
        for _, _, _, data in tensors:
            f.write(np.ascontiguousarray(data).tobytes())
            f.write(b"\0" * pad(data.nbytes))
    return len(head) + pad(len(head))


def layer_tensors(L, il, fused_gate_up=False):
    """The tensor list of one MoE layer (a synth.make_layer() dict) under the names the model files use."""
    H, F, E = L["hidden"], L["expert_ffn"], L["n_experts"]
    p = "blk.%d." % il
    out = [(p + "ffn_gate_inp.weight", [H, E], capi.F32, L["router"])]
    if fused_gate_up:
        assert L["gate_type"] == L["up_type"]
        both = np.concatenate([L["gate"], L["up"]], axis=1)  # per expert: ffn gate rows, then ffn up rows
        out.append((p + "ffn_gate_up_exps.weight", [H, 2 * F, E], L["gate_type"], both))
    else:
        out.append((p + "ffn_gate_exps.weight", [H, F, E], L["gate_type"], L["gate"]))
        out.append((p + "ffn_up_exps.weight", [H, F, E], L["up_type"], L["up"]))
    out.append((p + "ffn_down_exps.weight", [F, H, E], L["down_type"], L["down"]))
    if L.get("shared_gate_inp") is not None:
        out += [(p + "ffn_gate_inp_shexp.weight", [H], capi.F32, L["shared_gate_inp"]),
                (p + "ffn_gate_shexp.weight", [H, F], L["shared_type"], L["shared_gate"]),
                (p + "ffn_up_shexp.weight", [H, F], L["shared_type"], L["shared_up"]),
                (p + "ffn_down_shexp.weight", [F, H], L["shared_type"], L["shared_down"])]
    return out


class GgufFile:
    """Read-only view of a GGUF file through the library's parser."""

    def __init__(self, path):
        self.h = C.c_void_p()
        capi.call("wd_gguf_open", C.byref(self.h), str(path).encode())
        lib = capi.load()
        self.version = lib.wd_gguf_version(self.h)
        self.data_offset = lib.wd_gguf_data_offset(self.h)
        self.map_base, self.map_bytes, self.fd = lib.wd_gguf_map_base(self.h), lib.wd_gguf_map_bytes(self.h), lib.wd_gguf_fd(self.h)
        self.tensors = {}
        for i in range(lib.wd_gguf_tensor_count(self.h)):
            ti = capi.GgufTensorInfo()
            capi.call("wd_gguf_tensor", self.h, i, C.byref(ti))
            self.tensors[ti.name.decode()] = dict(dims=list(ti.dims[:ti.n_dims]), type=ti.type,
                                                  relative_offset=ti.relative_offset, bytes=ti.bytes, ptr=ti.data)

    def bytes_of(self, name):
        """Zero-copy uint8 view of a tensor's bytes; valid until close()."""
        t = self.tensors[name]
        return np.ctypeslib.as_array(C.cast(t["ptr"], C.POINTER(C.c_uint8)), shape=(t["bytes"],))

    def number(self, key, default=None):
        v = C.c_double()
        return v.value if capi.load().wd_gguf_meta_number(self.h, key.encode(), C.byref(v)) == 0 else default

    def string(self, key, default=None):
        s = capi.load().wd_gguf_meta_string(self.h, key.encode())
        return default if s is None else s.decode()

    def array(self, key):
        et, p = C.c_uint32(), C.c_void_p()
        n = capi.load().wd_gguf_meta_array(self.h, key.encode(), C.byref(et), C.byref(p))
        if n < 0:
            return None
        if et.value == STRING or n == 0:
            return n
        a = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n * np.dtype(_NP[et.value]).itemsize,))
        return a.view(_NP[et.value]).copy()

    def close(self):
        if self.h:
            capi.call("wd_gguf_close", self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
