"""Helpers for the GPU parity tests: numpy <-> device buffers through torch, calls through the C ABI."""
import ctypes as C

import numpy as np
import torch

from warpdecode_amd import capi

_NP2T = {np.dtype(np.float32): torch.float32, np.dtype(np.int8): torch.int8, np.dtype(np.uint8): torch.uint8,
         np.dtype(np.int16): torch.int16, np.dtype(np.int32): torch.int32, np.dtype(np.uint16): torch.int16,
         np.dtype(np.int64): torch.int64, np.dtype(np.uint64): torch.int64}


def init():
    capi.call("wd_init", 0)


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def dev(a):
    """numpy array -> device tensor holding the same bytes."""
    a = np.ascontiguousarray(a)
    if a.dtype in (np.uint16, np.uint64):
        a = a.view(np.int16 if a.dtype == np.uint16 else np.int64)
    return torch.from_numpy(a.copy()).cuda()


def empty(shape, dtype):
    dtype = np.dtype(dtype)
    return torch.zeros(shape, dtype=_NP2T[dtype], device="cuda")


def host(t, dtype=None):
    a = t.detach().cpu().numpy()
    if dtype is not None:
        a = a.view(dtype)
    return a


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def sync():
    torch.cuda.synchronize()


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def same_bits(a, b):
    return np.array_equal(bits(a), bits(b))


def view_f32(p, n):
    """Copy n floats from a raw device pointer (library-owned scratch) to the host."""
    out = np.empty(n, np.float32)
    capi.call("wd_memcpy_d2h", out.ctypes.data_as(C.c_void_p), C.c_void_p(p), n * 4, None)
    return out


def view(p, n, dtype):
    out = np.empty(n, dtype)
    capi.call("wd_memcpy_d2h", out.ctypes.data_as(C.c_void_p), C.c_void_p(p), out.nbytes, None)
    return out


class DeviceLayer:
    """Uploads a synth.make_layer() dict and builds the wd_moe_layer descriptor."""

    def __init__(self, L):
        from warpdecode_amd import synth
        self.L = L
        self.keep = {}
        d = capi.MoeLayer()
        d.hidden, d.expert_ffn, d.n_experts, d.top_k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
        d.expert_scale = float(L.get("w_scale", 1.0))
        d.gate_type, d.up_type, d.down_type = L["gate_type"], L["up_type"], L["down_type"]
        for name in ("router", "gate", "up", "down"):
            self.keep[name] = dev(L[name])
            setattr(d, name, self.keep[name].data_ptr())
        H, F = L["hidden"], L["expert_ffn"]
        d.gate_stride = F * synth.row_bytes(L["gate_type"], H)
        d.up_stride = F * synth.row_bytes(L["up_type"], H)
        d.down_stride = H * synth.row_bytes(L["down_type"], F)
        if L.get("shared_gate_inp") is not None:
            for name in ("shared_gate_inp", "shared_gate", "shared_up", "shared_down"):
                self.keep[name] = dev(L[name])
                setattr(d, name, self.keep[name].data_ptr())
        self.desc = d


class Scratch:
    def __init__(self, H, F, E, k):
        self.h = C.c_void_p()
        capi.call("wd_moe_scratch_create", C.byref(self.h), H, F, E, k)
        self.H, self.F, self.E, self.k = H, F, E, k

    def get(self, name, n, dtype):
        p = getattr(capi.load(), "wd_moe_scratch_" + name)(self.h)
        return view(p, n, dtype)

    def raw(self, name):
        return getattr(capi.load(), "wd_moe_scratch_" + name)(self.h)

    def close(self):
        if self.h:
            capi.call("wd_moe_scratch_destroy", self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
