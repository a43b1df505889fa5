"""ctypes bindings for the CPU oracle (oracle/libwdoracle.so) and, when it has been
built, for the reference's own CPU MoE header (oracle/_ref/libwdref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

F32, Q4_0, Q8_0, IQ4_NL, IQ3_S, IQ2_S = 0, 2, 8, 20, 21, 22

_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_i16p = C.POINTER(C.c_int16)
_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)


def build(force=False):
    """Compile the oracle (and the reference shim when /root/reference exists)."""
    so = os.path.join(_HERE, "libwdoracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-s", "-C", _HERE, "all"])
    return so


def _ptr(a, t):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(t)


class WdoLayer(C.Structure):
    _fields_ = [
        ("hidden", C.c_int), ("expert_ffn", C.c_int), ("n_experts", C.c_int), ("top_k", C.c_int),
        ("w_scale", C.c_float),
        ("router", _f32p),
        ("gate_type", C.c_int), ("up_type", C.c_int), ("down_type", C.c_int),
        ("gate", _u8p), ("up", _u8p), ("down", _u8p),
        ("shared_gate_inp", _f32p),
        ("shared_type", C.c_int),
        ("shared_gate", _u8p), ("shared_up", _u8p), ("shared_down", _u8p),
    ]


class WdoDump(C.Structure):
    _fields_ = [
        ("logits", _f32p), ("ids", C.POINTER(C.c_int)), ("weights", _f32p),
        ("gate_up", _f32p), ("act", _f32p), ("act_qs", _i8p), ("act_d", _u16p),
        ("expert_out", _f32p), ("routed", _f32p), ("shared_out", _f32p), ("shared_gate", _f32p),
        ("gate_up_partials", _i32p), ("down_partials", _i32p),
    ]


def _load():
    lib = C.CDLL(build())
    lib.wdo_iq3s_grid.restype = C.POINTER(C.c_uint32)
    lib.wdo_iq2s_grid.restype = C.POINTER(C.c_uint64)
    lib.wdo_row_bytes.restype = C.c_size_t
    lib.wdo_row_bytes.argtypes = [C.c_int, C.c_int]
    lib.wdo_f16_to_f32.restype = C.c_float
    lib.wdo_f16_to_f32.argtypes = [C.c_uint16]
    lib.wdo_f32_to_f16.restype = C.c_uint16
    lib.wdo_f32_to_f16.argtypes = [C.c_float]
    lib.wdo_quantize_q8_0.argtypes = [_f32p, C.c_int, _i8p, _u16p]
    lib.wdo_quantize_q8_K.argtypes = [_f32p, C.c_int, _i8p, _f32p, _i16p]
    lib.wdo_f32_to_f16_rn.restype = C.c_uint16
    lib.wdo_f32_to_f16_rn.argtypes = [C.c_float]
    lib.wdo_quantize_q8_1.restype = None
    lib.wdo_quantize_q8_1.argtypes = [_f32p, C.c_int, _i8p, _u16p]
    lib.wdo_gemv_q8_0_q8_1.restype = None
    lib.wdo_gemv_q8_0_q8_1.argtypes = [_u8p, C.c_int, C.c_int, _i8p, _u16p, _f32p, _i32p]
    lib.wdo_quantize_q8_0_f16.restype = None
    lib.wdo_quantize_q8_0_f16.argtypes = [_u16p, C.c_int, _i8p, _u16p]
    lib.wdo_gemv.argtypes = [C.c_int, _u8p, C.c_int, C.c_int, _i8p, C.c_void_p, _f32p, _i32p]
    lib.wdo_dequant_row.argtypes = [C.c_int, _u8p, C.c_int, _f32p]
    lib.wdo_gemv_q6_K.argtypes = [_u8p, C.c_int, C.c_int, _i8p, _f32p, _i16p, _f32p, _i32p]
    for n in ("wdo_exp_ggml", "wdo_silu_ggml", "wdo_sigmoid_ggml"):
        getattr(lib, n).restype = C.c_float
        getattr(lib, n).argtypes = [C.c_float]
    lib.wdo_dot_f32.restype = C.c_float
    lib.wdo_dot_f32.argtypes = [_f32p, _f32p, C.c_int]
    for n in ("wdo_expf_glibc", "wdo_sigmoid_exact", "wdo_round_half"):
        getattr(lib, n).restype = C.c_float
        getattr(lib, n).argtypes = [C.c_float]
    for n in ("wdo_expf_glibc_n", "wdo_libm_expf_n", "wdo_round_half_n"):
        getattr(lib, n).restype = None
        getattr(lib, n).argtypes = [_f32p, C.c_int, _f32p]
    for n in ("wdo_moe_branch_f32", "wdo_residual_add_f32"):
        getattr(lib, n).restype = C.c_float
        getattr(lib, n).argtypes = [C.c_float] * 3
    lib.wdo_hc_combine_f32.restype = None
    lib.wdo_hc_combine_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.wdo_hc_combine_moe_f32.restype = None
    lib.wdo_hc_combine_moe_f32.argtypes = [_f32p, _f32p, C.c_void_p, C.c_int, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.wdo_router_logits.argtypes = [_f32p, _f32p, C.c_int, C.c_int, _f32p]
    lib.wdo_softmax_row.argtypes = [_f32p, C.c_int, _f32p]
    lib.wdo_router_select.argtypes = [_f32p, C.c_int, C.c_int, C.c_float, C.POINTER(C.c_int), _f32p]
    lib.wdo_expert_ffn.argtypes = [C.c_int, C.c_int, C.c_int, _u8p, _u8p, _u8p, C.c_int, C.c_int, _f32p, _f32p,
                                   _f32p, _f32p, _i8p, _u16p, _i32p, _i32p]
    lib.wdo_moe_layer_mt.argtypes = [C.POINTER(WdoLayer), _f32p, _f32p, C.POINTER(WdoDump), C.c_int, C.c_int]
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


# ---------------------------------------------------------------------------------
# numpy-level API
# ---------------------------------------------------------------------------------
def iq3s_grid():
    return np.ctypeslib.as_array(lib().wdo_iq3s_grid(), shape=(512,)).copy()


def iq2s_grid():
    return np.ctypeslib.as_array(lib().wdo_iq2s_grid(), shape=(1024,)).copy()


def row_bytes(t, cols):
    return int(lib().wdo_row_bytes(t, cols))


def partials_per_row(t, cols):
    if t in (IQ3_S, IQ2_S):
        return cols // 256 * 8
    if t in (Q8_0, IQ4_NL):
        return cols // 32 * 8
    if t == Q4_0:
        return cols // 32
    raise ValueError(t)


def f16_to_f32(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return np.array([lib().wdo_f16_to_f32(int(b)) for b in bits.ravel()], dtype=np.float32).reshape(bits.shape)


def f32_to_f16(vals):
    vals = np.asarray(vals, dtype=np.float32)
    return np.array([lib().wdo_f32_to_f16(float(v)) for v in vals.ravel()], dtype=np.uint16).reshape(vals.shape)


def quantize_q8_0(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.size
    qs = np.empty(n, np.int8)
    d = np.empty(n // 32, np.uint16)
    lib().wdo_quantize_q8_0(_ptr(x, _f32p), n, _ptr(qs, _i8p), _ptr(d, _u16p))
    return qs, d


def f32_to_f16_rn(vals):
    """IEEE round-to-nearest-even float -> half bits."""
    vals = np.asarray(vals, dtype=np.float32)
    return np.array([lib().wdo_f32_to_f16_rn(float(v)) for v in vals.ravel()], dtype=np.uint16).reshape(vals.shape)


def quantize_q8_1(x):
    """src/lowbit.cuh:287-308: q = roundf(x / d), d = amax / 127, scale as half(d)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    qs, d = np.empty(x.size, np.int8), np.empty(x.size // 32, np.uint16)
    lib().wdo_quantize_q8_1(_ptr(x, _f32p), x.size, _ptr(qs, _i8p), _ptr(d, _u16p))
    return qs, d


def gemv_q8_0_q8_1(w, rows, cols, qs, d):
    """src/lowbit.cuh:310-341.  Returns (y f32[rows], block sums int32[rows][cols/32])."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    y, sums = np.empty(rows, np.float32), np.empty((rows, cols // 32), np.int32)
    lib().wdo_gemv_q8_0_q8_1(_ptr(w, _u8p), rows, cols, _ptr(np.ascontiguousarray(qs, np.int8), _i8p),
                             _ptr(np.ascontiguousarray(d, np.uint16), _u16p), _ptr(y, _f32p), _ptr(sums, _i32p))
    return y, sums


def quantize_q8_0_f16(x_bits):
    """src/warodecode.cu:1504-1520: Q8_0 activation from half input (bits)."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    qs, d = np.empty(x_bits.size, np.int8), np.empty(x_bits.size // 32, np.uint16)
    lib().wdo_quantize_q8_0_f16(_ptr(x_bits, _u16p), x_bits.size, _ptr(qs, _i8p), _ptr(d, _u16p))
    return qs, d


def quantize_q8_K(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.size
    qs = np.empty(n, np.int8)
    d = np.empty(n // 256, np.float32)
    bs = np.empty(n // 16, np.int16)
    lib().wdo_quantize_q8_K(_ptr(x, _f32p), n, _ptr(qs, _i8p), _ptr(d, _f32p), _ptr(bs, _i16p))
    return qs, d, bs


def gemv(t, w, rows, cols, act_qs, act_d, want_partials=False):
    w = np.ascontiguousarray(w, dtype=np.uint8)
    assert w.size == rows * row_bytes(t, cols), (w.size, rows, cols, t)
    out = np.empty(rows, np.float32)
    part = np.empty((rows, partials_per_row(t, cols)), np.int32) if want_partials else None
    act_qs = np.ascontiguousarray(act_qs, dtype=np.int8)
    want_d = np.float32 if t in (IQ3_S, IQ2_S) else np.uint16
    act_d = np.ascontiguousarray(act_d, dtype=want_d)
    lib().wdo_gemv(t, _ptr(w, _u8p), rows, cols, _ptr(act_qs, _i8p), act_d.ctypes.data_as(C.c_void_p),
                   _ptr(out, _f32p), _ptr(part, _i32p))
    return (out, part) if want_partials else out


def gemv_q6_K(w, rows, cols, act_qs, act_d, act_bsums, want_partials=False):
    """Q6_K x Q8_K rows (the output head): out f32 [rows], partials int32 [rows][cols/256][8]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    assert w.size == rows * (cols // 256) * 210
    out = np.empty(rows, np.float32)
    part = np.empty((rows, cols // 256 * 8), np.int32) if want_partials else None
    lib().wdo_gemv_q6_K(_ptr(w, _u8p), rows, cols, _ptr(np.ascontiguousarray(act_qs, np.int8), _i8p),
                        _ptr(np.ascontiguousarray(act_d, np.float32), _f32p),
                        _ptr(np.ascontiguousarray(act_bsums, np.int16), _i16p), _ptr(out, _f32p), _ptr(part, _i32p))
    return (out, part) if want_partials else out


def dequant_row(t, w_row, cols):
    w_row = np.ascontiguousarray(w_row, dtype=np.uint8)
    out = np.empty(cols, np.float32)
    lib().wdo_dequant_row(t, _ptr(w_row, _u8p), cols, _ptr(out, _f32p))
    return out


def exp_ggml(x):
    x = np.asarray(x, dtype=np.float32)
    return np.array([lib().wdo_exp_ggml(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def silu_ggml(x):
    x = np.asarray(x, dtype=np.float32)
    return np.array([lib().wdo_silu_ggml(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def sigmoid_ggml(x):
    return np.float32(lib().wdo_sigmoid_ggml(float(x)))


def _map_f32(name, x):
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.empty_like(x)
    getattr(lib(), name)(_ptr(x, _f32p), x.size, _ptr(out, _f32p))
    return out


def expf_glibc(x):
    return _map_f32("wdo_expf_glibc_n", x)


def libm_expf(x):
    return _map_f32("wdo_libm_expf_n", x)


def round_half(x):
    return _map_f32("wdo_round_half_n", x)


def sigmoid_exact(x):
    return np.float32(lib().wdo_sigmoid_exact(float(x)))


def hc_combine(residual, block_out, inject, round_half=False):
    """residual [hc][hidden] (a copy is updated and returned), block_out [hidden], inject [hc]."""
    res = np.array(residual, dtype=np.float32, order="C", copy=True)
    hc, hidden = res.shape
    lib().wdo_hc_combine_f32(_ptr(res, _f32p), _ptr(np.ascontiguousarray(block_out, np.float32), _f32p),
                             _ptr(np.ascontiguousarray(inject, np.float32), _f32p), hidden, hc, int(round_half))
    return res


def hc_combine_moe(residual, routed, shared, shared_gate, inject, round_half=False):
    """shared: float32 [hidden], or uint16 [hidden] holding half bits."""
    res = np.array(residual, dtype=np.float32, order="C", copy=True)
    hc, hidden = res.shape
    shared = np.ascontiguousarray(shared)
    assert shared.dtype in (np.float32, np.uint16)
    lib().wdo_hc_combine_moe_f32(_ptr(res, _f32p), _ptr(np.ascontiguousarray(routed, np.float32), _f32p),
                                 shared.ctypes.data_as(C.c_void_p), int(shared.dtype == np.uint16),
                                 _ptr(np.ascontiguousarray(shared_gate, np.float32).reshape(1), _f32p),
                                 _ptr(np.ascontiguousarray(inject, np.float32), _f32p), hidden, hc, int(round_half))
    return res


def dot_f32(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return np.float32(lib().wdo_dot_f32(_ptr(a, _f32p), _ptr(b, _f32p), a.size))


def router_logits(w, x):
    w = np.ascontiguousarray(w, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = w.shape
    out = np.empty(rows, np.float32)
    lib().wdo_router_logits(_ptr(w, _f32p), _ptr(x, _f32p), rows, cols, _ptr(out, _f32p))
    return out


def softmax_row(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    probs = np.empty_like(logits)
    lib().wdo_softmax_row(_ptr(logits, _f32p), logits.size, _ptr(probs, _f32p))
    return probs


def router_select(probs, k, w_scale=1.0):
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    ids = np.empty(k, np.int32)
    wts = np.empty(k, np.float32)
    lib().wdo_router_select(_ptr(probs, _f32p), probs.size, k, w_scale, ids.ctypes.data_as(C.POINTER(C.c_int)),
                            _ptr(wts, _f32p))
    return ids, wts


def route(logits, k, w_scale=1.0):
    return router_select(softmax_row(logits), k, w_scale)


def expert_ffn(gate_t, up_t, down_t, gate, up, down, H, F, x, want=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(H, np.float32)
    if want:
        gu = np.empty((2, F), np.float32)
        act = np.empty(F, np.float32)
        aq = np.empty(F, np.int8)
        ad = np.empty(F // 32, np.uint16)
        gp = np.empty((2, F, partials_per_row(gate_t, H)), np.int32)
        dp = np.empty((H, partials_per_row(down_t, F)), np.int32)
    else:
        gu = act = aq = ad = gp = dp = None
    lib().wdo_expert_ffn(gate_t, up_t, down_t, _ptr(gate, _u8p), _ptr(up, _u8p), _ptr(down, _u8p), H, F,
                         _ptr(x, _f32p), _ptr(out, _f32p), _ptr(gu, _f32p), _ptr(act, _f32p), _ptr(aq, _i8p),
                         _ptr(ad, _u16p), _ptr(gp, _i32p), _ptr(dp, _i32p))
    if want:
        return out, dict(gate_up=gu, act=act, act_qs=aq, act_d=ad, gate_up_partials=gp, down_partials=dp)
    return out


def moe_layer(layer, x, ids=None, weights=None, threads=1, want_partials=False):
    """layer: dict as produced by warpdecode_amd.synth.make_layer (numpy arrays).
    Returns (out[H], dump dict)."""
    H, F, E, k = layer["hidden"], layer["expert_ffn"], layer["n_experts"], layer["top_k"]
    x = np.ascontiguousarray(x, dtype=np.float32)
    L = WdoLayer()
    L.hidden, L.expert_ffn, L.n_experts, L.top_k = H, F, E, k
    L.w_scale = float(layer.get("w_scale", 1.0))
    keep = []

    def u8(a):
        a = np.ascontiguousarray(a, dtype=np.uint8)
        keep.append(a)
        return _ptr(a, _u8p)

    def f32(a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        keep.append(a)
        return _ptr(a, _f32p)

    L.router = f32(layer["router"])
    L.gate_type, L.up_type, L.down_type = layer["gate_type"], layer["up_type"], layer["down_type"]
    L.gate, L.up, L.down = u8(layer["gate"]), u8(layer["up"]), u8(layer["down"])
    if layer.get("shared_gate_inp") is not None:
        L.shared_gate_inp = f32(layer["shared_gate_inp"])
        L.shared_type = layer.get("shared_type", Q8_0)
        L.shared_gate, L.shared_up, L.shared_down = (u8(layer["shared_gate"]), u8(layer["shared_up"]),
                                                     u8(layer["shared_down"]))
    d = dict(
        logits=np.zeros(E, np.float32), ids=np.zeros(k, np.int32), weights=np.zeros(k, np.float32),
        gate_up=np.empty((k, 2, F), np.float32), act=np.empty((k, F), np.float32),
        act_qs=np.empty((k, F), np.int8), act_d=np.empty((k, F // 32), np.uint16),
        expert_out=np.empty((k, H), np.float32), routed=np.empty(H, np.float32),
        shared_out=np.zeros(H, np.float32), shared_gate=np.zeros(1, np.float32))
    if want_partials:
        d["gate_up_partials"] = np.empty((k, 2, F, partials_per_row(L.gate_type, H)), np.int32)
        d["down_partials"] = np.empty((k, H, partials_per_row(L.down_type, F)), np.int32)
    pre = 0
    if ids is not None:
        d["ids"][:] = ids
        d["weights"][:] = weights
        pre = 1
    D = WdoDump()
    D.logits, D.weights = _ptr(d["logits"], _f32p), _ptr(d["weights"], _f32p)
    D.ids = d["ids"].ctypes.data_as(C.POINTER(C.c_int))
    D.gate_up, D.act = _ptr(d["gate_up"], _f32p), _ptr(d["act"], _f32p)
    D.act_qs, D.act_d = _ptr(d["act_qs"], _i8p), _ptr(d["act_d"], _u16p)
    D.expert_out, D.routed = _ptr(d["expert_out"], _f32p), _ptr(d["routed"], _f32p)
    D.shared_out, D.shared_gate = _ptr(d["shared_out"], _f32p), _ptr(d["shared_gate"], _f32p)
    if want_partials:
        D.gate_up_partials = _ptr(d["gate_up_partials"], _i32p)
        D.down_partials = _ptr(d["down_partials"], _i32p)
    out = np.empty(H, np.float32)
    lib().wdo_moe_layer_mt(C.byref(L), _ptr(x, _f32p), _ptr(out, _f32p), C.byref(D), pre, threads)
    return out, d


# ---------------------------------------------------------------------------------
# The reference's own header (only where oracle/_ref/libwdref.so has been built)
# ---------------------------------------------------------------------------------
_ref = None


def ref_path():
    return os.path.join(_HERE, "_ref", "libwdref.so")


def ref():
    """Returns the ctypes handle of the compiled reference header, or None."""
    global _ref
    if _ref is None:
        p = ref_path()
        if not os.path.exists(p):
            return None
        r = C.CDLL(p)
        r.wdref_iq3s_grid.restype = C.POINTER(C.c_uint32)
        r.wdref_iq2s_grid.restype = C.POINTER(C.c_uint64)
        r.wdref_f16_to_f32.restype = C.c_float
        r.wdref_f16_to_f32.argtypes = [C.c_uint16]
        r.wdref_f32_to_f16.restype = C.c_uint16
        r.wdref_f32_to_f16.argtypes = [C.c_float]
        for n in ("wdref_exp", "wdref_silu", "wdref_sigmoid"):
            getattr(r, n).restype = C.c_float
            getattr(r, n).argtypes = [C.c_float]
        r.wdref_dot_f32.restype = C.c_float
        r.wdref_dot_f32.argtypes = [_f32p, _f32p, C.c_int]
        if hasattr(r, "wdref_round_half"):
            r.wdref_round_half.restype = C.c_float
            r.wdref_round_half.argtypes = [C.c_float]
            for n in ("wdref_moe_branch_f32", "wdref_residual_add_f32"):
                getattr(r, n).restype = C.c_float
                getattr(r, n).argtypes = [C.c_float] * 3
        r.wdref_quantize_q8_0.argtypes = [_f32p, C.c_int, _i8p, _u16p]
        r.wdref_quantize_q8_K.argtypes = [_f32p, C.c_int, _i8p, _f32p, _i16p]
        r.wdref_row.restype = C.c_float
        r.wdref_row.argtypes = [C.c_int, _u8p, _i8p, C.c_void_p, C.c_int, C.c_int]
        r.wdref_gemv.argtypes = [C.c_int, _u8p, C.c_int, C.c_int, _i8p, C.c_void_p, _f32p]
        r.wdref_run_layer.argtypes = [_u8p, _u8p, _u8p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p,
                                      C.POINTER(C.c_int), _f32p, C.c_int, C.c_int, _f32p]
        r.wdref_q8_0_chain.argtypes = [_u8p, _u8p, _u8p, C.c_int, C.c_int, _f32p, _f32p]
        r.wdref_accumulate.argtypes = [_f32p, _f32p, C.c_float, C.c_int]
        _ref = r
    return _ref


def ref_gemv(t, w, rows, cols, act_qs, act_d):
    r = ref()
    w = np.ascontiguousarray(w, dtype=np.uint8)
    out = np.empty(rows, np.float32)
    act_qs = np.ascontiguousarray(act_qs, dtype=np.int8)
    act_d = np.ascontiguousarray(act_d, dtype=np.float32 if t in (IQ3_S, IQ2_S) else np.uint16)
    r.wdref_gemv(t, _ptr(w, _u8p), rows, cols, _ptr(act_qs, _i8p), act_d.ctypes.data_as(C.c_void_p),
                 _ptr(out, _f32p))
    return out


def ref_row(t, w_row, cols, act_qs, act_d, scalar=False):
    r = ref()
    w_row = np.ascontiguousarray(w_row, dtype=np.uint8)
    act_qs = np.ascontiguousarray(act_qs, dtype=np.int8)
    act_d = np.ascontiguousarray(act_d, dtype=np.float32 if t in (IQ3_S, IQ2_S) else np.uint16)
    return np.float32(r.wdref_row(t, _ptr(w_row, _u8p), _ptr(act_qs, _i8p), act_d.ctypes.data_as(C.c_void_p),
                                  cols, 1 if scalar else 0))


def ref_run_layer(layer, x, ids, weights, threads=1):
    """Routed experts through the reference's run_layer (IQ2_S/IQ3_S gate and up only)."""
    r = ref()
    H, F = layer["hidden"], layer["expert_ffn"]
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    out = np.empty(H, np.float32)
    r.wdref_run_layer(_ptr(layer["gate"], _u8p), _ptr(layer["up"], _u8p), _ptr(layer["down"], _u8p),
                      layer["gate_type"], layer["up_type"], layer["down_type"], H, F, _ptr(x, _f32p),
                      ids.ctypes.data_as(C.POINTER(C.c_int)), _ptr(weights, _f32p), ids.size, threads,
                      _ptr(out, _f32p))
    return out


def ref_q8_0_chain(gate, up, down, H, F, x):
    r = ref()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(H, np.float32)
    r.wdref_q8_0_chain(_ptr(gate, _u8p), _ptr(up, _u8p), _ptr(down, _u8p), H, F, _ptr(x, _f32p), _ptr(out, _f32p))
    return out
