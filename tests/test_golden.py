"""Golden vectors recorded from the reference's own CPU MoE header (tests/golden/ref_vectors.npz, written by
tests/golden/make_fixtures.py).  The CPU oracle must reproduce them bit for bit everywhere (also where the
reference tree is absent); the HIP library is then held to the same vectors through the C ABI."""
import ctypes as C
import os

import numpy as np
import pytest

from warpdecode_amd import capi, synth

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz")
COLS = [256, 512, 2048, 2560]
TYPES = [("iq3_s", synth.IQ3_S), ("iq2_s", synth.IQ2_S), ("iq4_nl", synth.IQ4_NL), ("q8_0", synth.Q8_0)]


@pytest.fixture(scope="module")
def gold():
    return np.load(PATH, allow_pickle=False)


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def _act(gold, t, cols):
    if t in (synth.IQ3_S, synth.IQ2_S):
        return gold["q8_k_qs_%d" % cols], gold["q8_k_d_%d" % cols]
    return gold["q8_0_qs_%d" % cols], gold["q8_0_d_%d" % cols]


# ---- CPU oracle against the recorded reference outputs ---------------------------------------------------

@pytest.mark.parametrize("cols", COLS)
def test_oracle_quantisers(gold, oracle, cols):
    x = gold["x_%d" % cols]
    qs, d = oracle.quantize_q8_0(x)
    assert np.array_equal(qs, gold["q8_0_qs_%d" % cols]) and np.array_equal(d, gold["q8_0_d_%d" % cols])
    kq, kd, kb = oracle.quantize_q8_K(x)
    assert np.array_equal(kq, gold["q8_k_qs_%d" % cols]) and np.array_equal(kb, gold["q8_k_bsums_%d" % cols])
    assert np.array_equal(bits(kd), bits(gold["q8_k_d_%d" % cols]))


@pytest.mark.parametrize("cols", COLS)
@pytest.mark.parametrize("name,t", TYPES)
def test_oracle_rows(gold, oracle, name, t, cols):
    aq, ad = _act(gold, t, cols)
    y = oracle.gemv(t, gold["w_%s_%d" % (name, cols)], 4, cols, aq, ad)
    assert np.array_equal(bits(y), bits(gold["y_%s_%d" % (name, cols)]))
    # the reference's scalar twin gives the same bits as its AVX2 kernel
    assert np.array_equal(bits(gold["y_scalar_%s_%d" % (name, cols)]), bits(gold["y_%s_%d" % (name, cols)]))


def test_oracle_functions(gold, oracle):
    v = gold["fn_x"]
    assert np.array_equal(bits([oracle.exp_ggml(a) for a in v]), bits(gold["fn_exp"]))
    assert np.array_equal(bits([oracle.silu_ggml(a) for a in v]), bits(gold["fn_silu"]))
    assert np.array_equal(bits([oracle.sigmoid_ggml(a) for a in v]), bits(gold["fn_sigmoid"]))
    for n in (8, 31, 32, 100, 2048):
        assert bits(oracle.dot_f32(gold["dot_a_%d" % n], gold["dot_b_%d" % n])) == bits(gold["dot_y_%d" % n])


def _gold_layer(gold):
    H, F, E, k = (int(v) for v in gold["layer_geometry"])
    L = dict(hidden=H, expert_ffn=F, n_experts=E, top_k=k, w_scale=1.0, gate_type=synth.IQ3_S, up_type=synth.IQ3_S,
             down_type=synth.Q8_0, shared_type=synth.Q8_0, router=np.zeros((E, H), np.float32),
             shared_gate_inp=np.zeros(H, np.float32))
    for name in ("gate", "up", "down", "shared_gate", "shared_up", "shared_down"):
        L[name] = gold["layer_" + name]
    return L


def test_oracle_layer(gold, oracle):
    L = _gold_layer(gold)
    x, ids, wts = gold["layer_x"], gold["layer_ids"], gold["layer_weights"]
    out, dump = oracle.moe_layer(L, x, ids=ids, weights=wts)
    assert np.array_equal(bits(dump["routed"]), bits(gold["layer_routed"]))
    assert np.array_equal(bits(dump["shared_out"]), bits(gold["layer_shared"]))
    # zero gate vector: gate = sigmoid(0) = 0.5, out = routed + shared * 0.5 with one rounding each
    want = (gold["layer_routed"] + (gold["layer_shared"] * np.float32(0.5)).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(out), bits(want))


# ---- HIP library against the same vectors ----------------------------------------------------------------------

@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


@pytest.mark.gpu
@pytest.mark.parametrize("cols", COLS)
def test_gpu_quantisers(gold, g, cols):
    dx = g.dev(gold["x_%d" % cols])
    qs, d = g.empty(cols, np.int8), g.empty(cols // 32, np.uint16)
    capi.call("wd_q8_0_quantize_f32", g.ptr(dx), cols, g.ptr(qs), g.ptr(d), g.stream())
    kq, kd, kb = g.empty(cols, np.int8), g.empty(cols // 256, np.float32), g.empty(cols // 16, np.int16)
    capi.call("wd_q8_k_quantize_f32", g.ptr(dx), cols, g.ptr(kq), g.ptr(kd), g.ptr(kb), g.stream())
    g.sync()
    assert np.array_equal(g.host(qs), gold["q8_0_qs_%d" % cols])
    assert np.array_equal(g.host(d, np.uint16), gold["q8_0_d_%d" % cols])
    assert np.array_equal(g.host(kq), gold["q8_k_qs_%d" % cols])
    assert np.array_equal(g.host(kb), gold["q8_k_bsums_%d" % cols])
    assert np.array_equal(bits(g.host(kd)), bits(gold["q8_k_d_%d" % cols]))


@pytest.mark.gpu
@pytest.mark.parametrize("cols", COLS)
@pytest.mark.parametrize("name,t", TYPES)
def test_gpu_rows(gold, g, name, t, cols):
    aq, ad = _act(gold, t, cols)
    w, dq, dd = g.dev(gold["w_%s_%d" % (name, cols)]), g.dev(aq), g.dev(ad)
    y = g.empty(4, np.float32)
    fn = "wd_gemv_q8_k_f32" if t in (synth.IQ3_S, synth.IQ2_S) else "wd_gemv_q8_0_f32"
    capi.call(fn, t, g.ptr(w), 4, cols, g.ptr(dq), g.ptr(dd), g.ptr(y), None, g.stream())
    g.sync()
    assert np.array_equal(bits(g.host(y)), bits(gold["y_%s_%d" % (name, cols)]))


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [0, 4], ids=["fused", "staged"])
def test_gpu_layer(gold, g, flags):
    L = _gold_layer(gold)
    H, F, E, k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
    dl, s = g.DeviceLayer(L), g.Scratch(H, F, E, k)
    ids, wts = g.dev(gold["layer_ids"]), g.dev(gold["layer_weights"])
    capi.call("wd_memcpy_d2d", C.c_void_p(s.raw("ids")), g.ptr(ids), 4 * k, g.stream())
    capi.call("wd_memcpy_d2d", C.c_void_p(s.raw("weights")), g.ptr(wts), 4 * k, g.stream())
    dx, out = g.dev(gold["layer_x"]), g.empty(H, np.float32)
    capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), s.h, 1 | flags, g.stream())
    g.sync()
    assert np.array_equal(bits(s.get("accum", H, np.float32)), bits(gold["layer_routed"]))
    assert np.array_equal(bits(s.get("down_f32", H, np.float32)), bits(gold["layer_shared"]))
    want = (gold["layer_routed"] + (gold["layer_shared"] * np.float32(0.5)).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(g.host(out)), bits(want))
    # the shared expert on its own entry point
    capi.call("wd_shared_expert_f32", C.byref(dl.desc), g.ptr(dx), s.h, g.stream())
    g.sync()
    assert np.array_equal(bits(s.get("down_f32", H, np.float32)), bits(gold["layer_shared"]))
    assert s.get("shared_gate", 1, np.float32)[0] == np.float32(0.5)
