"""GPU parity of the hyper-connection combine that consumes the MoE layer's output (stand-alone and folded into the
layer's last dispatch) against the CPU oracle, bit for bit."""
import ctypes as C

import numpy as np
import pytest

from warpdecode_amd import capi, synth

pytestmark = pytest.mark.gpu

SEED = 20261014
MOE_SPLIT_AB = 0x100      # WD_MOE_SPLIT_AB


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


def _case(hc, hidden, seed):
    rng = synth.rng_for(SEED, 500, hc, hidden, seed)
    return dict(res=rng.normal(0, 1, (hc, hidden)).astype(np.float32), routed=rng.normal(0, 0.3, hidden).astype(np.float32),
                shared=rng.normal(0, 0.3, hidden).astype(np.float32), gate=np.array([rng.uniform(0, 1)], np.float32),
                inject=rng.normal(0, 2, hc).astype(np.float32))


@pytest.mark.parametrize("hc,hidden", [(4, 2048), (4, 2560), (1, 32), (3, 100), (16, 257)])
@pytest.mark.parametrize("round_half", [0, 1])
def test_hc_combine(g, oracle, hc, hidden, round_half):
    c = _case(hc, hidden, round_half)
    block = oracle.hc_combine_moe(np.zeros((1, hidden), np.float32), c["routed"], c["shared"], c["gate"],
                                  np.full(1, 1e30, np.float32))[0] * np.float32(0.5)   # weight 2 sigmoid(huge) = 2: the branch itself
    d_inject, d_block = g.dev(c["inject"]), g.dev(block)
    res = g.dev(c["res"])
    capi.call("wd_hc_combine_f32", g.ptr(res), g.ptr(d_block), g.ptr(d_inject), hidden, hc, round_half, g.stream())
    g.sync()
    assert g.same_bits(g.host(res), oracle.hc_combine(c["res"], block, c["inject"], round_half))
    for shared in (c["shared"], c["shared"].astype(np.float16).view(np.uint16)):
        res, d_routed, d_shared, d_gate = g.dev(c["res"]), g.dev(c["routed"]), g.dev(shared), g.dev(c["gate"])
        capi.call("wd_hc_combine_moe_f32", g.ptr(res), g.ptr(d_routed), g.ptr(d_shared), int(shared.dtype == np.uint16),
                  g.ptr(d_gate), g.ptr(d_inject), hidden, hc, round_half, g.stream())
        g.sync()
        assert g.same_bits(g.host(res), oracle.hc_combine_moe(c["res"], c["routed"], shared, c["gate"], c["inject"], round_half))


def test_hc_weights_over_the_exponential_range(g, oracle):
    """Many streams of one value each: the device's table-driven expf against the oracle's (which is pinned to the C
    library's) from underflow to overflow, thresholds included, and values that round to subnormal halves."""
    rng = synth.rng_for(SEED, 501)
    hc = 8192
    z = np.concatenate([rng.uniform(-105, 105, hc - 16), np.array([0.0, -0.0, 88.7, 88.8, 89.0, -87.4, -103.9, -103.98, -104.5, 200.0,
                                                                   -200.0, 1e-30, np.inf, -np.inf, 17.0, -17.0])]).astype(np.float32)
    inject = (z * np.float32(hc)).astype(np.float32)
    for block_value, round_half in ((1.0, 0), (3e-6, 1), (60000.0, 1)):
        block = np.array([block_value], np.float32)
        res0 = rng.normal(0, 1e-6 if round_half else 1.0, (hc, 1)).astype(np.float32)
        res, d_block, d_inject = g.dev(res0), g.dev(block), g.dev(inject)
        capi.call("wd_hc_combine_f32", g.ptr(res), g.ptr(d_block), g.ptr(d_inject), 1, hc, round_half, g.stream())
        g.sync()
        want = oracle.hc_combine(res0, block, inject, round_half)
        got = g.host(res)
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), (z[~same.ravel()][:5], got[~same][:5], want[~same][:5])


@pytest.mark.parametrize("flags", [0, capi.MOE_STAGED, MOE_SPLIT_AB])
@pytest.mark.parametrize("shape", [(2048, 512, 64, 8, synth.IQ3_S, synth.Q8_0, True, 4), (256, 64, 16, 4, synth.Q8_0, synth.Q8_0, False, 3),
                                   (2560, 640, 32, 10, synth.IQ2_S, synth.IQ4_NL, True, 4), (1792, 512, 16, 4, synth.Q8_0, synth.Q8_0, True, 16)])
def test_layer_with_combine(g, oracle, flags, shape):
    """wd_moe_layer_hc_f32 = the layer, then the combine on its output: layer output and all residual streams against
    the oracle (the last shape has the most streams the folded form takes)."""
    H, F, E, k, gate_t, down_t, shared, hc = shape
    L = synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=SEED, layer=700 + hc, router_sigma=1.0 / np.sqrt(H))
    rng = synth.rng_for(SEED, 502, H, hc)
    x = synth.rms_normed(rng, H)
    res0 = rng.normal(0, 1, (hc, H)).astype(np.float32)
    inject = rng.normal(0, 2, hc).astype(np.float32)
    want_out, _ = oracle.moe_layer(L, x)
    for round_half in (0, 1):
        dl, sc = g.DeviceLayer(L), g.Scratch(H, F, E, k)
        res, out, dx, d_inject = g.dev(res0), g.empty(H, np.float32), g.dev(x), g.dev(inject)
        capi.call("wd_moe_layer_hc_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), g.ptr(res), g.ptr(d_inject), hc,
                  round_half, sc.h, flags, g.stream())
        g.sync()
        assert capi.load().wd_moe_scratch_status(sc.h) == 0
        assert g.same_bits(g.host(out), want_out)
        assert g.same_bits(g.host(res), oracle.hc_combine(res0, want_out, inject, round_half))
        sc.close()


def test_hc_error_paths(g):
    x = g.empty(64, np.float32)
    lib = capi.load()
    L = synth.make_layer(256, 64, 8, 2, synth.Q8_0, synth.Q8_0, False, seed=SEED, layer=3)
    dl, sc = g.DeviceLayer(L), g.Scratch(256, 64, 8, 2)
    big = g.empty(17 * 256, np.float32)
    call = lambda hc, flags: lib.wd_moe_layer_hc_f32(C.byref(dl.desc), g.ptr(big), g.ptr(big), g.ptr(big), g.ptr(big), hc, 0, sc.h, flags, None)
    assert call(17, 0) == -1 and b"1..16 residual streams" in lib.wd_last_error()
    assert call(0, 0) == -1
    assert call(4, 0x10) == -1 and b"measurement flags" in lib.wd_last_error()      # WD_MOE_ONLY_A
    assert lib.wd_moe_layer_hc_f32(C.byref(dl.desc), g.ptr(big), g.ptr(big), None, g.ptr(big), 4, 0, sc.h, 0, None) == -1
    sc.close()
    assert lib.wd_hc_combine_f32(None, g.ptr(x), g.ptr(x), 16, 4, 0, None) == -1
    assert lib.wd_hc_combine_f32(g.ptr(x), g.ptr(x), g.ptr(x), 0, 4, 0, None) == -1
    assert lib.wd_hc_combine_moe_f32(g.ptr(x), g.ptr(x), None, 0, g.ptr(x), g.ptr(x), 16, 4, 0, None) == -1
