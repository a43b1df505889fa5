"""The layer pass that allocates nothing (static device scratch) against wd_moe_layer_f32: two calls in a row, the
second with a smaller layer, bit for bit; sizes beyond the static array are refused."""
import ctypes as C

import numpy as np
import pytest

from warpdecode_amd import capi, synth

pytestmark = pytest.mark.gpu
SEED = 20261014


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


def _both(g, L, x):
    dl = g.DeviceLayer(L)
    H, F, E, k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
    dx = g.dev(x)
    want, got = g.empty(H, np.float32), g.empty(H, np.float32)
    sc = g.Scratch(H, F, E, k)
    capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(want), sc.h, 0, g.stream())
    capi.call("wd_moe_layer_noalloc_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(got), 0, g.stream())
    g.sync()
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    sc.close()
    return g.host(got), g.host(want)


def test_no_alloc_layer_pass_matches_the_scratch_object_path(g):
    big = synth.make_c2(layer=400, n_experts=64)                                    # hidden 2048, ffn 512, top-10, shared expert
    small = synth.make_layer(1024, 256, 32, 4, synth.IQ2_S, synth.IQ4_NL, shared=False, layer=401,
                             router_sigma=1.0 / np.sqrt(1024.0))
    for step, L in enumerate([big, small, big]):
        x = synth.rms_normed(synth.rng_for(SEED, 90, step), L["hidden"])
        got, want = _both(g, L, x)
        assert np.isfinite(want).all()
        assert g.same_bits(got, want), step


def test_no_alloc_layer_pass_refuses_what_does_not_fit(g):
    L = synth.make_layer(512, 128, 16, 2, synth.Q8_0, synth.Q8_0, shared=False, layer=402)
    dl = g.DeviceLayer(L)
    dx, out = g.dev(synth.rms_normed(synth.rng_for(SEED, 91), 512)), g.empty(512, np.float32)
    for field, value in (("hidden", 8192), ("expert_ffn", 2048), ("n_experts", 2048), ("top_k", 17)):
        d = capi.MoeLayer.from_buffer_copy(dl.desc)
        setattr(d, field, value)
        with pytest.raises(capi.WdError):
            capi.call("wd_moe_layer_noalloc_f32", C.byref(d), g.ptr(dx), g.ptr(out), 0, g.stream())
    with pytest.raises(capi.WdError):                                                 # staged dispatches need the scratch object
        capi.call("wd_moe_layer_noalloc_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), 4, g.stream())
    g.sync()
