"""Layer stacks on the GPU against the CPU oracle applied layer by layer: the all-resident stack entry point
(with and without a routing trace, fused and staged) and the stack fed from the expert-slot cache (trace known
to the host with fills queued one layer ahead; router-driven with the ids going through the host)."""
import ctypes as C

import numpy as np
import pytest

from warpdecode_amd import capi, synth

pytestmark = pytest.mark.gpu
SEED = 20261014
H, F, E, K, NL = 512, 128, 32, 4, 3
SCALE = np.float32(2.0 ** -6)


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


@pytest.fixture(scope="module")
def layers():
    return [synth.make_layer(H, F, E, K, synth.IQ3_S, synth.Q8_0, shared=True, layer=80 + l,
                             router_sigma=1.0 / np.sqrt(H)) for l in range(NL)]


def _oracle_stack(oracle, layers, x, trace):
    x = x.copy()
    all_ids, out = [], None
    for l, L in enumerate(layers):
        if trace is None:
            out, dump = oracle.moe_layer(L, x)
        else:
            _, wts = oracle.route(oracle.router_logits(L["router"], x), K)
            out, dump = oracle.moe_layer(L, x, ids=trace[l], weights=wts)
        all_ids.append(dump["ids"].copy())
        x = (x + (out * SCALE).astype(np.float32)).astype(np.float32)
    return x, out, np.stack(all_ids)


def _descs(g, layers):
    dls = [g.DeviceLayer(L) for L in layers]
    arr = (capi.MoeLayer * len(layers))()
    for i, dl in enumerate(dls):
        arr[i] = dl.desc
    return dls, arr


def _trace(step):
    rng = np.random.default_rng(SEED + 100 + step)
    return np.stack([rng.choice(E, size=K, replace=False) for _ in range(NL)]).astype(np.int32)


@pytest.mark.parametrize("flags", [0, 4], ids=["fused", "staged"])
@pytest.mark.parametrize("use_trace", [False, True], ids=["router", "trace"])
def test_resident_stack(g, oracle, layers, flags, use_trace):
    dls, arr = _descs(g, layers)
    sc = g.Scratch(H, F, E, K)
    for step in range(2):
        x = synth.rms_normed(synth.rng_for(SEED, 81, step), H)
        tr = _trace(step) if use_trace else None
        dx, out = g.dev(x), g.empty(H, np.float32)
        dtr = g.dev(tr) if use_trace else None
        capi.call("wd_moe_stack_f32", arr, NL, g.ptr(dx), g.ptr(out), sc.h, g.ptr(dtr), float(SCALE), flags, g.stream())
        g.sync()
        wx, wout, _ = _oracle_stack(oracle, layers, x, tr)
        assert g.same_bits(g.host(dx), wx), (step, flags)
        assert g.same_bits(g.host(out), wout), (step, flags)
    sc.close()


@pytest.mark.parametrize("slots", [NL * E, 20], ids=["all-resident", "lru-20-slots"])
@pytest.mark.parametrize("use_trace", [False, True], ids=["router", "trace"])
def test_cached_stack(g, oracle, layers, slots, use_trace):
    import torch
    gb = F * synth.row_bytes(synth.IQ3_S, H)
    db = H * synth.row_bytes(synth.Q8_0, F)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), slots * (2 * gb + db), gb, gb, db, NL, E, 0)
    pinned = []
    for l, L in enumerate(layers):
        p = [torch.from_numpy(np.ascontiguousarray(L[n]).reshape(-1)).pin_memory() for n in ("gate", "up", "down")]
        pinned.append(p)
        capi.call("wd_expert_cache_register_layer", cache, l, *[C.c_void_p(t.data_ptr()) for t in p])
    dls, arr = _descs(g, layers)
    for i in range(NL):                      # the routed tensors live only in the cache
        arr[i].gate = arr[i].up = arr[i].down = None
    sc = g.Scratch(H, F, E, K)
    for step in range(5):
        x = synth.rms_normed(synth.rng_for(SEED, 82, step), H)
        tr = _trace(step) if use_trace else None
        dx, out = g.dev(x), g.empty(H, np.float32)
        dtr = g.dev(tr) if use_trace else None
        htr = tr.ctypes.data_as(C.c_void_p) if use_trace else None
        capi.call("wd_moe_stack_cached_f32", arr, NL, cache, g.ptr(dx), g.ptr(out), sc.h, htr, g.ptr(dtr), float(SCALE), 0,
                  g.stream())
        g.sync()
        wx, wout, _ = _oracle_stack(oracle, layers, x, tr)
        assert g.same_bits(g.host(dx), wx), step
        assert g.same_bits(g.host(out), wout), step
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert st.accesses == 5 * NL * K and st.hits + st.misses == st.accesses
    assert st.bytes_copied == st.misses * (2 * gb + db)
    if slots < NL * E:
        assert st.evictions > 0 and st.resident <= slots
    else:
        assert st.evictions == 0
    sc.close()
    capi.call("wd_expert_cache_destroy", cache)
