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


# 20 slots: fills one layer ahead; 30 slots (at least two tokens' experts): the whole token is acquired ahead, with evictions
@pytest.mark.parametrize("slots", [NL * E, 30, 20], ids=["all-resident", "lru-30-slots", "lru-20-slots"])
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


def test_graph_replayed_c2_stack(g, oracle):
    """The benchmark's own mechanics at reduced size: an 8-layer stack of C2-shaped layers (64 experts) captured
    into a HIP graph and replayed for several tokens with fresh inputs and routing traces in between, every
    replay checked against the oracle applied layer by layer (and against an eager run of the same token)."""
    import torch
    NLc, Ec, Kc, Hc, Fc = 8, 64, 10, 2048, 512
    Ls = [synth.make_c2(layer=100 + l, n_experts=Ec) for l in range(NLc)]
    dls, arr = _descs(g, Ls)
    sc = g.Scratch(Hc, Fc, Ec, Kc)
    scale = np.float32(2.0 ** -12)
    d_x = torch.zeros(Hc, dtype=torch.float32, device="cuda")
    d_out = torch.zeros(Hc, dtype=torch.float32, device="cuda")
    d_tr = torch.zeros((NLc, Kc), dtype=torch.int32, device="cuda")

    def launch():
        capi.call("wd_moe_stack_f32", arr, NLc, g.ptr(d_x), g.ptr(d_out), sc.h, g.ptr(d_tr), float(scale), 0,
                  C.c_void_p(torch.cuda.current_stream().cuda_stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    rng = np.random.default_rng(SEED + 300)
    for token in range(4):
        x = synth.rms_normed(synth.rng_for(SEED, 83, token), Hc)
        tr = np.stack([rng.choice(Ec, size=Kc, replace=False) for _ in range(NLc)]).astype(np.int32)
        d_x.copy_(torch.from_numpy(x).cuda())
        d_tr.copy_(torch.from_numpy(tr).cuda())
        graph.replay()
        torch.cuda.synchronize()
        got_x, got_out = d_x.cpu().numpy(), d_out.cpu().numpy()
        # oracle, layer by layer (router weights, ids from the trace)
        wx = x.copy()
        for l, L in enumerate(Ls):
            _, wts = oracle.route(oracle.router_logits(L["router"], wx), Kc)
            wout, _ = oracle.moe_layer(L, wx, ids=tr[l], weights=wts)
            wx = (wx + (wout * scale).astype(np.float32)).astype(np.float32)
        assert g.same_bits(got_x, wx), token
        assert g.same_bits(got_out, wout), token
        # the same token eagerly, between two replays
        d_x.copy_(torch.from_numpy(x).cuda())
        launch()
        torch.cuda.synchronize()
        assert g.same_bits(d_x.cpu().numpy(), wx), token
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    sc.close()


# ---- the stack as ONE launch of resident workgroups (layers of the 512-expert shape: hidden 2048, ffn 512) -------------
PER_LAYER = 0x200
VIEWS = (("ids", "k", np.int32), ("weights", "k", np.float32), ("logits", "E", np.float32), ("accum", "H", np.float32),
         ("down_f32", "H", np.float32), ("shared_gate", 1, np.float32))


def _run_stack(g, arr, n, x, tr, sc, flags):
    dx, out = g.dev(x), g.empty(2048, np.float32)
    dtr = g.dev(tr) if tr is not None else None
    capi.call("wd_moe_stack_f32", arr, n, g.ptr(dx), g.ptr(out), sc.h, g.ptr(dtr), float(2.0 ** -12), flags, g.stream())
    g.sync()
    views = {}
    for name, n_, dt in VIEWS:
        cnt = {"k": sc.k, "E": sc.E, "H": sc.H}.get(n_, n_)
        views[name] = sc.get(name, cnt, dt)
    return g.host(dx), g.host(out), views


# The last case is the shape the benchmark measures: 512 experts (every workgroup owns a router row, all eight selecting
# waves of workgroup 0 hold live logits, the poll of the logit records is full), top-10, a shared expert.
@pytest.mark.parametrize("gate_type,experts,k,shared,nl", [(synth.IQ3_S, 64, 10, True, 5), (synth.IQ2_S, 40, 6, True, 5),
                                                           (synth.IQ3_S, 128, 9, False, 5), (synth.IQ3_S, 512, 10, True, 3),
                                                           (synth.Q8_0, 64, 8, False, 4), (synth.Q8_0, 32, 5, True, 3)],
                         ids=["iq3s-64x10-shared", "iq2s-40x6-shared", "iq3s-128x9", "iq3s-512x10-shared", "q8-64x8", "q8-32x5-shared"])
def test_one_launch_stack_matches_per_layer_and_oracle(g, oracle, gate_type, experts, k, shared, nl):
    """The resident launch against the per-layer dispatches (every output and every view of the last layer, bit for
    bit) over launches in a row with stacks of different depth, with and without a routing trace; the first token
    (router-selected ids) and the second (ids from a trace) also against the oracle applied layer by layer."""
    Ls = [synth.make_layer(2048, 512, experts, k, gate_type, synth.Q8_0, shared=shared, layer=300 + l,
                           router_sigma=1.0 / np.sqrt(2048.0)) for l in range(nl)]
    dls, arr = _descs(g, Ls)
    sc_a, sc_b = g.Scratch(2048, 512, experts, k), g.Scratch(2048, 512, experts, k)
    rng = np.random.default_rng(SEED + 400)
    # The comparison below says nothing if the first form quietly took the dispatches per layer as well (a device that
    # does not hold the 512 workgroups at once makes it do so): the site profiler counts the launches of either form.
    lib = capi.load()
    site = {lib.wd_profile_site_name(i).decode(): i for i in range(64) if lib.wd_profile_site_name(i) != b"unknown"}
    site_resident = [i for name, i in site.items() if "resident" in name]
    assert len(site_resident) == 1, site

    def resident_launches():
        capi.call("wd_profile_flush_token")
        st, tokens = capi.ProfileSiteStat(), C.c_ulonglong()
        capi.call("wd_profile_site", site_resident[0], C.byref(st), C.byref(tokens))
        return st.calls

    capi.call("wd_profile_enable", 1)
    capi.call("wd_profile_reset")
    try:
        x0 = synth.rms_normed(synth.rng_for(SEED, 83, 0), 2048)
        _run_stack(g, arr, nl, x0, None, sc_a, 0)
        assert resident_launches() == 1
        _run_stack(g, arr, nl, x0, None, sc_b, PER_LAYER)
        assert resident_launches() == 1
    finally:
        capi.call("wd_profile_enable", 0)
        capi.call("wd_profile_reset")
    for token, depth in enumerate([nl, 2, nl, nl, min(3, nl), nl, 1, 1]):
        x = synth.rms_normed(synth.rng_for(SEED, 84, token), 2048)
        tr = None
        if token % 2 == 1:
            tr = np.stack([rng.choice(experts, size=k, replace=False) for _ in range(depth)]).astype(np.int32)
        got = _run_stack(g, arr, depth, x, tr, sc_a, 0)
        want = _run_stack(g, arr, depth, x, tr, sc_b, PER_LAYER)
        assert g.same_bits(got[0], want[0]) and g.same_bits(got[1], want[1]), (token, depth)
        for name, _, dt in VIEWS:
            if name in ("down_f32", "shared_gate") and not shared:
                continue
            assert np.array_equal(got[2][name].view(np.uint32), want[2][name].view(np.uint32)), (token, name)
        if token < 2:
            wx = x.copy()
            for l, L in enumerate(Ls[:depth]):
                if tr is None:
                    wout, _ = oracle.moe_layer(L, wx)
                else:
                    _, wts = oracle.route(oracle.router_logits(L["router"], wx), k)
                    wout, _ = oracle.moe_layer(L, wx, ids=tr[l], weights=wts)
                wx = (wx + (wout * np.float32(2.0 ** -12)).astype(np.float32)).astype(np.float32)
            assert g.same_bits(got[0], wx) and g.same_bits(got[1], wout), token
    assert capi.load().wd_moe_scratch_status(sc_a.h) == 0
    sc_a.close()
    sc_b.close()


# 150 slots hold three tokens' experts (a token's fills run beside the launch of the token before), 100 two tokens'
# (they wait for it); 320 (layer, expert) pairs compete for them
@pytest.mark.parametrize("slots", [150, 100], ids=["three-tokens-of-slots", "two-tokens-of-slots"])
def test_one_launch_stack_fed_from_the_slot_cache(g, oracle, slots):
    """The stack whose routed experts live in pinned host memory behind the slot pool, routing trace known to the host:
    one resident launch per token (the cache's counter says so), fills landing while it runs, against the all-resident
    stack on the same trace - outputs and the last layer's views bit for bit - and, with WD_MOE_PER_LAYER, the same
    through the per-layer dispatches."""
    import json
    import torch
    experts, k, nl, tokens = 64, 10, 5, 8
    Ls = [synth.make_layer(2048, 512, experts, k, synth.IQ3_S, synth.Q8_0, shared=True, layer=500 + l,
                           router_sigma=1.0 / np.sqrt(2048.0)) for l in range(nl)]
    gb, db = 512 * synth.row_bytes(synth.IQ3_S, 2048), 2048 * synth.row_bytes(synth.Q8_0, 512)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), slots * (2 * gb + db), gb, gb, db, nl, experts, 0)
    pinned = []
    for l, L in enumerate(Ls):
        p = [torch.from_numpy(np.ascontiguousarray(L[n]).reshape(-1)).pin_memory() for n in ("gate", "up", "down")]
        pinned.append(p)
        capi.call("wd_expert_cache_register_layer", cache, l, *[C.c_void_p(t.data_ptr()) for t in p])
    dls, arr = _descs(g, Ls)
    dls_bare, bare = _descs(g, Ls)   # (kept: the descriptors point into these tensors)
    for i in range(nl):                      # the routed tensors live only in the cache
        bare[i].gate = bare[i].up = bare[i].down = None
    sc_a, sc_b = g.Scratch(2048, 512, experts, k), g.Scratch(2048, 512, experts, k)
    rng = np.random.default_rng(SEED + 500)

    def counter():
        lib = capi.load()
        need = lib.wd_expert_cache_dump_json(cache, None, 0)
        buf = C.create_string_buffer(need + 1)
        lib.wd_expert_cache_dump_json(cache, buf, need + 1)
        return json.loads(buf.value.decode())["tokens_in_one_launch"]

    for token in range(tokens):
        x = synth.rms_normed(synth.rng_for(SEED, 86, token), 2048)
        tr = np.stack([rng.choice(experts, size=k, replace=False) for _ in range(nl)]).astype(np.int32)
        flags = PER_LAYER if token == tokens - 1 else 0
        dx, out, dtr = g.dev(x), g.empty(2048, np.float32), g.dev(tr)
        capi.call("wd_moe_stack_cached_f32", bare, nl, cache, g.ptr(dx), g.ptr(out), sc_a.h, tr.ctypes.data_as(C.c_void_p),
                  g.ptr(dtr), float(2.0 ** -12), flags, g.stream())
        g.sync()
        views = {name: sc_a.get(name, {"k": k, "E": experts, "H": 2048}.get(n_, n_), dt) for name, n_, dt in VIEWS}
        want = _run_stack(g, arr, nl, x, tr, sc_b, PER_LAYER)
        assert g.same_bits(g.host(dx), want[0]) and g.same_bits(g.host(out), want[1]), token
        for name, _, dt in VIEWS:
            assert np.array_equal(views[name].view(np.uint32), want[2][name].view(np.uint32)), (token, name)
        assert counter() == min(token + 1, tokens - 1), token
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert st.accesses == tokens * nl * k and st.evictions > 0 and st.resident <= slots
    assert capi.load().wd_moe_scratch_status(sc_a.h) == 0
    sc_a.close()
    sc_b.close()
    capi.call("wd_expert_cache_destroy", cache)


def test_one_launch_stack_wait_that_runs_out(g):
    """A wait limit of one poll: the launch ends normally with the status word set and NaN in its outputs; the next call
    on that scratch is refused by the host (the status word has a mirror in host memory), a replay of a graph recorded
    earlier returns NaN at once; after the reset the results are right again."""
    import torch
    Ls = [synth.make_c2(layer=320 + l, n_experts=64) for l in range(3)]
    dls, arr = _descs(g, Ls)
    sc, ref = g.Scratch(2048, 512, 64, 10), g.Scratch(2048, 512, 64, 10)
    x = synth.rms_normed(synth.rng_for(SEED, 85), 2048)
    want = _run_stack(g, arr, 3, x, None, ref, PER_LAYER)
    # a graph of the launch, recorded while all is well
    d_x, d_out = g.dev(x), g.empty(2048, np.float32)

    def launch():
        capi.call("wd_moe_stack_f32", arr, 3, g.ptr(d_x), g.ptr(d_out), sc.h, None, float(2.0 ** -12), 0,
                  C.c_void_p(torch.cuda.current_stream().cuda_stream))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert g.same_bits(g.host(d_x), want[0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    capi.call("wd_moe_scratch_set_wait_limit", sc.h, 1)
    bad = _run_stack(g, arr, 3, x, None, sc, 0)
    assert capi.load().wd_moe_scratch_status(sc.h) == 1
    assert np.isnan(bad[0]).all() and np.isnan(bad[1]).all()   # the failure is in the data too
    dx, out = g.dev(x), g.empty(2048, np.float32)
    rc = capi.load().wd_moe_stack_f32(arr, 3, g.ptr(dx), g.ptr(out), sc.h, None, float(2.0 ** -12), 0, g.stream())
    assert rc == -3 and "ran out" in capi.load().wd_last_error().decode()   # WD_ERR_STATE: refused by the host
    d_x.copy_(torch.from_numpy(x).cuda())
    graph.replay()                                   # refused on the device: nothing waits
    g.sync()
    assert np.isnan(g.host(d_x)).all() and np.isnan(g.host(d_out)).all()
    assert capi.load().wd_moe_scratch_status(sc.h) == 1
    capi.call("wd_moe_scratch_set_wait_limit", sc.h, 0)
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    for _ in range(3):
        got = _run_stack(g, arr, 3, x, None, sc, 0)
        assert g.same_bits(got[0], want[0]) and g.same_bits(got[1], want[1])
    d_x.copy_(torch.from_numpy(x).cuda())
    graph.replay()
    g.sync()
    assert g.same_bits(g.host(d_x), want[0]) and g.same_bits(g.host(d_out), want[1])
    sc.close()
    ref.close()


def test_one_launch_stack_keeps_the_descriptors_of_a_recorded_graph(g):
    """A graph recorded for one stack still computes that stack after the same scratch has run another one: every stack a
    scratch has seen keeps a device copy of its layer descriptors of its own."""
    import torch
    Ls = [synth.make_c2(layer=330 + l, n_experts=64) for l in range(4)]
    dls, arr = _descs(g, Ls)
    other = (capi.MoeLayer * 2)(arr[3], arr[2])
    sc, ref = g.Scratch(2048, 512, 64, 10), g.Scratch(2048, 512, 64, 10)
    x = synth.rms_normed(synth.rng_for(SEED, 86), 2048)
    want = _run_stack(g, arr, 2, x, None, ref, PER_LAYER)
    want_other = _run_stack(g, other, 2, x, None, ref, PER_LAYER)
    d_x, d_out = g.dev(x), g.empty(2048, np.float32)

    def launch():
        capi.call("wd_moe_stack_f32", arr, 2, g.ptr(d_x), g.ptr(d_out), sc.h, None, float(2.0 ** -12), 0,
                  C.c_void_p(torch.cuda.current_stream().cuda_stream))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    got_other = _run_stack(g, other, 2, x, None, sc, 0)     # another stack on the same scratch, eagerly
    assert g.same_bits(got_other[0], want_other[0]) and g.same_bits(got_other[1], want_other[1])
    d_x.copy_(torch.from_numpy(x).cuda())
    graph.replay()
    g.sync()
    assert g.same_bits(g.host(d_x), want[0]) and g.same_bits(g.host(d_out), want[1])
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    sc.close()
    ref.close()
