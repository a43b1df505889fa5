"""Site profiler on the GPU: which brackets fire on the fused, staged and cached paths of a small stack, that the
totals nest (a stack's device time holds its layers', a layer's holds its dispatches'), that a profiled pass gives
the bits of an unprofiled one, and the bookkeeping of the reference's profiler (src/qwen38_moe.cuh:296-535: nested
brackets of a site count once, a site without room reports dropped brackets, a bracket on a capturing stream is
not recorded)."""
import ctypes as C

import numpy as np
import pytest

from warpdecode_amd import capi, synth

pytestmark = pytest.mark.gpu
SEED = 20261103
H, F, E, K, NL = 512, 128, 32, 4, 3
SCALE = np.float32(2.0 ** -6)
SITES = {}


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


@pytest.fixture()
def prof():
    lib = capi.load()
    SITES.update({lib.wd_profile_site_name(i).decode(): i for i in range(64) if lib.wd_profile_site_name(i) != b"unknown"})
    capi.call("wd_profile_enable", 1)
    capi.call("wd_profile_reset")
    try:
        yield
    finally:
        capi.call("wd_profile_enable", 0)
        capi.call("wd_profile_reset")


def stat(name):
    st, tokens = capi.ProfileSiteStat(), C.c_ulonglong()
    capi.call("wd_profile_site", SITES[name], C.byref(st), C.byref(tokens))
    return st, tokens.value


def report():
    lib = capi.load()
    need = lib.wd_profile_report(None, 0)
    buf = C.create_string_buffer(need + 1)
    lib.wd_profile_report(buf, need + 1)
    return buf.value.decode()


def _stack(g, flags, tokens, layers, arr, sc):
    outs = []
    for t in range(tokens):
        x = synth.rms_normed(synth.rng_for(SEED, 1, t), H)
        dx, out = g.dev(x), g.empty(H, np.float32)
        capi.call("wd_moe_stack_f32", arr, NL, g.ptr(dx), g.ptr(out), sc.h, None, float(SCALE), flags, g.stream())
        g.sync()
        capi.call("wd_profile_flush_token")
        outs.append((g.host(dx).copy(), g.host(out).copy()))
    return outs


def _make(g):
    layers = [synth.make_layer(H, F, E, K, synth.IQ3_S, synth.Q8_0, shared=True, layer=40 + l,
                               router_sigma=1.0 / np.sqrt(H)) for l in range(NL)]
    dls = [g.DeviceLayer(L) for L in layers]
    arr = (capi.MoeLayer * NL)()
    for i, dl in enumerate(dls):
        arr[i] = dl.desc
    return layers, dls, arr


def test_sites_of_the_fused_and_the_staged_stack(g, prof):
    layers, dls, arr = _make(g)
    sc = g.Scratch(H, F, E, K)
    T = 3
    capi.call("wd_profile_enable", 0)
    plain = _stack(g, 0, T, layers, arr, sc)
    capi.call("wd_profile_enable", 1)
    capi.call("wd_profile_reset")
    got = _stack(g, 0, T, layers, arr, sc)
    for (ax, ao), (bx, bo) in zip(plain, got):
        assert g.same_bits(ax, bx) and g.same_bits(ao, bo)
    total, tokens = stat("moe.stack_total")
    layer, _ = stat("moe.routed_total")
    ab, _ = stat("moe.fused.ab")
    c, _ = stat("moe.fused.c")
    assert tokens == T
    assert (total.calls, layer.calls, ab.calls, c.calls) == (T, T * NL, T * NL, T * NL)
    for s in (total, layer, ab, c):
        assert s.recorded == s.calls and s.dropped == 0 and s.unreadable == 0 and s.device_ms > 0 and s.host_ms > 0
    # the brackets nest on one stream: an outer interval holds the inner ones
    assert total.device_ms >= 0.99 * layer.device_ms >= 0.98 * (ab.device_ms + c.device_ms)
    assert total.host_ms >= layer.host_ms >= ab.host_ms
    for name in ("moe.router.gemv", "moe.batch.gate_up", "moe.stack.resident", "moe.acquire"):
        assert stat(name)[0].recorded == 0
    text = report()
    assert text.startswith("[moe-profile] tokens=3 unit=ms_per_token\n")
    line = next(l for l in text.splitlines() if "moe.fused.ab" in l)
    assert "calls/token=3.00" in line and "recorded=9 dropped=0 evfail=0" in line
    assert "moe.router.gemv" not in text

    # one dispatch per operator: the reference's own stages
    capi.call("wd_profile_reset")
    staged = _stack(g, 4, T, layers, arr, sc)
    for (ax, ao), (bx, bo) in zip(plain, staged):
        assert g.same_bits(ax, bx) and g.same_bits(ao, bo)
    for name in ("moe.router.gemv", "moe.router.topk", "moe.rx_quant", "moe.batch.gate_up", "moe.batch.silu",
                 "moe.batch.q8_quant", "moe.batch.down", "moe.batch.accum"):
        s, _ = stat(name)
        assert s.calls == T * NL and s.device_ms > 0, name
    assert stat("moe.shared")[0].calls == 2 * T * NL      # its gate/up rows, then its down rows
    assert stat("moe.fused.ab")[0].recorded == 0
    parts = sum(stat(n)[0].device_ms for n in SITES if n.startswith(("moe.router.", "moe.batch.")) or n in ("moe.rx_quant", "moe.shared"))
    assert stat("moe.routed_total")[0].device_ms >= 0.98 * parts
    sc.close()


def test_sites_of_the_cached_stack(g, prof):
    import torch
    layers, dls, arr = _make(g)
    gb = F * synth.row_bytes(synth.IQ3_S, H)
    db = H * synth.row_bytes(synth.Q8_0, F)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), 20 * (2 * gb + db), gb, gb, db, NL, E, 0)
    pinned = []
    for l, L in enumerate(layers):
        p = [torch.from_numpy(np.ascontiguousarray(L[n]).reshape(-1)).pin_memory() for n in ("gate", "up", "down")]
        pinned.append(p)
        capi.call("wd_expert_cache_register_layer", cache, l, *[C.c_void_p(t.data_ptr()) for t in p])
    for i in range(NL):
        arr[i].gate = arr[i].up = arr[i].down = None
    sc = g.Scratch(H, F, E, K)
    T = 4
    for t in range(T):     # router-driven: ids to the host, acquire, expert dispatches - the reference's loop
        x = synth.rms_normed(synth.rng_for(SEED, 2, t), H)
        dx, out = g.dev(x), g.empty(H, np.float32)
        capi.call("wd_moe_stack_cached_f32", arr, NL, cache, g.ptr(dx), g.ptr(out), sc.h, None, None, float(SCALE), 0, g.stream())
        g.sync()
        capi.call("wd_device_sync")        # the fills' brackets are on the cache's own stream
        capi.call("wd_profile_flush_token")
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    for name in ("moe.router_select", "moe.router.d2h", "moe.router.sync", "moe.acquire", "moe.fused.a", "moe.fused.b", "moe.fused.c"):
        s, _ = stat(name)
        assert s.calls == T * NL and s.dropped == 0, name
    sel, d2h, syn, a = (stat(n)[0] for n in ("moe.router_select", "moe.router.d2h", "moe.router.sync", "moe.fused.a"))
    assert sel.host_ms >= syn.host_ms > 0 and sel.device_ms >= 0.98 * (a.device_ms + d2h.device_ms)
    fills, _ = stat("moe.cache.fill")
    assert 0 < fills.calls <= T * NL and st.misses > 0 and fills.device_ms > 0
    assert stat("moe.stack_total")[0].calls == T
    sc.close()
    capi.call("wd_expert_cache_destroy", cache)


def test_bookkeeping_of_caller_brackets(g, prof):
    site = SITES["moe.stage_total"]
    st = g.stream()
    # nested brackets of one site are one interval
    for _ in range(2):
        capi.call("wd_profile_begin", site, st)
    for _ in range(2):
        capi.call("wd_profile_end", site, st)
    capi.call("wd_profile_end", site, st)          # an end without a begin is ignored
    g.sync()
    capi.call("wd_profile_flush_token")
    s, tokens = stat("moe.stage_total")
    assert (s.calls, s.recorded, s.dropped, tokens) == (1, 1, 0, 1) and s.device_ms >= 0
    # more brackets in one token than a site has room for
    capi.call("wd_profile_reset")
    for _ in range(170):
        capi.call("wd_profile_begin", site, st)
        capi.call("wd_profile_end", site, st)
    g.sync()
    capi.call("wd_profile_flush_token")
    s, _ = stat("moe.stage_total")
    assert s.recorded == s.calls and s.recorded + s.dropped == 170 and 0 < s.dropped <= 42
    assert "dropped=%d" % s.dropped in report()
    # the next token has room again
    capi.call("wd_profile_begin", site, st)
    capi.call("wd_profile_end", site, st)
    g.sync()
    capi.call("wd_profile_flush_token")
    assert stat("moe.stage_total")[0].recorded == s.recorded + 1
    # switched off, the hooks do nothing
    capi.call("wd_profile_enable", 0)
    capi.call("wd_profile_begin", site, st)
    capi.call("wd_profile_end", site, st)
    capi.call("wd_profile_flush_token")
    assert stat("moe.stage_total")[0].recorded == s.recorded + 1 and stat("moe.stage_total")[1] == 2


def test_brackets_on_a_capturing_stream_are_dropped(g, prof):
    import torch
    layers, dls, arr = _make(g)
    sc = g.Scratch(H, F, E, K)
    d_x = torch.zeros(H, dtype=torch.float32, device="cuda")
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")

    def launch():
        capi.call("wd_moe_layer_f32", C.byref(arr[0]), g.ptr(d_x), g.ptr(d_out), sc.h, 0,
                  C.c_void_p(torch.cuda.current_stream().cuda_stream))

    x = synth.rms_normed(synth.rng_for(SEED, 3, 0), H)
    d_x.copy_(torch.from_numpy(x).cuda())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = d_out.cpu().numpy().copy()
    capi.call("wd_profile_flush_token")
    before = stat("moe.fused.ab")[0]
    assert before.recorded == 1 and before.dropped == 0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for _ in range(3):
        d_out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert g.same_bits(d_out.cpu().numpy(), want)
    capi.call("wd_profile_flush_token")
    after = stat("moe.fused.ab")[0]
    assert after.recorded == 1 and after.dropped == 1 and after.unreadable == 0
    sc.close()
