"""Layers built from a GGUF model file on the GPU: the tensors are found by name in a file written with the numpy
writer, parsed by the library's reader and used as they lie in the mapping - uploaded for the resident stack, or
registered as the expert cache's host source (separate gate/up tensors and the fused gate_up layout) - and the stack
results are compared bit for bit with the CPU oracle run on the arrays the file was written from."""
import ctypes as C

import numpy as np
import pytest

from warpdecode_amd import capi, ggufio, synth

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
    return [synth.make_layer(H, F, E, K, synth.IQ3_S, synth.Q8_0, shared=True, layer=140 + l,
                             router_sigma=1.0 / np.sqrt(H)) for l in range(NL)]


def _write(tmp_path, layers, fused):
    path = tmp_path / ("fused.gguf" if fused else "separate.gguf")
    tensors = sum((ggufio.layer_tensors(L, l, fused_gate_up=fused) for l, L in enumerate(layers)), [])
    meta = [("general.architecture", ggufio.STRING, "qwen38"), ("qwen38.block_count", ggufio.U32, NL),
            ("qwen38.embedding_length", ggufio.U32, H), ("qwen38.expert_feed_forward_length", ggufio.U32, F),
            ("qwen38.expert_count", ggufio.U32, E), ("qwen38.expert_used_count", ggufio.U32, K)]
    ggufio.write_gguf(path, tensors, meta)
    return path


def _layer_from_file(gf, il):
    """A synth-style layer dict whose arrays are views of the mapping."""
    p = "blk.%d." % il
    t = gf.tensors
    hidden, n_exp = t[p + "ffn_gate_inp.weight"]["dims"]
    ffn = t[p + "ffn_down_exps.weight"]["dims"][0]
    L = dict(hidden=hidden, expert_ffn=ffn, n_experts=n_exp, top_k=int(gf.number("qwen38.expert_used_count")), w_scale=1.0,
             down_type=t[p + "ffn_down_exps.weight"]["type"], shared_type=t[p + "ffn_gate_shexp.weight"]["type"])
    L["router"] = gf.bytes_of(p + "ffn_gate_inp.weight").view(np.float32).reshape(n_exp, hidden)
    L["down"] = gf.bytes_of(p + "ffn_down_exps.weight").reshape(n_exp, -1)
    if p + "ffn_gate_up_exps.weight" in t:
        both = gf.bytes_of(p + "ffn_gate_up_exps.weight").reshape(n_exp, -1)
        half = both.shape[1] // 2
        L["gate_type"] = L["up_type"] = t[p + "ffn_gate_up_exps.weight"]["type"]
        L["gate"], L["up"] = both[:, :half], both[:, half:]
        L["gate_up_stride"] = both.shape[1]
    else:
        L["gate_type"], L["up_type"] = t[p + "ffn_gate_exps.weight"]["type"], t[p + "ffn_up_exps.weight"]["type"]
        L["gate"] = gf.bytes_of(p + "ffn_gate_exps.weight").reshape(n_exp, -1)
        L["up"] = gf.bytes_of(p + "ffn_up_exps.weight").reshape(n_exp, -1)
    L["shared_gate_inp"] = gf.bytes_of(p + "ffn_gate_inp_shexp.weight").view(np.float32)
    for n in ("gate", "up", "down"):
        L["shared_" + n] = gf.bytes_of(p + "ffn_%s_shexp.weight" % n)
    return L


def _oracle_stack(oracle, layers, x):
    x = x.copy()
    out = None
    for L in layers:
        out, _ = oracle.moe_layer(L, x)
        x = (x + (out * SCALE).astype(np.float32)).astype(np.float32)
    return x, out


def _descs(g, Ls):
    dls = [g.DeviceLayer({k: (np.ascontiguousarray(v) if isinstance(v, np.ndarray) else v) for k, v in L.items()})
           for L in Ls]
    arr = (capi.MoeLayer * len(Ls))()
    for i, dl in enumerate(dls):
        arr[i] = dl.desc
    return dls, arr


@pytest.mark.parametrize("fused", [False, True], ids=["separate", "gate_up"])
def test_resident_stack_from_file(g, oracle, layers, tmp_path, fused):
    with ggufio.GgufFile(_write(tmp_path, layers, fused)) as gf:
        assert gf.number("qwen38.block_count") == NL
        Ls = [_layer_from_file(gf, l) for l in range(NL)]
        assert Ls[0]["hidden"] == H and Ls[0]["expert_ffn"] == F and Ls[0]["n_experts"] == E and Ls[0]["top_k"] == K
        dls, arr = _descs(g, Ls)
    sc = g.Scratch(H, F, E, K)           # the file is closed: the uploaded copies are all the stack needs
    for step in range(2):
        x = synth.rms_normed(synth.rng_for(SEED, 141, step), H)
        dx, out = g.dev(x), g.empty(H, np.float32)
        capi.call("wd_moe_stack_f32", arr, NL, g.ptr(dx), g.ptr(out), sc.h, None, float(SCALE), 0, g.stream())
        g.sync()
        wx, wout = _oracle_stack(oracle, layers, x)
        assert g.same_bits(g.host(dx), wx), step
        assert g.same_bits(g.host(out), wout), step
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    sc.close()


@pytest.mark.parametrize("attach", ["no", "before", "after", "found"],
                         ids=["pageable", "pread-attached-first", "pread-attached-late", "pread-found-in-proc-maps"])
@pytest.mark.parametrize("fused", [False, True], ids=["separate", "gate_up"])
def test_cached_stack_streams_experts_from_the_mapping(g, oracle, layers, tmp_path, fused, attach):
    """attach = no: the mapping is a pageable host source (hipMemcpyAsync per piece); otherwise the file is attached to
    the cache (named by the caller, or found by the cache itself through /proc/self/maps) and misses are read with pread()
    into the pinned ring (three reader threads), one DMA per miss."""
    import json
    gb = F * synth.row_bytes(synth.IQ3_S, H)
    db = H * synth.row_bytes(synth.Q8_0, F)
    slots = 20
    with ggufio.GgufFile(_write(tmp_path, layers, fused)) as gf:
        Ls = [_layer_from_file(gf, l) for l in range(NL)]
        cache = C.c_void_p()
        capi.call("wd_expert_cache_create", C.byref(cache), slots * (2 * gb + db), gb, gb, db, NL, E, 0)
        if attach == "before":
            capi.call("wd_expert_cache_attach_file", cache, C.c_void_p(gf.map_base), gf.map_bytes, gf.fd, 3)
        for l, L in enumerate(Ls):
            ptr = lambda a: C.c_void_p(a.ctypes.data)
            if fused:
                capi.call("wd_expert_cache_register_layer_strided", cache, l, ptr(L["gate"]), ptr(L["up"]), ptr(L["down"]),
                          L["gate_up_stride"], L["gate_up_stride"], db)
            else:
                capi.call("wd_expert_cache_register_layer", cache, l, ptr(L["gate"]), ptr(L["up"]), ptr(L["down"]))
        if attach == "after":
            capi.call("wd_expert_cache_attach_file", cache, C.c_void_p(gf.map_base), gf.map_bytes, gf.fd, 3)
        if attach == "found":
            n = C.c_int(0)
            capi.call("wd_expert_cache_attach_mappings", cache, 3, C.byref(n))
            assert n.value == 1          # one file holds every tensor
            capi.call("wd_expert_cache_attach_mappings", cache, 3, C.byref(n))
            assert n.value == 0          # nothing new the second time
        dls, arr = _descs(g, [dict(L, gate=L["gate"][:1], up=L["up"][:1], down=L["down"][:1]) for L in Ls])
        for i in range(NL):                  # routed tensors come from the cache only
            arr[i].gate = arr[i].up = arr[i].down = None
        sc = g.Scratch(H, F, E, K)
        for step in range(4):
            x = synth.rms_normed(synth.rng_for(SEED, 142, step), H)
            dx, out = g.dev(x), g.empty(H, np.float32)
            capi.call("wd_moe_stack_cached_f32", arr, NL, cache, g.ptr(dx), g.ptr(out), sc.h, None, None, float(SCALE), 0,
                      g.stream())
            g.sync()
            wx, wout = _oracle_stack(oracle, layers, x)
            assert g.same_bits(g.host(dx), wx), step
            assert g.same_bits(g.host(out), wout), step
        st = capi.CacheStats()
        capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
        assert st.accesses == 4 * NL * K and st.misses > 0 and st.bytes_copied == st.misses * (2 * gb + db)
        buf = C.create_string_buffer(1 << 16)
        capi.load().wd_expert_cache_dump_json(cache, buf, len(buf))
        mon = json.loads(buf.value.decode())
        if attach == "no":
            assert mon["fills_by_memcpy"] == st.misses and mon["fills_by_pread"] == 0
        else:
            assert mon["fills_by_pread"] == st.misses and mon["fills_by_memcpy"] == 0 and mon["fills_by_copy_kernel"] == 0
        sc.close()
        capi.call("wd_expert_cache_destroy", cache)


@pytest.mark.parametrize("depth", [1, 2])
def test_read_ahead_serves_router_driven_misses(g, oracle, layers, tmp_path, depth):
    """No trace known to the host: every layer's selection comes back from the device before its experts are acquired.
    With read-ahead on, the experts the previous token took are read from the file while the layers compute, and a miss
    that was predicted is filled from the ring.  The pool (8 slots for 3 layers x 4 experts per token) cannot keep a
    token's experts until the next token, so a token that repeats the previous input misses everywhere and every
    prediction comes true.  Whatever the source of a fill, the results are the oracle's."""
    import json
    gb = F * synth.row_bytes(synth.IQ3_S, H)
    db = H * synth.row_bytes(synth.Q8_0, F)
    with ggufio.GgufFile(_write(tmp_path, layers, False)) as gf:
        Ls = [_layer_from_file(gf, l) for l in range(NL)]
        cache = C.c_void_p()
        capi.call("wd_expert_cache_create", C.byref(cache), 8 * (2 * gb + db), gb, gb, db, NL, E, 0)
        capi.call("wd_expert_cache_attach_file", cache, C.c_void_p(gf.map_base), gf.map_bytes, gf.fd, 2)
        for l, L in enumerate(Ls):
            ptr = lambda a: C.c_void_p(a.ctypes.data)
            capi.call("wd_expert_cache_register_layer", cache, l, ptr(L["gate"]), ptr(L["up"]), ptr(L["down"]))
        capi.call("wd_expert_cache_set_read_ahead", cache, depth, 0)
        dls, arr = _descs(g, [dict(L, gate=L["gate"][:1], up=L["up"][:1], down=L["down"][:1]) for L in Ls])
        for i in range(NL):
            arr[i].gate = arr[i].up = arr[i].down = None
        sc = g.Scratch(H, F, E, K)
        lib = capi.load()
        xs = [synth.rms_normed(synth.rng_for(SEED, 143, i // 2), H) for i in range(8)]     # every input twice in a row
        for step, x in enumerate(xs):
            dx, out = g.dev(x), g.empty(H, np.float32)
            capi.call("wd_moe_stack_cached_f32", arr, NL, cache, g.ptr(dx), g.ptr(out), sc.h, None, None, float(SCALE), 0, g.stream())
            g.sync()
            wx, wout = _oracle_stack(oracle, layers, x)
            assert g.same_bits(g.host(dx), wx), step
            assert g.same_bits(g.host(out), wout), step
            import time
            time.sleep(0.05)         # the reader works in the background: give it the time a real layer stack would
        buf = C.create_string_buffer(1 << 16)
        lib.wd_expert_cache_dump_json(cache, buf, len(buf))
        mon = json.loads(buf.value.decode())
        ra = mon["read_ahead"]
        assert ra["depth"] == depth and ra["slots"] == 16 * depth
        assert ra["posted"] > 0 and ra["delivered"] > 0 and ra["failed"] == 0
        assert ra["fills"] > 0, ra                                           # predictions that came true were served from the ring
        assert ra["fills"] + mon["fills_by_pread"] == mon["misses"]          # every other miss took the on-demand path
        capi.call("wd_expert_cache_set_read_ahead", cache, 0, 0)             # off again: the ring is released
        dx, out = g.dev(xs[0]), g.empty(H, np.float32)
        capi.call("wd_moe_stack_cached_f32", arr, NL, cache, g.ptr(dx), g.ptr(out), sc.h, None, None, float(SCALE), 0, g.stream())
        g.sync()
        assert g.same_bits(g.host(out), _oracle_stack(oracle, layers, xs[0])[1])
        assert lib.wd_expert_cache_set_read_ahead(cache, 9, 0) == -1
        sc.close()
        capi.call("wd_expert_cache_destroy", cache)
