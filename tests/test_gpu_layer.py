"""GPU parity of the whole MoE layer against the CPU oracle: routed ids, router weights, the int32
chunk sums of every selected expert's gate/up/down projection, and the f32 layer output."""
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


def run_layer(g, L, x, partials=True, flags=0, ids=None, weights=None):
    H, F, E, k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
    dl = g.DeviceLayer(L)
    sc = g.Scratch(H, F, E, k)
    if partials:
        capi.call("wd_moe_scratch_enable_partials", sc.h, L["gate_type"], L["down_type"])
    if ids is not None:
        capi.call("wd_memcpy_h2d", C.c_void_p(sc.raw("ids")), np.asarray(ids, np.int32).ctypes.data_as(C.c_void_p),
                  4 * k, None)
        capi.call("wd_memcpy_h2d", C.c_void_p(sc.raw("weights")),
                  np.asarray(weights, np.float32).ctypes.data_as(C.c_void_p), 4 * k, None)
    dx, out = g.dev(x), g.empty(H, np.float32)
    capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream())
    g.sync()
    res = dict(out=g.host(out), ids=sc.get("ids", k, np.int32), weights=sc.get("weights", k, np.float32),
               logits=sc.get("logits", E, np.float32), accum=sc.get("accum", H, np.float32),
               act=sc.get("act", k * F, np.float32).reshape(k, F),
               act_qs=sc.get("act_qs", k * F, np.int8).reshape(k, F),
               act_d=sc.get("act_scales", k * (F // 32), np.uint16).reshape(k, F // 32))
    if L.get("shared_gate_inp") is not None:
        res["shared_gate"] = sc.get("shared_gate", 1, np.float32)
        res["down_f32"] = sc.get("down_f32", H, np.float32)
    if partials:
        from oracle import pyoracle
        pg, pd = pyoracle.partials_per_row(L["gate_type"], H), pyoracle.partials_per_row(L["down_type"], F)
        res["gate_up_partials"] = sc.get("gate_up_partials", k * 2 * F * pg, np.int32).reshape(k, 2, F, pg)
        res["down_partials"] = sc.get("down_partials", k * H * pd, np.int32).reshape(k, H, pd)
    sc.close()
    return res


def check_layer(g, oracle, L, x, **kw):
    """Three passes against the oracle: the fused dispatches, the fused dispatches with the int32 chunk sums
    exported (layers whose gate rows are not of a kind the fused kernels export take the staged dispatches for
    this by themselves), and the staged dispatches (one per operator, which also leave the quantised activation
    in the scratch)."""
    want, d = oracle.moe_layer(L, x, ids=kw.get("ids"), weights=kw.get("weights"), want_partials=True)
    base = kw.pop("flags", 0)
    for partials, flags in ((False, base), (True, base), (True, base | capi.MOE_STAGED)):
        got = run_layer(g, L, x, partials=partials, flags=flags, **kw)
        assert np.array_equal(got["ids"], d["ids"])
        assert g.same_bits(got["weights"], d["weights"])
        if kw.get("ids") is None:
            assert g.same_bits(got["logits"], d["logits"])
        assert g.same_bits(got["act"], d["act"])
        assert g.same_bits(got["accum"], d["routed"])
        if partials:
            assert np.array_equal(got["gate_up_partials"], d["gate_up_partials"])
            assert np.array_equal(got["down_partials"], d["down_partials"])
        if flags & capi.MOE_STAGED:
            assert np.array_equal(got["act_qs"], d["act_qs"]) and np.array_equal(got["act_d"], d["act_d"])
        if L.get("shared_gate_inp") is not None:
            assert g.same_bits(got["shared_gate"], d["shared_gate"])
            assert g.same_bits(got["down_f32"], d["shared_out"])
        assert g.same_bits(got["out"], want)
    rel = np.linalg.norm(got["out"] - want) / max(np.linalg.norm(want), 1e-30)
    assert rel <= 1e-5
    return got


@pytest.mark.parametrize("gate_t,down_t,shared", [(synth.IQ3_S, synth.Q8_0, True), (synth.Q8_0, synth.Q8_0, False),
                                                   (synth.IQ2_S, synth.IQ4_NL, True), (synth.IQ3_S, synth.IQ4_NL, False)])
def test_small_layers(g, oracle, gate_t, down_t, shared):
    for H, F, E, k in [(512, 64, 8, 2), (768, 96, 16, 4), (256, 32, 8, 8)]:
        L = synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=SEED, layer=H + k,
                             router_sigma=1.0 / np.sqrt(H))
        x = synth.rms_normed(synth.rng_for(SEED, 41, H), H)
        check_layer(g, oracle, L, x)


@pytest.mark.parametrize("gate_t,down_t", [(synth.IQ2_S, synth.IQ4_NL), (synth.IQ3_S, synth.Q8_0), (synth.Q8_0, synth.Q8_0)])
def test_model_shape_layers(g, oracle, gate_t, down_t):
    """Hidden 2560 / ffn 640 (the shapes of the reference's target model, src/qwen38_moe.cuh:3462-3514): rows
    longer than one 2048-column span in the router and in the Q8_0 row kernels, ffn not a power of two."""
    H, F, E, k = 2560, 640, 32, 6
    L = synth.make_layer(H, F, E, k, gate_t, down_t, True, seed=SEED, layer=77, router_sigma=1.0 / np.sqrt(H))
    x = synth.rms_normed(synth.rng_for(SEED, 49), H)
    check_layer(g, oracle, L, x)


@pytest.mark.parametrize("H,F,gate_t,down_t,shared", [(2048, 512, synth.IQ3_S, synth.Q8_0, True),
                                                      (2560, 640, synth.IQ2_S, synth.IQ4_NL, True),
                                                      (1792, 512, synth.IQ3_S, synth.Q8_0, False),
                                                      (2048, 512, synth.Q8_0, synth.Q8_0, True)])
def test_more_routed_items_than_the_device_holds(g, oracle, H, F, gate_t, down_t, shared):
    """Top-16: 16 * ffn / 8 = 1024 or 1280 (rung, row group) items of routed gate/up work, more than the workgroups an
    MI355X holds at once, so the routed workgroups of the merged dispatch walk them in a loop; 17 matrices in the down
    dispatch (waves with two matrices each at hidden 2560, one of them without a second)."""
    E, k = 32, 16
    L = synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=SEED, layer=79, router_sigma=1.0 / np.sqrt(H))
    x = synth.rms_normed(synth.rng_for(SEED, 51, H), H)
    check_layer(g, oracle, L, x)


@pytest.mark.parametrize("H,F,E,k,gate_t,down_t,shared", [
    (256, 32, 8, 1, synth.IQ3_S, synth.Q8_0, False),          # the smallest layer the limits allow
    (256, 32, 1024, 16, synth.IQ2_S, synth.IQ4_NL, True),     # most experts, largest top-k
    (2560, 640, 8, 1, synth.IQ2_S, synth.IQ4_NL, False),      # one matrix in the down dispatch
    (2560, 640, 16, 2, synth.IQ3_S, synth.Q8_0, False),       # two: one paired wave
    (512, 32, 8, 8, synth.Q8_0, synth.Q8_0, True),            # every expert selected
    (3072, 96, 16, 4, synth.IQ3_S, synth.IQ4_NL, True),       # more than 2560 columns, odd number of down blocks
    (4096, 1024, 16, 4, synth.Q8_0, synth.Q8_0, True)])       # two full spans, down rows of 32 blocks
def test_corners_of_the_documented_limits(g, oracle, H, F, E, k, gate_t, down_t, shared):
    L = synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=SEED, layer=80 + k, router_sigma=1.0 / np.sqrt(H))
    x = synth.rms_normed(synth.rng_for(SEED, 52, H + E), H)
    check_layer(g, oracle, L, x)


@pytest.mark.parametrize("shared", [True, False])
def test_iq4_nl_down_rows_of_16_blocks(g, oracle, shared):
    """IQ4_NL down projection at ffn 512: the aligned fetch of four 16-block rows (with and without the Q8_0 shared
    expert, which takes the same routine)."""
    H, F, E, k = 2048, 512, 16, 5
    L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.IQ4_NL, shared, seed=SEED, layer=78, router_sigma=1.0 / np.sqrt(H))
    x = synth.rms_normed(synth.rng_for(SEED, 50), H)
    check_layer(g, oracle, L, x)


def test_c0_layer(g, oracle):
    """Workload C0: hidden 2048, 64 experts, top-8, ffn 512, all Q8_0."""
    L = synth.make_c0()
    for s in range(2):
        x = synth.rms_normed(synth.rng_for(SEED, 42, s), 2048)
        check_layer(g, oracle, L, x)


def test_c2_layer(g, oracle):
    """Workload C2: 512 experts, top-10, IQ3_S gate/up, Q8_0 down, shared expert."""
    L = synth.make_c2()
    for s in range(2):
        x = synth.rms_normed(synth.rng_for(SEED, 43, s), 2048)
        got = check_layer(g, oracle, L, x)
        assert len(set(got["ids"].tolist())) == 10 and abs(float(got["weights"].sum()) - 1.0) < 1e-5


def test_preselected(g, oracle):
    L = synth.make_c2(n_experts=64)
    x = synth.rms_normed(synth.rng_for(SEED, 44), 2048)
    ids = np.array([5, 63, 0, 17, 9, 33, 2, 41, 60, 12], np.int32)
    wts = np.full(10, 0.1, np.float32)
    check_layer(g, oracle, L, x, flags=capi.MOE_PRESELECTED, ids=ids, weights=wts)


def test_linearity_of_combine(g, oracle):
    """Size-independent property at full C2 size: with preselected ids the routed sum is the ordered
    weighted sum of single-expert passes (each run with weight 1)."""
    L = synth.make_c2(n_experts=128)
    x = synth.rms_normed(synth.rng_for(SEED, 45), 2048)
    ids = np.arange(10, dtype=np.int32) * 7
    wts = np.linspace(0.02, 0.18, 10).astype(np.float32)
    full = run_layer(g, L, x, partials=False, flags=capi.MOE_PRESELECTED, ids=ids, weights=wts)
    acc = np.zeros(2048, np.float32)
    L1 = dict(L); L1["top_k"] = 1
    for j in range(10):
        one = run_layer(g, L1, x, partials=False, flags=capi.MOE_PRESELECTED, ids=ids[j:j + 1],
                        weights=np.ones(1, np.float32))
        acc = (acc + (one["accum"] * wts[j]).astype(np.float32)).astype(np.float32)
    assert g.same_bits(acc, full["accum"])


def _fused_vs_oracle(g, oracle, L, x, flags=0):
    want, d = oracle.moe_layer(L, x)
    got = run_layer(g, L, x, partials=False, flags=flags)
    assert np.array_equal(got["ids"], d["ids"]), (got["ids"], d["ids"])
    assert g.same_bits(got["weights"], d["weights"])
    assert g.same_bits(got["logits"], d["logits"])
    assert g.same_bits(got["out"], want)


@pytest.mark.parametrize("flags", [0, 0x100], ids=["merged", "split"])
def test_selection_edge_rows(g, oracle, flags):
    """The selection inside the fused dispatches on rows that defeat its fast path: exact ties between
    experts (duplicated router rows), all logits equal (zero router), a row dominated by one expert so that the
    other exponentials underflow, and fewer experts than one wave holds."""
    H, F, k = 512, 64, 4
    for E in (8, 64, 512):
        L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.Q8_0, True, seed=SEED, layer=900 + E,
                             router_sigma=1.0 / np.sqrt(H))
        x = synth.rms_normed(synth.rng_for(SEED, 46, E), H)
        _fused_vs_oracle(g, oracle, L, x, flags)
        dup = dict(L)
        r = L["router"].copy()
        r[1::2] = r[0::2]                       # every odd expert ties with its even neighbour
        dup["router"] = r
        _fused_vs_oracle(g, oracle, dup, x, flags)
        zero = dict(L)
        zero["router"] = np.zeros_like(L["router"])
        _fused_vs_oracle(g, oracle, zero, x, flags)
        spike = dict(L)
        r = L["router"].copy()
        r[E // 2] = x * np.float32(200.0 / H)    # logit 200: every other exponential underflows to zero
        r[E // 2 + 1] = r[E // 2]
        spike["router"] = r
        _fused_vs_oracle(g, oracle, spike, x, flags)
        # near-ties: pairs of experts whose logits differ in the last places only, so that their exponentials are
        # equal or adjacent floats and the order of the probabilities is decided by rounding
        near = dict(L)
        r = L["router"].copy()
        r[1::2] = r[0::2]
        j = int(np.argmax(np.abs(x)))
        r[1::2, j] = np.nextafter(r[1::2, j], np.float32(np.inf))
        near["router"] = r
        _fused_vs_oracle(g, oracle, near, x, flags)
        # logits of minus infinity: all but two experts, i.e. fewer finite logits than k
        minf = dict(L)
        r = L["router"].copy()
        r[2:] = np.where(x > 0, np.float32(-np.inf), np.float32(np.inf))[None, :]
        minf["router"] = r
        _fused_vs_oracle(g, oracle, minf, x, flags)


@pytest.mark.parametrize("E,k", [(8, 1), (64, 8), (128, 8), (512, 10), (512, 16), (520, 10), (1024, 16)])
def test_selection_many_rows(g, oracle, E, k):
    """Ids and weights of many random rows at three logit scales (the selection thresholds on row maxima and ranks the
    candidates above the threshold), and a row whose large logits all sit in a few rows of lanes, so that there are
    more candidates than the fast path holds."""
    H, F = 256, 32
    for si, sigma in enumerate((1e-3, 1.0 / 16, 0.5)):
        L = synth.make_layer(H, F, E, k, synth.Q8_0, synth.Q8_0, False, seed=SEED, layer=960 + si, router_sigma=sigma)
        dl = g.DeviceLayer(L)
        sc = g.Scratch(H, F, E, k)
        out = g.empty(H, np.float32)
        for t in range(10):
            x = synth.rms_normed(synth.rng_for(SEED, 48, 1000 * E + 16 * si + t), H)
            want, d = oracle.moe_layer(L, x)
            dx = g.dev(x)
            capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, 0, g.stream())
            g.sync()
            assert np.array_equal(sc.get("ids", k, np.int32), d["ids"]), (E, k, sigma, t)
            assert g.same_bits(sc.get("weights", k, np.float32), d["weights"]), (E, k, sigma, t)
            assert g.same_bits(g.host(out), want), (E, k, sigma, t)
        sc.close()
    if E >= 512:
        L = synth.make_layer(H, F, E, k, synth.Q8_0, synth.Q8_0, False, seed=SEED, layer=970, router_sigma=1.0 / 16)
        x = synth.rms_normed(synth.rng_for(SEED, 49, E), H)
        r = L["router"].copy()
        for i in range(144):                     # logits 3 + i / 144 in nine rows of 16 lanes
            r[i] = x * np.float32((3.0 + i / 144.0) / H)
        L["router"] = r
        _fused_vs_oracle(g, oracle, L, x)


def test_selection_more_than_512_experts(g, oracle):
    H, F, k = 256, 32, 10
    for E in (520, 1024):
        L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.Q8_0, False, seed=SEED, layer=950 + E,
                             router_sigma=1.0 / np.sqrt(H))
        x = synth.rms_normed(synth.rng_for(SEED, 47, E), H)
        _fused_vs_oracle(g, oracle, L, x)
        dup = dict(L)
        r = L["router"].copy()
        r[E // 2:] = r[:E - E // 2]
        dup["router"] = r
        _fused_vs_oracle(g, oracle, dup, x)


def test_expert_counts_the_selection_cannot_take_are_refused(g, oracle):
    """The router's selection sums probabilities in groups of eight experts and holds at most 1024 of them
    (src/qwen38_moe.cuh:686-688): other counts are an error on every path that selects, not a silently different
    result; a pass on a given selection takes any count."""
    L = synth.make_layer(256, 64, 12, 2, synth.IQ3_S, synth.Q8_0, shared=True)
    dl, sc = g.DeviceLayer(L), g.Scratch(256, 64, 12, 2)
    x = synth.rms_normed(synth.rng_for(SEED, 45), 256)
    dx, out = g.dev(x), g.empty(256, np.float32)
    lib = capi.load()
    for flags in (0, capi.MOE_SPLIT_AB, capi.MOE_STAGED):
        assert lib.wd_moe_layer_f32(C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream()) == -1, flags
        assert "multiple of 8" in lib.wd_last_error().decode()
    arr = (capi.MoeLayer * 1)(dl.desc)
    assert lib.wd_moe_stack_f32(arr, 1, g.ptr(dx), g.ptr(out), sc.h, None, 1.0, 0, g.stream()) == -1
    sc.close()
    check_layer(g, oracle, L, x, flags=capi.MOE_PRESELECTED, ids=np.array([11, 3], np.int32), weights=np.array([0.25, 0.5], np.float32))


def test_status_word_is_clear(g):
    sc = g.Scratch(512, 64, 8, 2)
    assert capi.load().wd_moe_scratch_status(sc.h) == 0
    sc.close()


def test_bounded_wait_gives_up_and_recovers(g, oracle):
    """Failure path of the in-dispatch hand-off, forced from the host: with a wait limit of one poll the routed
    workgroups give up before the ids are published, the status word says so, every kernel still ends; with the
    default limit restored the same scratch gives the oracle's result again."""
    L = synth.make_c2(n_experts=64)
    H, F, E, k = 2048, 512, 64, 10
    x = synth.rms_normed(synth.rng_for(SEED, 48), H)
    dl, sc = g.DeviceLayer(L), g.Scratch(H, F, E, k)
    dx, out = g.dev(x), g.empty(H, np.float32)
    lib = capi.load()
    capi.call("wd_moe_scratch_set_wait_limit", sc.h, 1)
    capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, 0, g.stream())
    g.sync()
    assert lib.wd_moe_scratch_status(sc.h) == 1
    assert np.isnan(g.host(out)).all()       # the failure is in the data too: no caller takes garbage for a result
    capi.call("wd_moe_scratch_set_wait_limit", sc.h, 0)
    assert lib.wd_moe_scratch_status(sc.h) == 0
    capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, 0, g.stream())
    g.sync()
    want, d = oracle.moe_layer(L, x)
    assert lib.wd_moe_scratch_status(sc.h) == 0
    assert np.array_equal(sc.get("ids", k, np.int32), d["ids"])
    assert g.same_bits(g.host(out), want)
    sc.close()


def test_fused_gate_up_tensor_layout(g, oracle):
    """One tensor with 2 * ffn rows per expert (gate rows, then up rows), as the reference's target model stores
    them (src/qwen38_moe.cuh:3462-3514): the layer descriptor addresses it in place, resident and through the
    slot pool."""
    import torch
    H, F, E, k = 512, 64, 16, 4
    L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.Q8_0, True, seed=SEED, layer=60, router_sigma=1.0 / np.sqrt(H))
    x = synth.rms_normed(synth.rng_for(SEED, 50), H)
    want, d = oracle.moe_layer(L, x)
    rb = synth.row_bytes(synth.IQ3_S, H)
    gate = np.ascontiguousarray(L["gate"]).reshape(E, F * rb)
    up = np.ascontiguousarray(L["up"]).reshape(E, F * rb)
    fused = np.ascontiguousarray(np.concatenate([gate, up], axis=1))          # [E][2 F rows]
    dl = g.DeviceLayer(L)
    dfused = g.dev(fused.reshape(-1))
    desc = dl.desc
    desc.gate = dfused.data_ptr()
    desc.up = dfused.data_ptr() + F * rb
    desc.gate_stride = desc.up_stride = 2 * F * rb
    sc = g.Scratch(H, F, E, k)
    dx, out = g.dev(x), g.empty(H, np.float32)
    for flags in (0, capi.MOE_STAGED):
        capi.call("wd_moe_layer_f32", C.byref(desc), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream())
        g.sync()
        assert np.array_equal(sc.get("ids", k, np.int32), d["ids"])
        assert g.same_bits(g.host(out), want)
    # the same tensor as the host source of a slot pool
    db = H * synth.row_bytes(synth.Q8_0, F)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), 6 * (2 * F * rb + db), F * rb, F * rb, db, 1, E, 0)
    hf = torch.from_numpy(fused.reshape(-1).copy()).pin_memory()
    hd = torch.from_numpy(np.ascontiguousarray(L["down"]).reshape(-1)).pin_memory()
    capi.call("wd_expert_cache_register_layer_strided", cache, 0, C.c_void_p(hf.data_ptr()),
              C.c_void_p(hf.data_ptr() + F * rb), C.c_void_p(hd.data_ptr()), 2 * F * rb, 2 * F * rb, db)
    lib = capi.load()
    desc.gate = desc.up = desc.down = None
    desc.slot_of_expert = lib.wd_expert_cache_slot_table(cache, 0)
    desc.slot_pool = lib.wd_expert_cache_pool(cache)
    desc.slot_bytes, desc.slot_gate_bytes, desc.slot_up_bytes = 2 * F * rb + db, F * rb, F * rb
    arr = (capi.MoeLayer * 1)(desc)
    out2 = g.empty(H, np.float32)
    dx2 = g.dev(x)
    capi.call("wd_moe_stack_cached_f32", arr, 1, cache, g.ptr(dx2), g.ptr(out2), sc.h, None, None, 0.0, 0, g.stream())
    g.sync()
    assert g.same_bits(g.host(out2), want)
    sc.close()
    capi.call("wd_expert_cache_destroy", cache)


def test_alignment_chooses_the_fetch_path(g, oracle):
    """The C2 layer shape (hidden 2048, ffn 512) takes the coalesced fetch paths (aligned 16-byte words regrouped through
    LDS) when every routed and shared tensor starts on a 16-byte boundary, and the per-block loads otherwise.  The same
    layer with its tensors moved 2 bytes into their allocations (GGUF only promises 2-byte alignment of blocks) must
    give the same bits; token batches through both placements too."""
    import torch
    H, F, E, k = 2048, 512, 16, 4
    L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.Q8_0, True, seed=SEED, layer=61, router_sigma=1.0 / np.sqrt(H))
    xs = np.stack([synth.rms_normed(synth.rng_for(SEED, 51, t), H) for t in range(2)])
    want = [oracle.moe_layer(L, x) for x in xs]
    for shift in (0, 2):
        dl = g.DeviceLayer(L)
        keep = {}
        for name in ("gate", "up", "down", "shared_gate", "shared_up", "shared_down"):
            raw = np.ascontiguousarray(L[name]).reshape(-1)
            buf = torch.zeros(raw.size + 32, dtype=torch.uint8, device="cuda")
            buf[shift:shift + raw.size] = torch.from_numpy(raw).cuda()
            keep[name] = buf
            setattr(dl.desc, name, buf.data_ptr() + shift)
        sc = g.Scratch(H, F, E, k)
        for x, (w_out, d) in zip(xs, want):
            dx, out = g.dev(x), g.empty(H, np.float32)
            for flags in (0, 0x100):     # merged and split dispatches
                capi.call("wd_moe_layer_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream())
                g.sync()
                assert np.array_equal(sc.get("ids", k, np.int32), d["ids"]), (shift, flags)
                assert g.same_bits(g.host(out), w_out), (shift, flags)
        scs = [sc, g.Scratch(H, F, E, k)]
        arr = (C.c_void_p * 2)(*[s.h for s in scs])
        dx, out = g.dev(xs), g.empty((2, H), np.float32)
        capi.call("wd_moe_layer_tokens_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), 2, arr, 0, g.stream())
        g.sync()
        got = g.host(out)
        for t in range(2):
            assert g.same_bits(got[t], want[t][0]), (shift, t)
        assert capi.load().wd_moe_scratch_status(sc.h) == 0
        for s in scs:
            s.close()
