"""M tokens through one layer (speculative-verify batch): every selected expert is read once for all
tokens that routed to it, and each token's result is bit-identical to its own one-token pass and to
the CPU oracle."""
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


def correlated_tokens(H, T, seed, mix=0.6):
    rng = synth.rng_for(SEED, 71, seed)
    base = rng.normal(0, 1, H)
    xs = []
    for _ in range(T):
        v = mix * base + (1 - mix) * rng.normal(0, 1, H)
        xs.append((v / np.sqrt(np.mean(v ** 2))).astype(np.float32))
    return np.stack(xs)


def run_tokens(g, dl, L, xs, flags=0, ids=None, weights=None):
    H, F, E, k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
    T = xs.shape[0]
    scs = [g.Scratch(H, F, E, k) for _ in range(T)]
    if ids is not None:
        for t in range(T):
            capi.call("wd_memcpy_h2d", C.c_void_p(scs[t].raw("ids")), np.ascontiguousarray(ids[t], np.int32).ctypes.data_as(C.c_void_p), 4 * k, None)
            capi.call("wd_memcpy_h2d", C.c_void_p(scs[t].raw("weights")), np.ascontiguousarray(weights[t], np.float32).ctypes.data_as(C.c_void_p), 4 * k, None)
    arr = (C.c_void_p * T)(*[s.h for s in scs])
    dx, out = g.dev(xs), g.empty((T, H), np.float32)
    capi.call("wd_moe_layer_tokens_f32", C.byref(dl.desc), g.ptr(dx), g.ptr(out), T, arr, flags, g.stream())
    g.sync()
    res = dict(out=g.host(out), ids=np.stack([s.get("ids", k, np.int32) for s in scs]),
               weights=np.stack([s.get("weights", k, np.float32) for s in scs]),
               accum=np.stack([s.get("accum", H, np.float32) for s in scs]),
               act=np.stack([s.get("act", (k + 1) * F, np.float32).reshape(k + 1, F) for s in scs]))
    for s in scs:
        s.close()
    return res


def run_single(g, dl, L, x, flags=0, ids=None, weights=None):
    r = run_tokens(g, dl, L, x[None, :], flags, None if ids is None else ids[None], None if weights is None else weights[None])
    return {n: v[0] for n, v in r.items()}


@pytest.mark.parametrize("T", [1, 4, 8])
def test_c4_tokens(g, oracle, T):
    """Workload C4: T tokens through the 512-expert top-10 IQ3_S/Q8_0 layer with overlapping routing."""
    L = synth.make_c2()
    dl = g.DeviceLayer(L)
    xs = correlated_tokens(2048, T, T)
    got = run_tokens(g, dl, L, xs)
    union = set(got["ids"].ravel().tolist())
    if T == 4:
        assert 10 < len(union) < 40        # the sets overlap but are not identical
    for t in range(T):
        want, d = oracle.moe_layer(L, xs[t])
        assert np.array_equal(got["ids"][t], d["ids"])
        assert g.same_bits(got["weights"][t], d["weights"])
        assert g.same_bits(got["act"][t][:10], d["act"])
        assert g.same_bits(got["accum"][t], d["routed"])
        assert g.same_bits(got["out"][t], want)
    one = run_tokens(g, dl, L, xs[:1])
    assert g.same_bits(one["out"][0], got["out"][0])


@pytest.mark.parametrize("gate_t,down_t,shared,H,F,E,k", [
    (synth.IQ2_S, synth.Q8_0, True, 512, 64, 16, 4),
    (synth.IQ3_S, synth.Q8_0, False, 768, 96, 8, 8),
    (synth.Q8_0, synth.Q8_0, False, 512, 64, 8, 2),         # not on the union path: one pass per token
    (synth.IQ3_S, synth.IQ4_NL, True, 512, 64, 8, 2),       # union pass for gate/up, the one-token down dispatch per token
    (synth.IQ2_S, synth.IQ4_NL, True, 2560, 640, 32, 10),   # the model's own types and shapes: the aligned multi-token down dispatch
    (synth.IQ3_S, synth.Q8_0, True, 2560, 640, 16, 4),      # 20-block Q8_0 down rows: the aligned multi-token down dispatch
    (synth.IQ3_S, synth.IQ4_NL, True, 2048, 512, 16, 4),    # 16-block IQ4_NL down rows, idem
    (synth.IQ2_S, synth.IQ4_NL, False, 2560, 640, 16, 8),   # idem without a shared expert
])
def test_tokens_equal_single_passes(g, oracle, gate_t, down_t, shared, H, F, E, k):
    L = synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=SEED, layer=7, router_sigma=1.0 / np.sqrt(H))
    dl = g.DeviceLayer(L)
    xs = correlated_tokens(H, 5, H)
    got = run_tokens(g, dl, L, xs)
    for t in range(5):
        one = run_single(g, dl, L, xs[t])
        assert np.array_equal(got["ids"][t], one["ids"])
        assert g.same_bits(got["out"][t], one["out"]) and g.same_bits(got["accum"][t], one["accum"])
        want, _ = oracle.moe_layer(L, xs[t])
        assert g.same_bits(got["out"][t], want)


def test_tokens_preselected_full_overlap(g, oracle):
    """All tokens name the same experts in different orders: one union entry per expert."""
    L = synth.make_c2(n_experts=32)
    dl = g.DeviceLayer(L)
    T, k = 4, 10
    xs = correlated_tokens(2048, T, 3)
    rng = np.random.default_rng(SEED)
    base = rng.choice(32, size=k, replace=False)
    ids = np.stack([rng.permutation(base) for _ in range(T)]).astype(np.int32)
    wts = rng.uniform(0.05, 0.15, (T, k)).astype(np.float32)
    got = run_tokens(g, dl, L, xs, flags=capi.MOE_PRESELECTED, ids=ids, weights=wts)
    for t in range(T):
        want, _ = oracle.moe_layer(L, xs[t], ids=ids[t], weights=wts[t])
        assert g.same_bits(got["out"][t], want)


def test_tokens_errors(g):
    L = synth.make_layer(512, 64, 8, 2, synth.IQ3_S, synth.Q8_0, False)
    dl = g.DeviceLayer(L)
    sc = g.Scratch(512, 64, 8, 2)
    arr = (C.c_void_p * 2)(sc.h, sc.h)
    x = g.empty((2, 512), np.float32)
    lib = capi.load()
    assert lib.wd_moe_layer_tokens_f32(C.byref(dl.desc), g.ptr(x), g.ptr(x), 2, arr, 0, None) == -1   # shared scratch
    assert lib.wd_moe_layer_tokens_f32(C.byref(dl.desc), g.ptr(x), g.ptr(x), 9, arr, 0, None) == -1
    sc.close()


@pytest.mark.parametrize("shape", ["c2", "model", "small-unaligned"])
def test_tokens_on_a_table_of_expert_views(g, oracle, shape):
    """wd_moe_layer_tokens_pairs_f32: the pass over (gate, up, down) views given expert by expert - the form in which the
    reference's token batch receives acquired experts (src/qwen38_moe.cuh:2907-3109) - with entry numbers as ids.  The
    views here point into resident tensors, in a shuffled order with a few entries nobody selects; every token must
    come out as from the pass over the tensors themselves, i.e. as from the oracle."""
    if shape == "c2":
        L, T = synth.make_c2(n_experts=64), 4
    elif shape == "model":
        L, T = synth.make_layer(2560, 640, 32, 8, synth.IQ2_S, synth.IQ4_NL, shared=True, seed=SEED + 3), 3
    else:
        L, T = synth.make_layer(512, 64, 16, 4, synth.IQ3_S, synth.Q8_0, shared=False, seed=SEED + 4), 5
    H, F, E, k = L["hidden"], L["expert_ffn"], L["n_experts"], L["top_k"]
    dl = g.DeviceLayer(L)
    if shape == "small-unaligned":     # views that are only 2-byte aligned: the tensors copied to an odd-word offset
        for name in ("gate", "up", "down"):
            raw = np.concatenate([np.zeros(2, np.uint8), np.ascontiguousarray(L[name]).reshape(-1)])
            dl.keep[name + "_shifted"] = g.dev(raw)
            setattr(dl.desc, name, dl.keep[name + "_shifted"].data_ptr() + 2)
    xs = correlated_tokens(H, T, 31 + T)
    ref = run_tokens(g, dl, L, xs)
    rng = np.random.default_rng(SEED + 55)
    union = sorted(set(ref["ids"].ravel().tolist()))
    entries = union + [e for e in range(E) if e not in union][:3]
    order = rng.permutation(len(entries))
    entries = [entries[i] for i in order]
    entry_of = {e: i for i, e in enumerate(entries)}
    d = dl.desc
    P = C.c_void_p * len(entries)
    hg = P(*[d.gate + e * d.gate_stride for e in entries])
    hu = P(*[d.up + e * d.up_stride for e in entries])
    hd = P(*[d.down + e * d.down_stride for e in entries])
    scs = [g.Scratch(H, F, E, k) for _ in range(T)]
    for t in range(T):
        vids = np.array([entry_of[e] for e in ref["ids"][t]], np.int32)
        capi.call("wd_memcpy_h2d", C.c_void_p(scs[t].raw("ids")), vids.ctypes.data_as(C.c_void_p), 4 * k, None)
        capi.call("wd_memcpy_h2d", C.c_void_p(scs[t].raw("weights")), np.ascontiguousarray(ref["weights"][t]).ctypes.data_as(C.c_void_p), 4 * k, None)
    arr = (C.c_void_p * T)(*[s.h for s in scs])
    dx, out = g.dev(xs), g.empty((T, H), np.float32)
    lib = capi.load()
    for rep in range(6):       # more calls than the ring of pointer tables has entries
        capi.call("wd_moe_layer_tokens_pairs_f32", C.byref(d), hg, hu, hd, len(entries), g.ptr(dx), g.ptr(out), T, arr,
                  capi.MOE_PRESELECTED, g.stream())
    g.sync()
    got = g.host(out)
    for t in range(T):
        want, dump = oracle.moe_layer(L, xs[t])
        assert g.same_bits(got[t], want), (shape, t)
        assert g.same_bits(scs[t].get("accum", H, np.float32), dump["routed"]), (shape, t)
        assert g.same_bits(got[t], ref["out"][t])
    assert lib.wd_moe_layer_tokens_pairs_f32(C.byref(d), hg, hu, hd, len(entries), g.ptr(dx), g.ptr(out), T, arr, 0, g.stream()) == -1
    assert lib.wd_moe_layer_tokens_pairs_f32(C.byref(d), hg, hu, hd, 129, g.ptr(dx), g.ptr(out), T, arr, capi.MOE_PRESELECTED, g.stream()) == -1
    for s in scs:
        s.close()
