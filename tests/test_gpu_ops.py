"""GPU parity of the stand-alone operators against the CPU oracle, through the C ABI.
Integer outputs (quants, ids, int32 chunk sums) and the f32 results of every operator whose float
order the reference fixes must match bit for bit; the dense Q4_0 GEMV (no canonical float order in
the reference) is held to 1e-5 relative."""
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


def _act_cases(n, seed):
    rng = np.random.default_rng(seed)
    xs = [rng.normal(0, 1, n), rng.normal(0, 1e-3, n), rng.normal(0, 1e-6, n), rng.uniform(-5, 5, n), np.zeros(n)]
    x = rng.normal(0, 1, n); x[:256] = 0.0; xs.append(x)
    x = rng.normal(0, 1, n); x[n // 2 + 3] = -37.5; xs.append(x)
    xs.append(np.round(rng.normal(0, 20, n)) / 254.0 * 3.0)       # exact .5 products: half-to-even
    xs.append(rng.normal(0, 3e-7, n))                              # fp16 scale below 2^-24 in some blocks
    x = rng.normal(0, 1, n); x[:256] = np.nan; xs.append(x)        # blocks of nothing but NaN: fmaxf from 0 drops them all
    return [np.asarray(v, np.float32) for v in xs]


@pytest.mark.parametrize("n", [256, 2048, 2560, 512 * 11])
def test_quantize_q8_k(g, oracle, n):
    for x in _act_cases(n, SEED + n):
        dx = g.dev(x)
        qs, d, bs = g.empty(n, np.int8), g.empty(n // 256, np.float32), g.empty(n // 16, np.int16)
        capi.call("wd_q8_k_quantize_f32", g.ptr(dx), n, g.ptr(qs), g.ptr(d), g.ptr(bs), g.stream())
        g.sync()
        oq, od, ob = oracle.quantize_q8_K(x)
        assert np.array_equal(g.host(qs), oq)
        assert g.same_bits(g.host(d), od)
        assert np.array_equal(g.host(bs), ob)


@pytest.mark.parametrize("n", [32, 512, 2048, 512 * 11, 32 * 37])
def test_quantize_q8_0(g, oracle, n):
    for x in _act_cases(max(n, 256), SEED + 7 * n):
        x = x[:n].copy()
        dx = g.dev(x)
        qs, d = g.empty(n, np.int8), g.empty(n // 32, np.uint16)
        capi.call("wd_q8_0_quantize_f32", g.ptr(dx), n, g.ptr(qs), g.ptr(d), g.stream())
        g.sync()
        oq, od = oracle.quantize_q8_0(x)
        assert np.array_equal(g.host(qs), oq)
        assert np.array_equal(g.host(d, np.uint16), od)


@pytest.mark.parametrize("rows,cols", [(64, 2048), (512, 2048), (512, 2560), (5, 96), (9, 2048 + 17), (3, 7)])
def test_router_gemv(g, oracle, rows, cols):
    rng = synth.rng_for(SEED, 11, rows, cols)
    w = rng.normal(0, 0.05, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, cols).astype(np.float32)
    dw, dx, out = g.dev(w), g.dev(x), g.empty(rows, np.float32)
    capi.call("wd_router_gemv_f32", g.ptr(dw), g.ptr(dx), g.ptr(out), rows, cols, g.stream())
    g.sync()
    assert g.same_bits(g.host(out), oracle.router_logits(w, x))


def _logit_rows(n, seed):
    rng = np.random.default_rng(seed)
    rows = [rng.normal(0, s, n) for s in (0.5, 1.0, 3.0, 10.0, 40.0)]
    rows.append(np.zeros(n))                                            # all equal
    r = np.full(n, -5.0); r[[n - 1, 3, n // 2]] = 3.0; r[5] = 2.0; rows.append(r)   # exact ties
    r = np.full(n, -np.inf); r[[1, 6]] = [1.0, 2.0]; rows.append(r)     # -inf cells
    r = rng.normal(0, 1, n); r[2] = 300.0; rows.append(r)               # everything else underflows
    r = np.round(rng.normal(0, 2, n)); rows.append(r)                   # many duplicate logits
    r = rng.normal(0, 1, n); r[0] = 1e-40; r[1] = -1e-40; rows.append(r)  # denormal logits
    return [np.asarray(v, np.float32) for v in rows]


@pytest.mark.parametrize("n,k", [(8, 2), (64, 8), (512, 10), (1024, 16), (72, 8)])
def test_topk_softmax(g, oracle, n, k):
    for scale in (1.0, 2.5):
        for logits in _logit_rows(n, SEED + n):
            dl = g.dev(logits)
            ids, wts = g.empty(k, np.int32), g.empty(k, np.float32)
            capi.call("wd_topk_softmax", g.ptr(dl), n, k, scale, g.ptr(ids), g.ptr(wts), g.stream())
            g.sync()
            oi, ow = oracle.route(logits, k, scale)
            assert np.array_equal(g.host(ids), oi), (logits[:8], g.host(ids), oi)
            assert g.same_bits(g.host(wts), ow)


def _quant_act(oracle, t, x):
    if t in (synth.IQ3_S, synth.IQ2_S):
        qs, d, _ = oracle.quantize_q8_K(x)
    else:
        qs, d = oracle.quantize_q8_0(x)
    return qs, d


GEMV_SHAPES = {
    synth.IQ3_S: [(512, 2048), (64, 2560), (5, 256), (33, 4096)],
    synth.IQ2_S: [(640, 2560), (512, 2048), (3, 256)],
    # the streaming kernel (eight rows per wave, 16- or 32-block chunks, single waves or four per workgroup, ragged row
    # counts), then shapes that take the general kernel
    synth.Q8_0: [(2048, 512), (512, 2048), (640, 2560), (2048, 8192), (1003, 2048), (5, 1024), (8203, 2048), (9, 16384),
                 (33, 512), (7, 96), (18, 32), (12, 32768), (40, 768),
                 # long rows and few of them: four waves share a row group
                 (100, 4096), (8, 8192), (515, 8192), (9, 4096), (8184, 4096), (4100, 8192), (21, 16384), (2563, 2560), (100, 5120),
                 (24, 10240)],
    synth.IQ4_NL: [(2560, 640), (2048, 512), (5, 96), (9, 32 * 5)],
    # C1 incl. the lm_head; then ragged row counts for every lanes-per-row case of the streaming kernel (columns a
    # multiple of 256 whose 8-block groups per row divide 64) and shapes that take the general kernel
    synth.Q4_0: [(2048, 2048), (2048, 8192), (8192, 2048), (128256, 2048), (1003, 2048), (5, 256), (67, 512), (131, 8192),
                 (7, 16384), (33, 1024), (6, 96), (40, 768), (9, 32768)],
}


@pytest.mark.parametrize("t", list(GEMV_SHAPES))
def test_gemv_single(g, oracle, t):
    for rows, cols in GEMV_SHAPES[t]:
        rng = synth.rng_for(SEED, 21, t, rows, cols)
        w = synth.matrix(t, rng, rows, cols)
        x = rng.normal(0, 1, cols).astype(np.float32)
        qs, d = _quant_act(oracle, t, x)
        ppr = oracle.partials_per_row(t, cols)
        dw, dq, dd = g.dev(w), g.dev(qs), g.dev(d)
        out, part = g.empty(rows, np.float32), g.empty((rows, ppr), np.int32)
        fn = "wd_gemv_q8_k_f32" if t in (synth.IQ3_S, synth.IQ2_S) else "wd_gemv_q8_0_f32"
        capi.call(fn, t, g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out), g.ptr(part), g.stream())
        out2 = g.empty(rows, np.float32)
        capi.call(fn, t, g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out2), None, g.stream())
        g.sync()
        want, wpart = oracle.gemv(t, w, rows, cols, qs, d, want_partials=True)
        assert np.array_equal(g.host(part), wpart), (t, rows, cols)
        if t == synth.Q4_0:
            # tolerance 1e-5 relative to the magnitude of the terms (float order is free there)
            rb = synth.row_bytes(t, cols)
            mag = np.array([np.abs(oracle.dequant_row(t, w[r], cols)).sum() for r in range(min(rows, 64))]).mean()
            assert np.allclose(g.host(out), want, rtol=1e-5, atol=1e-5 * mag), (rows, cols)
            assert np.allclose(g.host(out2), want, rtol=1e-5, atol=1e-5 * mag)
        else:
            assert g.same_bits(g.host(out), want), (t, rows, cols)
            assert g.same_bits(g.host(out2), want), (t, rows, cols)


# the output head of the Qwen3 MoE models (151936 x 2048), then ragged super-block counts (partial last pass, rows that
# do not start on 16-byte boundaries), one super-block, many passes
Q6K_SHAPES = [(151936, 2048), (1000, 4096), (37, 256), (129, 768), (65, 1280), (33, 2304), (9, 8192), (3, 32768)]


@pytest.mark.parametrize("rows,cols", Q6K_SHAPES)
def test_gemv_q6_k(g, oracle, rows, cols):
    rng = synth.rng_for(SEED, 27, rows, cols)
    w = synth.matrix(synth.Q6_K, rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    qs, d, bs = oracle.quantize_q8_K(x)
    dw, dq, dd, db = g.dev(w), g.dev(qs), g.dev(d), g.dev(bs)
    out, out2, part = g.empty(rows, np.float32), g.empty(rows, np.float32), g.empty((rows, cols // 256 * 8), np.int32)
    capi.call("wd_gemv_q6_k_q8_k_f32", g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(db), g.ptr(out), g.ptr(part), g.stream())
    capi.call("wd_gemv_q6_k_q8_k_f32", g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(db), g.ptr(out2), None, g.stream())
    g.sync()
    want, wpart = oracle.gemv_q6_K(w, rows, cols, qs, d, bs, want_partials=True)
    assert np.array_equal(g.host(part), wpart), (rows, cols)
    assert g.same_bits(g.host(out), want), (rows, cols)
    assert g.same_bits(g.host(out2), want), (rows, cols)


def test_gemv_q6_k_head_from_f32_and_misaligned(g, oracle):
    """The head as the caller runs it (quantise on the device, then the GEMV), and the same matrix 2 bytes into an
    allocation (GGUF blocks are only 2-byte aligned): the unaligned fetch must give the same bits."""
    import torch
    rows, cols = 515, 2048
    rng = synth.rng_for(SEED, 28, rows, cols)
    w = synth.matrix(synth.Q6_K, rng, rows, cols)
    x = synth.rms_normed(rng, cols)
    dx = g.dev(x)
    dq, dd, db = g.empty(cols, np.int8), g.empty(cols // 256, np.float32), g.empty(cols // 16, np.int16)
    capi.call("wd_q8_k_quantize_f32", g.ptr(dx), cols, g.ptr(dq), g.ptr(dd), g.ptr(db), g.stream())
    out = g.empty(rows, np.float32)
    dw = g.dev(w)
    capi.call("wd_gemv_q6_k_q8_k_f32", g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(db), g.ptr(out), None, g.stream())
    shifted = torch.zeros(w.size + 16, dtype=torch.uint8, device="cuda")
    shifted[2:2 + w.size] = dw.reshape(-1)
    out_s = g.empty(rows, np.float32)
    capi.call("wd_gemv_q6_k_q8_k_f32", shifted.data_ptr() + 2, rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(db), g.ptr(out_s), None, g.stream())
    g.sync()
    qs, d, bs = oracle.quantize_q8_K(x)
    want = oracle.gemv_q6_K(w, rows, cols, qs, d, bs)
    assert g.same_bits(g.host(out), want)
    assert g.same_bits(g.host(out_s), want)
    # against the dequantised weights in float64: the integer path is the exact product of the quantised operands
    xq = (qs.astype(np.float64).reshape(-1, 256) * d.astype(np.float64)[:, None]).reshape(-1)
    ref = np.array([oracle.dequant_row(synth.Q6_K, w[r], cols).astype(np.float64) @ xq for r in range(64)])
    assert np.allclose(g.host(out)[:64], ref, rtol=1e-4, atol=1e-6)


def test_q8_0_gemv_misaligned_base(g, oracle):
    """A Q8_0 matrix 2 bytes into an allocation takes the general kernel: same bits as the streaming one."""
    import torch
    rows, cols = 77, 2048
    rng = synth.rng_for(SEED, 24, rows, cols)
    w = synth.matrix(synth.Q8_0, rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    qs, d = oracle.quantize_q8_0(x)
    dq, dd = g.dev(qs), g.dev(d)
    dw = g.dev(w)
    shifted = torch.zeros(w.size + 16, dtype=torch.uint8, device="cuda")
    shifted[2:2 + w.size] = dw.reshape(-1)
    out, out_s = g.empty(rows, np.float32), g.empty(rows, np.float32)
    capi.call("wd_gemv_q8_0_f32", synth.Q8_0, g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out), None, g.stream())
    capi.call("wd_gemv_q8_0_f32", synth.Q8_0, shifted.data_ptr() + 2, rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out_s), None, g.stream())
    g.sync()
    want = oracle.gemv(synth.Q8_0, w, rows, cols, qs, d)
    assert g.same_bits(g.host(out), want) and g.same_bits(g.host(out_s), want)


# cols, then the rows of every item: the projections of a block on one activation (2048 columns), the long rows of a down
# projection (8192), a list longer than one launch takes (18 items), and lists with items the shared kernel does not
# take (fewer than 8 rows; 8192 rows and more; a base 2 bytes into an allocation), which are launched by themselves
@pytest.mark.parametrize("cols,rows_list,shift", [(2048, [2048, 512, 512, 1024, 64, 2048], None), (8192, [512, 256, 2048], None),
                                                  (4096, [1024] * 18, None), (2048, [96, 5, 8192, 40, 8], None),
                                                  (1024, [48, 16, 200], None), (2048, [256, 77, 128], 1)],
                         ids=["2048-projections", "8192-down", "18-items", "odd-ones-out", "1024-general-kernel", "misaligned-item"])
def test_q8_0_gemv_batch(g, oracle, cols, rows_list, shift):
    """wd_gemv_q8_0_batch_f32 against the same matrices one call each (the same bits) and against the oracle; two
    activations shared out over the items."""
    import torch
    rng = synth.rng_for(SEED, 29, cols, len(rows_list))
    acts = []
    for a in range(2):
        x = rng.normal(0, 1, cols).astype(np.float32)
        qs, d = oracle.quantize_q8_0(x)
        acts.append((qs, d, g.dev(qs), g.dev(d)))
    items = (capi.GemvItem * len(rows_list))()
    keep, singles, wants = [], [], []
    for i, rows in enumerate(rows_list):
        w = synth.matrix(synth.Q8_0, rng, rows, cols)
        qs, d, dq, dd = acts[i % 2]
        if shift == i:
            buf = torch.zeros(w.size + 16, dtype=torch.uint8, device="cuda")
            buf[2:2 + w.size] = g.dev(w).reshape(-1)
            wptr = buf.data_ptr() + 2
        else:
            buf = g.dev(w)
            wptr = buf.data_ptr()
        out, single = g.empty(rows, np.float32), g.empty(rows, np.float32)
        keep.append((buf, out))
        singles.append(single)
        items[i].d_w, items[i].rows, items[i].d_act_qs, items[i].d_act_scales, items[i].d_out = wptr, rows, dq.data_ptr(), dd.data_ptr(), out.data_ptr()
        capi.call("wd_gemv_q8_0_f32", synth.Q8_0, wptr, rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(single), None, g.stream())
        wants.append(oracle.gemv(synth.Q8_0, w, rows, cols, qs, d))
    capi.call("wd_gemv_q8_0_batch_f32", synth.Q8_0, items, len(rows_list), cols, g.stream())
    g.sync()
    for i, rows in enumerate(rows_list):
        got = g.host(keep[i][1])
        assert g.same_bits(got, g.host(singles[i])), (i, rows)
        assert g.same_bits(got, wants[i]), (i, rows)


# the projections of a Llama-3.2-1B block (q, k, v on one activation; gate and up), a shape the streaming kernel does not
# take (2560 columns: ten 8-block groups), a list of 17
@pytest.mark.parametrize("cols,rows_list", [(2048, [2048, 512, 512]), (2048, [8192, 8192]), (2560, [64, 128]), (2048, [256] * 17),
                                            (8192, [2048, 100])],
                         ids=["qkv", "gate-up", "general-kernel", "17-items", "down-and-ragged"])
def test_q4_0_gemv_batch(g, oracle, cols, rows_list):
    """The same for Q4_0 matrices: the same bits as one call each (the float order of Q4_0 is this library's own, so the
    oracle is met within 1e-5 as in the single-matrix tests; the int32 block sums are covered there)."""
    rng = synth.rng_for(SEED, 30, cols, len(rows_list))
    x = rng.normal(0, 1, cols).astype(np.float32)
    qs, d = oracle.quantize_q8_0(x)
    dq, dd = g.dev(qs), g.dev(d)
    items = (capi.GemvItem * len(rows_list))()
    keep, singles, wants, mats = [], [], [], []
    for i, rows in enumerate(rows_list):
        w = synth.matrix(synth.Q4_0, rng, rows, cols)
        mats.append(w)
        dw, out, single = g.dev(w), g.empty(rows, np.float32), g.empty(rows, np.float32)
        keep.append((dw, out))
        singles.append(single)
        items[i].d_w, items[i].rows, items[i].d_act_qs, items[i].d_act_scales, items[i].d_out = dw.data_ptr(), rows, dq.data_ptr(), dd.data_ptr(), out.data_ptr()
        capi.call("wd_gemv_q8_0_f32", synth.Q4_0, g.ptr(dw), rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(single), None, g.stream())
        wants.append(oracle.gemv(synth.Q4_0, w, rows, cols, qs, d))
    capi.call("wd_gemv_q8_0_batch_f32", synth.Q4_0, items, len(rows_list), cols, g.stream())
    g.sync()
    for i, rows in enumerate(rows_list):
        got = g.host(keep[i][1])
        assert g.same_bits(got, g.host(singles[i])), (i, rows)
        mag = np.array([np.abs(oracle.dequant_row(synth.Q4_0, mats[i][r], cols)).sum() for r in range(min(rows, 16))]).mean()
        assert np.allclose(got, wants[i], rtol=1e-5, atol=1e-5 * mag), (i, rows)


def test_q8_0_gemv_batch_refuses_what_it_cannot_take(g):
    items = (capi.GemvItem * 1)()
    lib = capi.load()
    assert lib.wd_gemv_q8_0_batch_f32(synth.IQ4_NL, items, 1, 2048, g.stream()) != 0    # Q8_0 and Q4_0 matrices only
    assert lib.wd_gemv_q8_0_batch_f32(synth.Q8_0, items, 0, 2048, g.stream()) != 0      # no items
    assert lib.wd_gemv_q8_0_batch_f32(synth.Q8_0, items, 1, 2040, g.stream()) != 0      # not whole blocks
    assert lib.wd_gemv_q8_0_batch_f32(synth.Q8_0, items, 1, 2048, g.stream()) != 0      # null pointers in the item


def test_q4_0_gemv_misaligned_base(g, oracle):
    """A matrix that starts 2 bytes into an allocation (GGUF blocks are only 2-byte aligned) takes the general
    kernel instead of the streaming one; both must give the same block sums."""
    import torch
    rows, cols = 300, 2048
    rng = synth.rng_for(SEED, 23, rows, cols)
    w = synth.matrix(synth.Q4_0, rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    qs, d = oracle.quantize_q8_0(x)
    raw = torch.zeros(w.size + 64, dtype=torch.uint8, device="cuda")
    want, wpart = oracle.gemv(synth.Q4_0, w, rows, cols, qs, d, want_partials=True)
    dq, dd = g.dev(qs), g.dev(d)
    for shift in (0, 2, 16, 18):
        raw[shift:shift + w.size] = torch.from_numpy(w.reshape(-1)).cuda()
        out, part = g.empty(rows, np.float32), g.empty((rows, cols // 32), np.int32)
        capi.call("wd_gemv_q8_0_f32", synth.Q4_0, C.c_void_p(raw.data_ptr() + shift), rows, cols, g.ptr(dq), g.ptr(dd),
                  g.ptr(out), g.ptr(part), g.stream())
        g.sync()
        assert np.array_equal(g.host(part), wpart), shift
        assert np.allclose(g.host(out), want, rtol=1e-5, atol=1e-7), shift


@pytest.mark.parametrize("t,rows,cols,experts", [(synth.IQ3_S, 512, 2048, 20), (synth.IQ2_S, 640, 2560, 20),
                                                  (synth.IQ3_S, 37, 512, 3)])
def test_gemv_experts_q8k(g, oracle, t, rows, cols, experts):
    rng = synth.rng_for(SEED, 22, t, rows, cols)
    ws = [synth.matrix(t, rng, rows, cols) for _ in range(experts)]
    x = rng.normal(0, 1, cols).astype(np.float32)
    qs, d = _quant_act(oracle, t, x)
    dws = [g.dev(w) for w in ws]
    table = g.dev(np.array([w.data_ptr() for w in dws], np.uint64))
    dq, dd = g.dev(qs), g.dev(d)
    ppr = oracle.partials_per_row(t, cols)
    out, part = g.empty((experts, rows), np.float32), g.empty((experts, rows, ppr), np.int32)
    capi.call("wd_gemv_q8_k_experts_f32", t, g.ptr(table), experts, rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out),
              g.ptr(part), g.stream())
    g.sync()
    for e in range(experts):
        want, wpart = oracle.gemv(t, ws[e], rows, cols, qs, d, want_partials=True)
        assert np.array_equal(g.host(part)[e], wpart)
        assert g.same_bits(g.host(out)[e], want)


@pytest.mark.parametrize("t,rows,cols,experts", [(synth.Q8_0, 2048, 512, 10), (synth.IQ4_NL, 2560, 640, 10),
                                                  (synth.Q8_0, 21, 96, 4)])
def test_gemv_experts_q8_0(g, oracle, t, rows, cols, experts):
    rng = synth.rng_for(SEED, 23, t, rows, cols)
    ws = [synth.matrix(t, rng, rows, cols) for _ in range(experts)]
    xs = rng.normal(0, 1, (experts, cols)).astype(np.float32)
    qd = [oracle.quantize_q8_0(xs[e]) for e in range(experts)]
    qs = np.stack([q for q, _ in qd]); d = np.stack([s for _, s in qd])
    dws = [g.dev(w) for w in ws]
    table = g.dev(np.array([w.data_ptr() for w in dws], np.uint64))
    dq, dd = g.dev(qs), g.dev(d)
    out = g.empty((experts, rows), np.float32)
    capi.call("wd_gemv_q8_0_experts_f32", t, g.ptr(table), experts, rows, cols, g.ptr(dq), g.ptr(dd), g.ptr(out),
              None, g.stream())
    g.sync()
    for e in range(experts):
        assert g.same_bits(g.host(out)[e], oracle.gemv(t, ws[e], rows, cols, qs[e], d[e]))


def test_elementwise(g, oracle):
    rng = np.random.default_rng(SEED + 31)
    F, k, H = 512, 10, 2048
    gu = np.concatenate([rng.normal(0, 2, (k, 2, F - 8)), rng.normal(0, 30, (k, 2, 8))], axis=2).astype(np.float32)
    dgu, act = g.dev(gu), g.empty((k, F), np.float32)
    capi.call("wd_silu_mul_experts_f32", g.ptr(dgu), g.ptr(act), F, k, g.stream())
    g.sync()
    want = (oracle.silu_ggml(gu[:, 0, :]) * gu[:, 1, :]).astype(np.float32)
    assert g.same_bits(g.host(act), want)

    ex = rng.normal(0, 1, (k, H)).astype(np.float32)
    w = rng.uniform(0, 0.3, k).astype(np.float32)
    acc0 = rng.normal(0, 1, H).astype(np.float32)
    dex, dw, dacc = g.dev(ex), g.dev(w), g.dev(acc0)
    capi.call("wd_weighted_accum_experts_f32", g.ptr(dex), g.ptr(dw), g.ptr(dacc), H, k, g.stream())
    g.sync()
    want = acc0.copy()
    for j in range(k):
        want = (want + (ex[j] * w[j]).astype(np.float32)).astype(np.float32)
    assert g.same_bits(g.host(dacc), want)
    # negative control: a fused multiply-add accumulation is a different function
    fused = acc0.astype(np.float64)
    for j in range(k):
        fused = np.float32(fused + ex[j].astype(np.float64) * np.float64(w[j])).astype(np.float64)
    assert not g.same_bits(fused.astype(np.float32), want)

    sh = rng.normal(0, 1, H).astype(np.float32)
    gate = np.array([0.37], np.float32)
    dsh, dg = g.dev(sh), g.dev(gate)
    capi.call("wd_add_shared_f32", g.ptr(dacc), g.ptr(dsh), g.ptr(dg), H, g.stream())
    g.sync()
    assert g.same_bits(g.host(dacc), (want + (sh * gate[0]).astype(np.float32)).astype(np.float32))


def test_error_paths(g):
    x = g.empty(300, np.float32)
    lib = capi.load()
    assert lib.wd_q8_k_quantize_f32(g.ptr(x), 300, g.ptr(x), g.ptr(x), g.ptr(x), None) == -1
    assert lib.wd_topk_softmax(g.ptr(x), 64, 17, 1.0, g.ptr(x), g.ptr(x), None) == -1
    assert lib.wd_gemv_q8_0_f32(synth.IQ3_S, g.ptr(x), 4, 256, g.ptr(x), g.ptr(x), g.ptr(x), None, None) == -1
    assert lib.wd_gemv_q8_k_f32(synth.IQ3_S, g.ptr(x), 4, 100, g.ptr(x), g.ptr(x), g.ptr(x), None, None) == -1
    assert lib.wd_gemv_q6_k_q8_k_f32(g.ptr(x), 4, 300, g.ptr(x), g.ptr(x), g.ptr(x), g.ptr(x), None, None) == -1
    assert lib.wd_gemv_q6_k_q8_k_f32(g.ptr(x), 4, 65536, g.ptr(x), g.ptr(x), g.ptr(x), g.ptr(x), None, None) == -1


# ---- the plain Q8_0 x Q8_1 path, the half-input quantiser, the element-wise conversions ------------------------------
@pytest.mark.parametrize("n", [32, 2048, 6144, 32 * 37])
def test_quantize_q8_1(g, oracle, n):
    for x in _act_cases(max(n, 256), SEED + 13 * n):
        x = x[:n].copy()
        dx = g.dev(x)
        qs, d = g.empty(n, np.int8), g.empty(n // 32, np.uint16)
        capi.call("wd_q8_1_quantize_f32", g.ptr(dx), n, g.ptr(qs), g.ptr(d), g.stream())
        g.sync()
        oq, od = oracle.quantize_q8_1(x)
        assert np.array_equal(g.host(qs), oq)
        assert np.array_equal(g.host(d, np.uint16), od)


@pytest.mark.parametrize("rows,cols", [(64, 2048), (5, 96), (9, 2048 + 64), (320, 2048), (2048, 320), (3, 4096 + 32)])
def test_gemv_q8_0_q8_1(g, oracle, rows, cols):
    """launch_q8_0_gemv_q8_1_f32 (src/lowbit.cuh:343-362): quantise, then the row sums in block order - quants, scales,
    int32 block sums and f32 results all bit-identical to the oracle."""
    rng = synth.rng_for(SEED, 77, rows, cols)
    w = np.ascontiguousarray(synth.q8_0_matrix(rng, rows, cols)).reshape(-1)
    for x in _act_cases(max(cols, 256), SEED + rows + cols)[:4]:
        x = x[:cols].copy()
        dw, dx = g.dev(w), g.dev(x)
        qs, d = g.empty(cols, np.int8), g.empty(cols // 32, np.uint16)
        y, sums = g.empty(rows, np.float32), g.empty(rows * (cols // 32), np.int32)
        capi.call("wd_q8_1_quantize_f32", g.ptr(dx), cols, g.ptr(qs), g.ptr(d), g.stream())
        capi.call("wd_gemv_q8_0_q8_1_f32", g.ptr(dw), rows, cols, g.ptr(qs), g.ptr(d), g.ptr(y), g.ptr(sums), g.stream())
        g.sync()
        oq, od = oracle.quantize_q8_1(x)
        oy, osums = oracle.gemv_q8_0_q8_1(w, rows, cols, oq, od)
        assert np.array_equal(g.host(qs), oq) and np.array_equal(g.host(d, np.uint16), od)
        assert np.array_equal(g.host(sums).reshape(rows, -1), osums)
        assert g.same_bits(g.host(y), oy)
    lib = capi.load()
    assert lib.wd_gemv_q8_0_q8_1_f32(g.ptr(dw), rows, 33, g.ptr(qs), g.ptr(d), g.ptr(y), None, g.stream()) == -1


@pytest.mark.parametrize("n", [32, 2048, 32 * 37])
def test_quantize_q8_0_from_half(g, oracle, n):
    rng = np.random.default_rng(SEED + 17 * n)
    for scale in (1.0, 1e-3, 3e-6, 300.0):
        xh = (rng.normal(0, 1, n) * scale).astype(np.float16)
        xh[:8] = 0
        dx = g.dev(xh.view(np.uint16))
        qs, d = g.empty(n, np.int8), g.empty(n // 32, np.uint16)
        capi.call("wd_q8_0_quantize_f16", g.ptr(dx), n, g.ptr(qs), g.ptr(d), g.stream())
        g.sync()
        oq, od = oracle.quantize_q8_0_f16(xh.view(np.uint16))
        assert np.array_equal(g.host(qs), oq), scale
        assert np.array_equal(g.host(d, np.uint16), od), scale


def test_half_float_conversions(g, oracle):
    """Every half widens exactly; floats narrow by IEEE round-to-nearest-even (numpy's float16 conversion and the oracle's
    agree, tests/test_oracle_pins.py)."""
    halves = np.arange(65536, dtype=np.uint16)
    dh, df = g.dev(halves), g.empty(65536, np.float32)
    capi.call("wd_convert_f16_to_f32", g.ptr(dh), g.ptr(df), 65536, g.stream())
    g.sync()
    want = halves.view(np.float16).astype(np.float32)
    got = g.host(df)
    finite = ~np.isnan(want)
    assert g.same_bits(got[finite], want[finite]) and np.isnan(got[~finite]).all()
    rng = np.random.default_rng(SEED + 31)
    v = (rng.normal(size=100001) * 10.0 ** rng.integers(-9, 5, 100001)).astype(np.float32)
    v[:6] = [65504, 65520, 2.0 ** -25, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, -0.0]
    dv, dout = g.dev(v), g.empty(v.size, np.uint16)
    capi.call("wd_convert_f32_to_f16", g.ptr(dv), g.ptr(dout), v.size, g.stream())
    g.sync()
    with np.errstate(over="ignore"):
        assert np.array_equal(g.host(dout, np.uint16), v.astype(np.float16).view(np.uint16))
    assert np.array_equal(g.host(dout, np.uint16)[:2000], oracle.f32_to_f16_rn(v[:2000]))
