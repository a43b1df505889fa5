"""Pins the CPU oracle (oracle/wd_oracle.c) before anything is compared against it.

Three kinds of evidence, chosen so that a dropped term, a wrong sign or index or a
transposed operand fails at least one of them:
  * bit-for-bit agreement with the reference's own CPU header compiled as-is
    (oracle/_ref, skipped where it was not built),
  * closed forms and known answers the reference's tests hold
    (tests/lowbit_cuda_test.cu:50-98, tests/qwen38_moe_cuda_test.cu:237-254),
  * mathematics: an independent dequantiser + float64 dot, numpy float16, libm exp,
    numpy softmax/top-k, hand-built tie / underflow rows.
"""
import ctypes as C
import hashlib
import os
import re

import numpy as np
import pytest

from warpdecode_amd import synth

SEED = 20261014


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


# ----------------------------------------------------------------------------- codebooks
def test_codebook_digests(oracle):
    g3, g2 = oracle.iq3s_grid(), oracle.iq2s_grid()
    inc = open(os.path.join(os.path.dirname(__file__), "..", "warpdecode_amd", "csrc", "wd_codebooks.inc")).read()
    h3 = re.search(r'WD_IQ3S_GRID_SHA256 "([0-9a-f]+)"', inc).group(1)
    h2 = re.search(r'WD_IQ2S_GRID_SHA256 "([0-9a-f]+)"', inc).group(1)
    assert hashlib.sha256(g3.astype("<u4").tobytes()).hexdigest() == h3
    assert hashlib.sha256(g2.astype("<u8").tobytes()).hexdigest() == h2
    # structure: IQ3_S magnitudes are odd 1..15, IQ2_S magnitudes are 8/25/43; first entries known
    b3 = g3.astype("<u4").view(np.uint8)
    assert set(np.unique(b3)) <= set(range(1, 16, 2))
    assert set(np.unique(g2.astype("<u8").view(np.uint8))) == {8, 25, 43}
    assert g3[0] == 0x01010101 and g2[0] == 0x0808080808080808
    assert len(np.unique(g3)) == 512 and len(np.unique(g2)) == 1024


def test_codebooks_equal_reference(refcpu):
    r = refcpu.ref()
    g3 = np.ctypeslib.as_array(r.wdref_iq3s_grid(), shape=(512,))
    g2 = np.ctypeslib.as_array(r.wdref_iq2s_grid(), shape=(1024,))
    assert np.array_equal(g3, refcpu.iq3s_grid())
    assert np.array_equal(g2, refcpu.iq2s_grid())


# ----------------------------------------------------------------------------- f16
def test_f16_to_f32_all_halves(oracle):
    allh = np.arange(65536, dtype=np.uint16)
    mine = oracle.f16_to_f32(allh)
    want = allh.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(bits(mine)[~nan], bits(want)[~nan])
    assert np.all(np.isnan(mine[nan]))


def test_f32_to_f16_rne(oracle):
    rng = np.random.default_rng(SEED)
    vals = np.concatenate([
        rng.normal(0, 1, 20000), rng.normal(0, 1e-4, 20000), rng.normal(0, 1e-6, 5000),
        rng.uniform(-70000, 70000, 5000),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)[:0x7c00],      # exact halves
        np.float32(2.0) ** np.arange(-26, 17),
    ]).astype(np.float32)
    # halfway points between consecutive halves (ties must go to even)
    h = np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    vals = np.concatenate([vals, mid, -mid])
    mine = oracle.f32_to_f16(vals)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    # Documented deviation of the reference header: magnitudes below 2^-24 go to
    # signed zero (IEEE would round (2^-25, 2^-24) up to the smallest subnormal).
    tiny = np.abs(vals) < np.float32(2.0 ** -24)
    assert np.array_equal(mine[~tiny], want[~tiny])
    assert np.all((mine[tiny] & 0x7fff) == 0)


def test_f16_equal_reference(refcpu):
    r = refcpu.ref()
    rng = np.random.default_rng(SEED + 1)
    vals = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 4000), rng.normal(0, 3e-8, 2000),
                           [0.0, -0.0, 65504.0, 65520.0, 1e9, -1e9, np.inf, 2.0 ** -24, 2.0 ** -25,
                            1.5 * 2.0 ** -25, 2.0 ** -14]]).astype(np.float32)
    for v in vals:
        assert refcpu.lib().wdo_f32_to_f16(float(v)) == r.wdref_f32_to_f16(float(v)), v
    for h in range(0, 65536, 7):
        a, b = refcpu.lib().wdo_f16_to_f32(h), r.wdref_f16_to_f32(h)
        assert (np.isnan(a) and np.isnan(b)) or bits(a) == bits(b)


# ----------------------------------------------------------------------------- quantisers
def _act_cases(n):
    rng = np.random.default_rng(SEED + 2)
    xs = [rng.normal(0, 1, n), rng.normal(0, 1e-3, n), rng.normal(0, 1e-6, n), rng.uniform(-5, 5, n),
          np.zeros(n)]
    x = rng.normal(0, 1, n)
    x[:256] = 0.0                       # one all-zero block
    xs.append(x)
    x = rng.normal(0, 1, n)
    x[300] = -37.5                      # negative element carries the maximum
    xs.append(x)
    x = np.round(rng.normal(0, 20, n)) / 254.0 * 3.0   # many exact .5 products -> half-even
    xs.append(x)
    return [np.asarray(v, np.float32) for v in xs]


def test_q8_0_invariants(oracle):
    for x in _act_cases(1024):
        qs, d = oracle.quantize_q8_0(x)
        amax = np.abs(x.reshape(-1, 32)).max(axis=1)
        assert np.all(np.abs(qs.astype(int)) <= 127)
        big = amax / 127.0 >= 2.0 ** -24
        want_d = (amax / np.float32(127.0)).astype(np.float32).astype(np.float16).view(np.uint16)
        assert np.array_equal(d[big], want_d[big])
        # the element of largest magnitude maps to +-127 and reconstruction error is bounded
        nz = amax > 0
        assert np.all(np.abs(qs.reshape(-1, 32)).max(axis=1)[nz] == 127)
        rec = qs.reshape(-1, 32).astype(np.float64) * (amax / 127.0)[:, None]
        assert np.all(np.abs(rec - x.reshape(-1, 32)) <= (amax / 127.0)[:, None] * 0.5001 + 1e-12)


def test_q8_K_invariants(oracle):
    for x in _act_cases(1024):
        qs, d, bs = oracle.quantize_q8_K(x)
        q = qs.reshape(-1, 256).astype(int)
        assert np.array_equal(bs.reshape(-1, 16), q.reshape(-1, 16, 16).sum(axis=2))
        amax = np.abs(x.reshape(-1, 256)).max(axis=1)
        nz = amax > 0
        assert np.all(d[~nz] == 0) and np.all(q[~nz] == 0)
        assert np.all(d[nz] < 0)                                   # always-negative scale
        assert np.all(np.sign(q[nz]) * np.sign(x.reshape(-1, 256)[nz]) <= 0)   # quants carry -sign(x)
        rec = q * d[:, None].astype(np.float64)
        assert np.all(np.abs(rec - x.reshape(-1, 256)) <= (amax / 127.0 * 0.5001)[:, None] + 1e-12)


def test_quantisers_equal_reference(refcpu):
    r = refcpu.ref()
    f32p, i8p = C.POINTER(C.c_float), C.POINTER(C.c_int8)
    for x in _act_cases(2048):
        qs, d = refcpu.quantize_q8_0(x)
        rq, rd = np.empty_like(qs), np.empty_like(d)
        r.wdref_quantize_q8_0(x.ctypes.data_as(f32p), x.size, rq.ctypes.data_as(i8p),
                              rd.ctypes.data_as(C.POINTER(C.c_uint16)))
        assert np.array_equal(qs, rq) and np.array_equal(d, rd)
        qs, d, bs = refcpu.quantize_q8_K(x)
        rq, rd, rb = np.empty_like(qs), np.empty_like(d), np.empty_like(bs)
        r.wdref_quantize_q8_K(x.ctypes.data_as(f32p), x.size, rq.ctypes.data_as(i8p), rd.ctypes.data_as(f32p),
                              rb.ctypes.data_as(C.POINTER(C.c_int16)))
        assert np.array_equal(qs, rq) and np.array_equal(bits(d), bits(rd)) and np.array_equal(bs, rb)


# ----------------------------------------------------------------------------- row dots
def _put_half(buf, off, v):
    buf[off:off + 2] = np.frombuffer(np.float16(v).tobytes(), np.uint8)


def test_row_closed_forms(oracle):
    """tests/lowbit_cuda_test.cu:50-98: unit blocks against an all-ones activation."""
    one = np.float16(1.0).view(np.uint16)
    # Q8_0: d=1, 32 quants of 1 -> 32
    w = np.zeros(34, np.uint8); _put_half(w, 0, 1.0); w[2:] = 1
    out = oracle.gemv(oracle.Q8_0, w, 1, 32, np.ones(32, np.int8), np.array([one], np.uint16))
    assert out[0] == 32.0
    # IQ4_NL: nibble 8 -> code 1 everywhere -> 32
    w = np.zeros(18, np.uint8); _put_half(w, 0, 1.0); w[2:] = 0x88
    out = oracle.gemv(oracle.IQ4_NL, w, 1, 32, np.ones(32, np.int8), np.array([one], np.uint16))
    assert out[0] == 32.0
    # Q4_0: nibble 9 -> code 1 everywhere -> 32
    w = np.zeros(18, np.uint8); _put_half(w, 0, 1.0); w[2:] = 0x99
    out = oracle.gemv(oracle.Q4_0, w, 1, 32, np.ones(32, np.int8), np.array([one], np.uint16))
    assert out[0] == 32.0
    # IQ2_S zero block: grid[0] = eight 8s, ls = 1, x0.125 -> every value 1 -> 256
    w = np.zeros(82, np.uint8); _put_half(w, 0, 1.0)
    out = oracle.gemv(oracle.IQ2_S, w, 1, 256, np.ones(256, np.int8), np.array([1.0], np.float32))
    assert out[0] == 256.0
    # IQ3_S zero block: grid[0] = four 1s, ls = 1 -> 256
    w = np.zeros(110, np.uint8); _put_half(w, 0, 1.0)
    out = oracle.gemv(oracle.IQ3_S, w, 1, 256, np.ones(256, np.int8), np.array([1.0], np.float32))
    assert out[0] == 256.0


@pytest.mark.parametrize("t", [synth.IQ3_S, synth.IQ2_S, synth.Q8_0, synth.IQ4_NL, synth.Q4_0])
@pytest.mark.parametrize("cols", [256, 512, 2048, 2560])
def test_row_brute_force(oracle, t, cols):
    """Integer partials sum to the exact dot of independently decoded codes; float result
    agrees with a float64 dot of the dequantised row."""
    rng = synth.rng_for(SEED, 77, t, cols)
    rows = 6
    w = synth.matrix(t, rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    if t in (synth.IQ3_S, synth.IQ2_S):
        qs, d, _ = oracle.quantize_q8_K(x)
        act_val = qs.reshape(-1, 256).astype(np.float64) * d[:, None].astype(np.float64)
    else:
        qs, d = oracle.quantize_q8_0(x)
        act_val = qs.reshape(-1, 32).astype(np.float64) * oracle.f16_to_f32(d)[:, None].astype(np.float64)
    out, part = oracle.gemv(t, w, rows, cols, qs, d, want_partials=True)
    be = synth.BLOCK_ELEMS[t]
    for r in range(rows):
        deq = oracle.dequant_row(t, w[r], cols).astype(np.float64)
        want = float(np.dot(deq, act_val.ravel()))
        scale = float(np.sum(np.abs(deq * act_val.ravel()))) + 1e-30
        assert abs(out[r] - want) <= 2e-6 * scale
        # integer side: per block, sum of the chunk partials == exact integer dot of codes
        blocks = cols // be
        dw = oracle.f16_to_f32(w[r].reshape(blocks, -1)[:, :2].copy().view(np.uint16).ravel()).astype(np.float64)
        if t == synth.IQ2_S:
            dw = dw * 0.125
        codes = np.rint(deq.reshape(blocks, be) / np.where(dw == 0, 1, dw)[:, None])
        ok = dw != 0
        exact = (codes * qs.reshape(blocks, be).astype(np.float64)).sum(axis=1)
        got = part[r].reshape(blocks, -1).sum(axis=1)
        assert np.array_equal(got[ok], exact[ok].astype(np.int64))


def test_row_chunk_lane_order(oracle):
    """A mistake in which values form chunk lane c (or a transposed 4x8 split) changes the
    per-lane partials even when block sums agree: check lanes against numpy for Q8_0."""
    rng = synth.rng_for(SEED, 78)
    w = synth.q8_0_matrix(rng, 3, 128)
    qs = rng.integers(-127, 128, 128, dtype=np.int8)
    d = np.full(4, np.float16(0.5).view(np.uint16), np.uint16)
    _, part = oracle.gemv(oracle.Q8_0, w, 3, 128, qs, d, want_partials=True)
    wq = w.reshape(3, 4, 34)[:, :, 2:].view(np.int8).astype(int)
    want = (wq.reshape(3, 4, 8, 4) * qs.astype(int).reshape(4, 8, 4)).sum(axis=3)
    assert np.array_equal(part.reshape(3, 4, 8), want)


@pytest.mark.parametrize("t", [synth.IQ3_S, synth.IQ2_S, synth.Q8_0, synth.IQ4_NL])
@pytest.mark.parametrize("cols", [256, 512, 2048, 2560, 5120, 2560 + 32])
def test_rows_equal_reference(refcpu, t, cols):
    be = synth.BLOCK_ELEMS[t]
    if cols % be:
        pytest.skip("not a whole number of blocks")
    rng = synth.rng_for(SEED, 79, t, cols)
    rows = 8
    w = synth.matrix(t, rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    if t in (synth.IQ3_S, synth.IQ2_S):
        qs, d, _ = refcpu.quantize_q8_K(x)
    else:
        qs, d = refcpu.quantize_q8_0(x)
    mine = refcpu.gemv(t, w, rows, cols, qs, d)
    ref_avx = refcpu.ref_gemv(t, w, rows, cols, qs, d)
    ref_sc = np.array([refcpu.ref_row(t, w[r], cols, qs, d, scalar=True) for r in range(rows)], np.float32)
    assert np.array_equal(bits(mine), bits(ref_avx))
    assert np.array_equal(bits(mine), bits(ref_sc))


# ----------------------------------------------------------------------------- transcendentals
def _exp_inputs():
    rng = np.random.default_rng(SEED + 3)
    return np.concatenate([rng.uniform(-100, 10, 20000), rng.normal(0, 3, 20000), rng.uniform(-200, -80, 2000),
                           [0.0, -0.0, 1.0, -1.0, 88.0, 88.7, 89.0, 130.0, -87.3, -103.9, -104.0, -126.0, -150.0,
                            -1e30, -np.inf]]).astype(np.float32)


def test_exp_against_libm(oracle):
    x = _exp_inputs()
    got = oracle.exp_ggml(x).astype(np.float64)
    with np.errstate(over="ignore", under="ignore"):
        want = np.exp(x.astype(np.float64))
    assert oracle.exp_ggml(np.float32(0.0)) == 1.0
    normal = (want > 1e-37) & (want < 3e38)
    assert np.all(np.abs(got[normal] - want[normal]) <= 3.0e-7 * want[normal])     # ~2.5 ulp
    assert np.all(got[want < 1e-46] == 0.0)
    assert oracle.exp_ggml(np.float32(-np.inf)) == 0.0


def test_exp_silu_equal_reference(refcpu):
    r = refcpu.ref()
    x = _exp_inputs()
    mine = refcpu.exp_ggml(x)
    want = np.array([r.wdref_exp(float(v)) for v in x], np.float32)
    assert np.array_equal(bits(mine), bits(want))
    xs = x[np.isfinite(x)][:8000]
    mine = refcpu.silu_ggml(xs)
    want = np.array([r.wdref_silu(float(v)) for v in xs], np.float32)
    assert np.array_equal(bits(mine), bits(want))
    for v in (-3.0, 0.0, 0.25, 9.0):
        assert bits(refcpu.sigmoid_ggml(v)) == bits(np.float32(r.wdref_sigmoid(v)))


def test_silu_sigmoid_math(oracle):
    assert oracle.sigmoid_ggml(0.0) == 0.5
    x = np.linspace(-20, 20, 401).astype(np.float32)
    want = x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64)))
    assert np.allclose(oracle.silu_ggml(x), want, rtol=1e-6, atol=1e-30)


# ----------------------------------------------------------------------------- f32 dot
@pytest.mark.parametrize("n", [32, 2048, 2560, 2048 + 17, 5])
def test_dot_f32(oracle, n):
    rng = np.random.default_rng(SEED + n)
    a, b = rng.normal(0, 1, n).astype(np.float32), rng.normal(0, 1, n).astype(np.float32)
    got = oracle.dot_f32(a, b)
    want = np.dot(a.astype(np.float64), b.astype(np.float64))
    assert abs(got - want) <= 1e-6 * np.sum(np.abs(a.astype(np.float64) * b))
    # the accumulator assignment is observable: 32 exact strided partial sums of small integers
    ai = rng.integers(-8, 9, n).astype(np.float32)
    bi = rng.integers(-8, 9, n).astype(np.float32)
    assert oracle.dot_f32(ai, bi) == float(np.dot(ai.astype(np.int64), bi.astype(np.int64)))
    if oracle.ref() is not None:
        f32p = C.POINTER(C.c_float)
        want = oracle.ref().wdref_dot_f32(a.ctypes.data_as(f32p), b.ctypes.data_as(f32p), n)
        assert bits(got) == bits(np.float32(want))


def test_dot_f32_order_is_not_plain(oracle):
    """Negative control: the 4x8 accumulator order differs from a left-to-right float sum
    on ordinary data, so a test against it can see a wrong order."""
    rng = np.random.default_rng(SEED + 9)
    diff = 0
    for _ in range(50):
        a, b = rng.normal(0, 1, 2048).astype(np.float32), rng.normal(0, 1, 2048).astype(np.float32)
        s = np.float32(0)
        for v in (a * b):
            s = np.float32(s + v)
        diff += int(bits(s) != bits(oracle.dot_f32(a, b)))
    assert diff > 10


# ----------------------------------------------------------------------------- router
def test_router_known_answer(oracle):
    """tests/qwen38_moe_cuda_test.cu:40-50,237-254: router rows r+1, x = 1 over 32 columns
    -> logits 32,64,96,128 -> top-2 ids {3,2}, weights ~{1,0}."""
    w = np.repeat(np.arange(1, 5, dtype=np.float32)[:, None], 32, axis=1)
    logits = oracle.router_logits(w, np.ones(32, np.float32))
    assert np.array_equal(logits, [32, 64, 96, 128])
    # n = 4 is not a multiple of 8 -> scalar tail of the softmax; still the same chain
    ids, wts = oracle.route(logits, 2)
    assert list(ids) == [3, 2] and wts[0] > 0.999 and wts[1] < 0.001


@pytest.mark.parametrize("n,k", [(64, 8), (512, 10), (1024, 16), (8, 8)])
def test_router_against_numpy(oracle, n, k):
    rng = np.random.default_rng(SEED + n + k)
    for trial in range(40):
        logits = rng.normal(0, 1 + trial % 3, n).astype(np.float32)
        probs = oracle.softmax_row(logits)
        l64 = logits.astype(np.float64)
        want = np.exp(l64 - l64.max()); want /= want.sum()
        assert np.allclose(probs, want, rtol=2e-6, atol=1e-12)
        ids, wts = oracle.router_select(probs, k)
        order = np.lexsort((np.arange(n), -probs.astype(np.float64)))[:k]       # prob desc, id asc
        assert np.array_equal(ids, order)
        top = probs[order].astype(np.float64)
        assert np.allclose(wts, top / top.sum(), rtol=1e-6)
        assert len(set(ids.tolist())) == k and abs(float(wts.sum()) - 1.0) < 1e-5


def test_router_edge_rows(oracle):
    n, k = 64, 4
    # all-equal logits: uniform probabilities, ties fall to the lowest indices in order
    ids, wts = oracle.route(np.zeros(n, np.float32), k)
    assert list(ids) == [0, 1, 2, 3] and np.all(wts == np.float32(0.25))
    # exact ties between far-apart cells
    l = np.full(n, -5.0, np.float32); l[[40, 7, 23]] = 3.0; l[11] = 2.0
    ids, wts = oracle.route(l, k)
    assert list(ids) == [7, 23, 40, 11] and wts[0] == wts[1] == wts[2] > wts[3]
    # -inf cells get probability 0 and are never preferred over finite ones
    l = np.full(n, -np.inf, np.float32); l[[5, 9]] = [1.0, 2.0]
    probs = oracle.softmax_row(l)
    assert probs[0] == 0.0 and abs(probs[5] + probs[9] - 1.0) < 1e-6
    ids, wts = oracle.route(l, 3)
    assert list(ids[:2]) == [9, 5] and ids[2] == 0 and wts[2] == 0.0
    # w_scale applied after the division, skipped for 1.0
    l = np.random.default_rng(3).normal(0, 1, n).astype(np.float32)
    ids1, w1 = oracle.route(l, k, 1.0)
    ids2, w2 = oracle.route(l, k, 2.5)
    assert np.array_equal(ids1, ids2) and np.array_equal(w2, (w1 * np.float32(2.5)).astype(np.float32))
    # tiny sum is clamped at 2^-14 before the division
    probs = np.zeros(n, np.float32); probs[3] = 1e-6; probs[4] = 2e-6
    ids, wts = oracle.router_select(probs, 2)
    assert list(ids) == [4, 3] and wts[0] == np.float32(2e-6) / np.float32(6.103515625e-5)


# ----------------------------------------------------------------------------- expert chain and layer
def _small_layer(gate_t, down_t, shared, H=512, F=64, E=8, k=2, seed=SEED):
    return synth.make_layer(H, F, E, k, gate_t, down_t, shared, seed=seed, layer=3,
                            router_sigma=1.0 / np.sqrt(H))


@pytest.mark.parametrize("gate_t,down_t", [(synth.IQ3_S, synth.Q8_0), (synth.IQ2_S, synth.IQ4_NL),
                                           (synth.IQ3_S, synth.IQ4_NL), (synth.IQ2_S, synth.Q8_0)])
def test_layer_equals_reference_run_layer(refcpu, gate_t, down_t):
    L = _small_layer(gate_t, down_t, shared=False)
    x = synth.rms_normed(synth.rng_for(SEED, 5), L["hidden"])
    out, dump = refcpu.moe_layer(L, x)
    # one thread only: the reference's fork-join pool can hand a late worker a task of the next
    # parallel_for (stale function pointer) and then never finishes; its arithmetic is what is pinned
    ref = refcpu.ref_run_layer(L, x, dump["ids"], dump["weights"], threads=1)
    assert np.array_equal(bits(out), bits(ref))
    out_mt, _ = refcpu.moe_layer(L, x, threads=4)
    assert np.array_equal(bits(out), bits(out_mt))


def test_q8_0_chain_equals_reference(refcpu):
    """The Q8_0 expert chain (workload C0 experts and the shared expert)."""
    rng = synth.rng_for(SEED, 6)
    H, F = 512, 128
    g, u, d = synth.q8_0_matrix(rng, F, H), synth.q8_0_matrix(rng, F, H), synth.q8_0_matrix(rng, H, F)
    x = synth.rms_normed(rng, H)
    mine = refcpu.expert_ffn(synth.Q8_0, synth.Q8_0, synth.Q8_0, g, u, d, H, F, x)
    ref = refcpu.ref_q8_0_chain(g, u, d, H, F, x)
    assert np.array_equal(bits(mine), bits(ref))


def test_layer_composition(oracle):
    """Whole layer == its parts recombined by hand in numpy float32 (product rounded, then sum,
    top-k order; shared expert added last)."""
    L = _small_layer(synth.IQ3_S, synth.Q8_0, shared=True, k=3)
    x = synth.rms_normed(synth.rng_for(SEED, 7), L["hidden"])
    out, d = oracle.moe_layer(L, x)
    ids, wts = oracle.route(oracle.router_logits(L["router"], x), 3)
    assert np.array_equal(ids, d["ids"]) and np.array_equal(wts, d["weights"])
    acc = np.zeros(L["hidden"], np.float32)
    for j, e in enumerate(ids):
        eo = oracle.expert_ffn(L["gate_type"], L["up_type"], L["down_type"], L["gate"][e], L["up"][e], L["down"][e],
                               L["hidden"], L["expert_ffn"], x)
        assert np.array_equal(bits(eo), bits(d["expert_out"][j]))
        acc = (acc + (eo * wts[j]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(acc), bits(d["routed"]))
    so = oracle.expert_ffn(synth.Q8_0, synth.Q8_0, synth.Q8_0, L["shared_gate"], L["shared_up"], L["shared_down"],
                           L["hidden"], L["expert_ffn"], x)
    g = oracle.sigmoid_ggml(oracle.dot_f32(L["shared_gate_inp"], x))
    want = (acc + (so * g).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(out), bits(want))
    # negative control: a fused multiply-add combine is a different function
    fused = np.zeros(L["hidden"], np.float64)
    for j in range(3):
        fused = np.float32(fused + d["expert_out"][j].astype(np.float64) * np.float64(wts[j])).astype(np.float64)
    assert not np.array_equal(bits(fused.astype(np.float32)), bits(d["routed"]))


def test_layer_against_float64_model(oracle):
    """End-to-end sanity against a dequantise-everything float64 model of the same layer
    (tolerance only: the quantised activations are part of the function)."""
    L = _small_layer(synth.IQ3_S, synth.Q8_0, shared=True, k=2)
    H, F = L["hidden"], L["expert_ffn"]
    x = synth.rms_normed(synth.rng_for(SEED, 8), H)
    out, d = oracle.moe_layer(L, x)

    def deq(t, m, rows, cols):
        rb = synth.row_bytes(t, cols)
        return np.stack([oracle.dequant_row(t, m.ravel()[r * rb:(r + 1) * rb], cols) for r in range(rows)]).astype(np.float64)

    def ffn(g, u, dn):
        a = g @ x
        a = a / (1 + np.exp(-a)) * (u @ x)
        return dn @ a

    want = np.zeros(H)
    for j, e in enumerate(d["ids"]):
        want += d["weights"][j] * ffn(deq(L["gate_type"], L["gate"][e], F, H), deq(L["up_type"], L["up"][e], F, H),
                                      deq(L["down_type"], L["down"][e], H, F))
    gate = 1 / (1 + np.exp(-float(np.dot(L["shared_gate_inp"].astype(np.float64), x))))
    want += gate * ffn(deq(synth.Q8_0, L["shared_gate"], F, H), deq(synth.Q8_0, L["shared_up"], F, H),
                       deq(synth.Q8_0, L["shared_down"], H, F))
    err = np.linalg.norm(out - want) / np.linalg.norm(want)
    assert err < 0.02, err


# ---- Q6_K x Q8_K (the output head) ------------------------------------------------------------------------
def _q6k_codes(w_row, cols):
    """Independent reading of the Q6_K layout by value index: (code - 32) and the sub-block scale of every value."""
    nb = cols // 256
    blk = np.asarray(w_row, np.uint8).reshape(nb, 210).astype(np.int64)
    i = np.arange(256)
    half, q, l = i >> 7, (i & 127) >> 5, i & 31
    lo = blk[:, 64 * half + 32 * (q & 1) + l]
    low4 = np.where(q < 2, lo & 15, lo >> 4)
    high2 = (blk[:, 128 + 32 * half + l] >> (2 * q)) & 3
    sc = blk[:, 192 + 8 * half + 2 * q + (l >> 4)]
    sc = np.where(sc > 127, sc - 256, sc)
    return (low4 | (high2 << 4)) - 32, sc


def test_q6_k_known_answer(oracle):
    """tests/lowbit_cuda_test.cu:60-68: every code 33 (value +1), scales 1, d = 1, against an activation of ones."""
    raw = np.zeros(210, np.uint8)
    raw[0:128], raw[128:192], raw[192:208] = 0x11, 0xAA, 1
    raw[208:210] = np.array([1.0], np.float16).view(np.uint8)
    qs, d, bs = oracle.quantize_q8_K(np.ones(256, np.float32))
    y, part = oracle.gemv_q6_K(raw, 1, 256, qs, d, bs, want_partials=True)
    assert abs(float(y[0]) - 256.0) < 0.02
    assert np.array_equal(part[0], np.full(8, 32 * int(qs[0]), np.int32))   # 32 values of +1 per float lane


@pytest.mark.parametrize("cols", [256, 768, 2048, 4096])
def test_q6_k_brute_force(oracle, cols):
    rng = synth.rng_for(SEED, 300, cols)
    rows = 6
    w = synth.q6_k_matrix(rng, rows, cols)
    x = rng.normal(0, 1, cols).astype(np.float32)
    x[256 * (cols // 512):256 * (cols // 512) + 256] *= 1e-3     # one quiet super-block
    qs, d, bs = oracle.quantize_q8_K(x)
    y, part = oracle.gemv_q6_K(w, rows, cols, qs, d, bs, want_partials=True)
    a = qs.astype(np.int64).reshape(-1, 256)
    for r in range(rows):
        code, sc = _q6k_codes(w[r], cols)
        # the eight lane sums of a super-block add up to the exact integer dot of that super-block
        exact = (code * sc * a).sum(axis=1)
        assert np.array_equal(part[r].reshape(-1, 8).astype(np.int64).sum(axis=1), exact), (cols, r)
        # lane m holds bytes 4m..4m+3 of every 32-value chunk, before the -32 offset is moved to the 16-value sums
        raw = ((code + 32) * sc * a).reshape(-1, 8, 8, 4).sum(axis=(1, 3))          # [sb][m]
        sc16 = sc.reshape(-1, 16, 16)[:, :, 0]
        corr = 32 * (bs.astype(np.int64).reshape(-1, 16) * sc16).reshape(-1, 8, 2).sum(axis=2)
        assert np.array_equal(part[r].reshape(-1, 8).astype(np.int64), raw - corr), (cols, r)
        dq = oracle.dequant_row(14, w[r], cols).astype(np.float64)
        dw = np.asarray(w[r], np.uint8).reshape(-1, 210)[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
        assert np.allclose(dq.reshape(-1, 256), dw[:, None] * sc * code, rtol=0, atol=0)  # the C dequantiser reads the same layout
        act = (a * d.astype(np.float64)[:, None]).reshape(-1)
        ref = float(dq @ act)
        assert abs(float(y[r]) - ref) <= 1e-5 * np.abs(dq * act).sum(), (cols, r)


def test_q6_k_float_lanes_are_not_a_plain_sum(oracle):
    """Negative control: adding the super-block products in plain order gives other bits on some rows, so a check
    of the eight-lane order would notice a kernel that sums differently."""
    rng = synth.rng_for(SEED, 301)
    cols, rows = 2048, 64
    w = synth.q6_k_matrix(rng, rows, cols)
    qs, d, bs = oracle.quantize_q8_K(rng.normal(0, 1, cols).astype(np.float32))
    y, part = oracle.gemv_q6_K(w, rows, cols, qs, d, bs, want_partials=True)
    differs = 0
    for r in range(rows):
        dw = np.asarray(w[r], np.uint8).reshape(-1, 210)[:, 208:210].copy().view(np.float16).astype(np.float32)[:, 0]
        acc = np.float32(0)
        for sb in range(cols // 256):
            acc = np.float32(acc + np.float32(dw[sb] * d[sb]) * np.float32(part[r].reshape(-1, 8)[sb].sum()))
        differs += int(acc.view(np.uint32) != y[r].view(np.uint32))
    assert differs > 0


# ---- hyper-connection combine of the FFN branch (the consumer of the layer's output) ---------------------------
def test_exp2f_table_from_decimal_arithmetic():
    """Entry i is the double nearest to 2^(i/32), minus i << 47 (e_exp2f_data.c of glibc / the ARM optimized routines)."""
    from decimal import Decimal, getcontext
    getcontext().prec = 60
    text = open(os.path.join(os.path.dirname(__file__), "..", "warpdecode_amd", "csrc", "wd_exp2f_table.inc")).read()
    got = [int(v, 16) for v in re.findall(r"0x([0-9a-f]{16})ull", text)]
    want = []
    for i in range(32):
        bits = np.array([float(Decimal(2) ** (Decimal(i) / Decimal(32)))], np.float64).view(np.uint64)[0]
        want.append((int(bits) - (i << 47)) & (2 ** 64 - 1))
    assert got == want


def _exp_probe_inputs():
    rng = synth.rng_for(SEED, 400)
    edges = np.array([0.0, -0.0, 1.0, -1.0, 88.0, 88.7, 88.72283, 88.72284, 88.8, 89.0, 128.0, -87.0, -87.33655, -103.0,
                      -103.97, -103.972, -103.98, -104.0, -150.0, 1e-8, -1e-8, 1e-40, np.inf, -np.inf, np.nan, 3.4e38, -3.4e38],
                     np.float32)
    near = np.concatenate([np.nextafter(np.float32(v), np.float32(s)).reshape(1) for v in (88.72283, -103.972, -87.33655)
                           for s in (np.inf, -np.inf)]).astype(np.float32)
    return np.concatenate([edges, near, rng.uniform(-105.0, 90.0, 2_000_000).astype(np.float32),
                           rng.normal(0.0, 4.0, 1_000_000).astype(np.float32),
                           (rng.integers(0, 2 ** 32, 1_000_000, dtype=np.uint64).astype(np.uint32)).view(np.float32)])


def test_expf_glibc_equals_the_c_library(oracle):
    """The restated routine against the host C library's expf (glibc on x86-64, the routine the reference ports,
    src/qwen38_exact_math.cuh:20-30) over four million inputs: thresholds, random bit patterns, the working range."""
    x = _exp_probe_inputs()
    got, want = oracle.expf_glibc(x), oracle.libm_expf(x)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), (x[~same][:5], got[~same][:5], want[~same][:5])
    # and the function is what it claims to be: within half a unit in the last place of the float64 exponential
    xs = x[np.isfinite(x) & (np.abs(x) < 80)][:200000]
    ref = np.exp(xs.astype(np.float64))
    assert np.all(np.abs(oracle.expf_glibc(xs).astype(np.float64) - ref) <= 0.502 * np.spacing(ref.astype(np.float32)).astype(np.float64))


def test_round_half_equals_numpy_and_reference(oracle, refcpu):
    rng = synth.rng_for(SEED, 401)
    x = np.concatenate([
        (rng.integers(0, 2 ** 32, 1_000_000, dtype=np.uint64).astype(np.uint32)).view(np.float32),
        rng.normal(0, 1, 200000).astype(np.float32), rng.normal(0, 1e-6, 200000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.996, 65520.0, 70000.0, 2.0 ** -14, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, np.inf, -np.inf, 1.0009765625, 1.00048828125],
                 np.float32)])
    x = x[~np.isnan(x)]
    got = oracle.round_half(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    r = refcpu.ref()
    assert hasattr(r, "wdref_round_half")
    if True:
        for v in x[:20000]:
            assert np.float32(r.wdref_round_half(float(v))).view(np.uint32) == np.float32(oracle.lib().wdo_round_half(float(v))).view(np.uint32)


def test_branch_and_residual_steps(oracle, refcpu):
    """One rounded multiply then one rounded add (no fused multiply-add): against numpy float32 steps, the reference's
    header compiled in place, and the known answer of tests/issue1_ffn_precision_test.cpp:14-37."""
    rng = synth.rng_for(SEED, 402)
    a, b, c = (rng.normal(0, 1, 50000).astype(np.float32) for _ in range(3))
    lib = oracle.lib()
    fused_differs = 0
    for i in range(a.size):
        want = np.float32(a[i] + np.float32(b[i] * c[i]))
        got = np.float32(lib.wdo_moe_branch_f32(float(a[i]), float(b[i]), float(c[i])))
        assert got.view(np.uint32) == want.view(np.uint32)
        assert np.float32(lib.wdo_residual_add_f32(float(a[i]), float(b[i]), float(c[i]))).view(np.uint32) == want.view(np.uint32)
        fused_differs += int(np.float32(np.float64(b[i]) * np.float64(c[i]) + np.float64(a[i])) != want)
        if i < 5000:
            r = refcpu.ref()
            assert np.float32(r.wdref_moe_branch_f32(float(a[i]), float(b[i]), float(c[i]))).view(np.uint32) == want.view(np.uint32)
            assert np.float32(r.wdref_residual_add_f32(float(a[i]), float(b[i]), float(c[i]))).view(np.uint32) == want.view(np.uint32)
    assert fused_differs > 100          # the sample tells a fused multiply-add from the two-step form
    routed = np.float32(0.0)
    for e in range(10):
        half = oracle.round_half(np.array([1.0 if e % 2 == 0 else 1.0009765625], np.float32))[0]
        routed = np.float32(np.float64(np.float32(0.1)) * np.float64(half) + np.float64(routed))   # fmaf: exact product, one rounding
    moe = np.float32(lib.wdo_moe_branch_f32(float(routed), -0.00048828125, 0.5))
    out = np.float32(lib.wdo_residual_add_f32(0.333251953125, float(moe), 1.25))
    assert moe == np.float32(routed + np.float32(np.float32(0.5) * np.float32(-0.00048828125)))
    assert out == np.float32(np.float32(0.333251953125) + np.float32(np.float32(1.25) * moe))


@pytest.mark.parametrize("hc,hidden,round_half", [(4, 2048, False), (4, 2048, True), (3, 96, False), (1, 32, True), (8, 2560, False)])
def test_hc_combine_against_numpy(oracle, hc, hidden, round_half):
    """src/qwen38_hc.cuh:2530-2547 and :2241-2263 step by step in numpy float32, the weight through the C library's expf."""
    rng = synth.rng_for(SEED, 403, hc, hidden)
    res = rng.normal(0, 1, (hc, hidden)).astype(np.float32)
    routed = rng.normal(0, 0.3, hidden).astype(np.float32)
    shared = rng.normal(0, 0.3, hidden).astype(np.float32)
    gate = np.float32(rng.uniform(0, 1))
    inject = rng.normal(0, 2, hc).astype(np.float32)
    z = (inject * np.float32(1.0 / np.float32(hc))).astype(np.float32)
    e = oracle.libm_expf(-z)
    w = (np.float32(2.0) * (np.float32(1.0) / (np.float32(1.0) + e)).astype(np.float32)).astype(np.float32)

    def finish(v):
        with np.errstate(over="ignore"):
            return v.astype(np.float16).astype(np.float32) if round_half else v

    block = (routed + (shared * gate).astype(np.float32)).astype(np.float32)
    want = finish((res + (block[None, :] * w[:, None]).astype(np.float32)).astype(np.float32))
    got = oracle.hc_combine(res, block, inject, round_half)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got = oracle.hc_combine_moe(res, routed, shared, gate, inject, round_half)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    sh16 = shared.astype(np.float16)
    block16 = (routed + (sh16.astype(np.float32) * gate).astype(np.float32)).astype(np.float32)
    want16 = finish((res + (block16[None, :] * w[:, None]).astype(np.float32)).astype(np.float32))
    got = oracle.hc_combine_moe(res, routed, sh16.view(np.uint16), gate, inject, round_half)
    assert np.array_equal(got.view(np.uint32), want16.view(np.uint32))
    for c in range(hc):                 # the weight itself: 2 / (1 + exp(-inject / hc)) to float accuracy
        assert abs(float(w[c]) - 2.0 / (1.0 + np.exp(-float(inject[c]) / hc))) < 1e-6


# ---- the plain Q8_0 x Q8_1 path and the half-input quantiser (src/lowbit.cuh:287-362, src/warodecode.cu:1504-1520) ----
def test_f32_to_f16_rn_equals_numpy(oracle):
    """IEEE round-to-nearest-even against numpy's float16 conversion (an implementation of its own): ties, the subnormal
    range, overflow to infinity, and 200,000 values over thirteen decades."""
    edge = np.array([1.0, 65504, 65519.996, 65520, 2.0 ** -24, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                     1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, -(1 + 2.0 ** -11), 0.0, -0.0, 6.0e-8, 3.0e-8], np.float32)
    rng = np.random.default_rng(SEED + 901)
    many = (rng.normal(size=200000) * 10.0 ** rng.integers(-9, 5, 200000)).astype(np.float32)
    for v in (edge, many):
        with np.errstate(over="ignore"):
            assert np.array_equal(oracle.f32_to_f16_rn(v), v.astype(np.float16).view(np.uint16))


def test_q8_1_quantiser_closed_forms(oracle):
    """d = amax / 127 and q = roundf(x / d): with amax = 63.5 the scale is exactly 0.5, so x = j / 2 must give q = j; halves
    go away from zero (2.5 -> 3, -2.5 -> -3, where the Q8_0 quantiser's round-to-even gives 2 and -2); a zero block stays
    zero with a zero scale; the scale is half(d)."""
    x = np.zeros(96, np.float32)
    x[:32] = np.arange(-16, 16) * 0.5
    x[31] = 63.5
    x[64:96] = [127, 2.5, -2.5, 3.5, -3.5, 0.49999997, 126.5, -126.5] + [0] * 24
    q, d = oracle.quantize_q8_1(x)
    assert q[:31].tolist() == list(range(-16, 15)) and q[31] == 127
    assert not q[32:64].any() and d[1] == 0
    assert q[64:72].tolist() == [127, 3, -3, 4, -4, 0, 127, -127]
    assert oracle.quantize_q8_0(x[64:96])[0][:5].tolist() == [127, 2, -2, 4, -4]      # the other rounding, for contrast
    assert oracle.f16_to_f32(d).tolist() == [0.5, 0.0, 1.0]
    rng = np.random.default_rng(SEED + 902)
    x = rng.normal(0, 3, 4096).astype(np.float32)
    q, d = oracle.quantize_q8_1(x)
    amax = np.abs(x.reshape(-1, 32)).max(axis=1)
    scale = (amax / np.float32(127)).astype(np.float32)
    want = np.where(x.reshape(-1, 32) / scale[:, None] >= 0, np.floor(x.reshape(-1, 32) / scale[:, None] + np.float32(0.5)),
                    np.ceil(x.reshape(-1, 32) / scale[:, None] - np.float32(0.5)))
    # (floor(t + 0.5) in float32 can differ from roundf(t) only when t + 0.5 rounds up across an integer: none here)
    assert np.array_equal(q.reshape(-1, 32), want.astype(np.int8))
    assert np.array_equal(d, scale.astype(np.float16).view(np.uint16))


def test_q8_0_q8_1_gemv_against_exact_integers_and_a_sequential_sum(oracle):
    """With unit scales and small quants every product and partial sum is an integer below 2^24: the row sum must equal the
    integer dot product whatever the order.  With real scales the sum is order-dependent: it must equal the plain
    sequential float32 loop over the blocks (multiply the scales, multiply by the integer sum, add) and differ from a
    pairwise sum on this sample; the exported block sums are the exact int32 dot products."""
    rng = np.random.default_rng(SEED + 903)
    rows, cols = 7, 2048
    nb = cols // 32
    one = np.float16(1.0).view(np.uint16)

    def pack(dw, qw):
        w = np.empty((rows, nb, 34), np.uint8)
        w[:, :, :2] = dw.astype(np.uint16).reshape(rows, nb, 1).view(np.uint8).reshape(rows, nb, 2)
        w[:, :, 2:] = qw.view(np.uint8).reshape(rows, nb, 32)
        return w.reshape(-1)

    qw = rng.integers(-8, 9, (rows, nb, 32)).astype(np.int8)
    qx = rng.integers(-8, 9, cols).astype(np.int8)
    y, sums = oracle.gemv_q8_0_q8_1(pack(np.full((rows, nb), one), qw), rows, cols, qx, np.full(nb, one, np.uint16))
    exact = (qw.reshape(rows, cols).astype(np.int64) * qx.astype(np.int64)).sum(axis=1)
    assert np.array_equal(y, exact.astype(np.float32))
    assert np.array_equal(sums, (qw.astype(np.int64) * qx.reshape(nb, 32)).sum(axis=2))

    qw = rng.integers(-127, 128, (rows, nb, 32)).astype(np.int8)
    qx = rng.integers(-127, 128, cols).astype(np.int8)
    dw = rng.uniform(0.001, 0.02, (rows, nb)).astype(np.float16)
    dx = rng.uniform(0.001, 0.02, nb).astype(np.float16)
    y, sums = oracle.gemv_q8_0_q8_1(pack(dw.view(np.uint16), qw), rows, cols, qx, dx.view(np.uint16))
    dots = (qw.astype(np.int64) * qx.reshape(nb, 32)).sum(axis=2)
    assert np.array_equal(sums, dots)
    seq = np.zeros(rows, np.float32)
    for b in range(nb):
        scale = dw[:, b].astype(np.float32) * dx[b].astype(np.float32)
        seq = (seq + scale * dots[:, b].astype(np.float32)).astype(np.float32)
    assert np.array_equal(y.view(np.uint32), seq.view(np.uint32))
    prods = (dw.astype(np.float32) * dx.astype(np.float32)[None, :] * dots.astype(np.float32)).astype(np.float32)
    pairwise = prods.copy()
    while pairwise.shape[1] > 1:
        pairwise = (pairwise[:, 0::2] + pairwise[:, 1::2]).astype(np.float32)
    assert not np.array_equal(pairwise[:, 0].view(np.uint32), y.view(np.uint32))


def test_q8_0_quantiser_from_half_input(oracle):
    """The values widened to float go through inv = 127 / amax and lrintf (half to even), clamped to +-127; on input that
    is representable in half the quants equal the float quantiser's; the scale is the IEEE half of amax / 127, which for
    a block of tiny values is a subnormal half where the float quantiser's block-scale conversion stores zero."""
    rng = np.random.default_rng(SEED + 904)
    xh = rng.normal(0, 2, 2048).astype(np.float16)
    xh[32:64] = 0
    xh[64:96] = (2.0 ** -24 * rng.integers(-80, 81, 32)).astype(np.float16)   # amax / 127 between 2^-25 and 2^-24
    xh[64] = np.float16(84 * 2.0 ** -24)
    q, d = oracle.quantize_q8_0_f16(xh.view(np.uint16))
    qf, df = oracle.quantize_q8_0(xh.astype(np.float32))
    assert np.array_equal(q, qf)
    amax = np.abs(xh.astype(np.float32).reshape(-1, 32)).max(axis=1)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float32).astype(np.float16).view(np.uint16))
    assert d[1] == 0 and d[2] == 1 and df[2] == 0
    assert np.array_equal(d[3:], df[3:])
