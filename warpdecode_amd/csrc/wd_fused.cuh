// Fused MoE layer: two dispatches per layer (three when the caller asks for the split form).
//   AB router logits (+ shared-expert gate logit), one row per wave; the router workgroup that finishes last
//      runs softmax/top-k and publishes the ids inside the dispatch; the shared expert's gate/up + SwiGLU and
//      the routed gate/up + SwiGLU run in the same launch: the routed workgroups quantise x and stage the
//      codebooks while the router runs and pick the ids up as soon as they appear
//      (k_layer_a + k_layer_b are the same work as two launches: ids given by the caller, IQ4_NL gate/up,
//      or WD_MOE_SPLIT_AB)
//   C  Q8_0 re-quantisation of the k+1 activations, all down projections, the ordered weighted
//      sum, the gated shared branch and the optional residual update
// Activation quantisation is redone by every workgroup that needs it (8 KB of f32 from L2 and a
// few dozen instructions per lane) instead of being a dispatch of its own.
#pragma once
#include <type_traits>

#include "wd_kernels.cuh"

namespace wd {

struct LayerArgs {
    int H, F, E, k;
    float w_scale;
    const float *x;
    const float *router;
    MatSrc gate_up, down;        // resolved through ids (global scratch)
    const float *sh_inp;         // null = no shared expert
    const uint8_t *sh_gate, *sh_up, *sh_down;
    float *logits;               // [E]
    int32_t *ids;                // [k]
    float *weights;              // [k]
    const int32_t *ids_override; // null or [k]
    float *act;                  // [k+1][F]
    float *shared_gate;          // [1]: logit after A, sigmoid after B
    float *expert_out;           // null or [k][H]
    float *accum, *down_f32, *out;
    float *residual;             // null, [H] (residual += out * residual_scale), or [hc][H] when hc > 0
    float residual_scale;
    const float *hc_inject;      // hc > 0: [hc] inject projections; residual[c] += out * 2 sigmoid(inject[c] / hc)
    int hc, hc_round_half;
    int dry;                     // measurement aid: every workgroup returns at once
    int preselected;
    int n_router_wgs;            // workgroups of dispatch A that take router rows
    int n_routed_items;          // merged dispatch: (expert rung, group of eight rows) items shared by the routed workgroups
    unsigned *arrive;            // device counter of finished router workgroups (zero between dispatches)
    uint32_t *ids_tagged;        // [kTagCopies][16] selected ids published inside the merged dispatch (kTagInvalid = not yet)
    int clear_tagged;            // dispatch C resets ids_tagged when it is done with the layer
    unsigned *status;            // [0] set to 1 when a bounded wait inside a dispatch ran out
    unsigned spin_limit;         // polls (about a microsecond each) before such a wait gives up
    unsigned long long *trace;   // profiling aid: null, or [3][16][8] time stamps (100 MHz) of workgroup trace_wg
    int trace_wg;
    // the PART variants of the dispatches also store the exact int32 chunk sums of the routed rows:
    int32_t *gup_part;           // [k][2][F][8 * H / 256]
    int32_t *down_part;          // [k][H][8 * F / 32]
};

constexpr int kTagCopies = 16;           // replicas of the published ids, 64 bytes apart, so that pollers spread over lines
constexpr uint32_t kTagInvalid = 0xffffffffu;
constexpr unsigned kSpinLimit = 1u << 16;  // default number of polls before a wait gives up (tens of milliseconds; a wait lasts microseconds)

// Time stamp `i` of dispatch `d` (0 = A, 1 = B, 2 = C) for the traced workgroup; lane 0 of every wave.
// TRACE false: compiled out (the kernels that take the stamps as a template parameter run without their tests then).
template <bool TRACE = true>
WD_DEV void mark(const LayerArgs &a, int d, int i) {
    if (!TRACE) return;
    if (a.trace && static_cast<int>(blockIdx.x) == a.trace_wg && (threadIdx.x & 63) == 0 && (threadIdx.x >> 6) < 15)
        a.trace[(d * 16 + (threadIdx.x >> 6)) * 8 + i] = wall_clock64();
}

// ---- in-workgroup quantisers (results in LDS) ------------------------------------------------
// Q8_0 of n values (multiple of 32): four threads per block, eight values per thread.
// The step on eight loaded values (v0, v1 = x[base .. base + 8)); all four threads of a block must call it.
WD_DEV void lds_quantize_q8_0_step(const float4 &v0, const float4 &v1, bool on, int base, int8_t *qs, uint16_t *d, int tid) {
    float amax = __builtin_fmaxf(
        __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v0.x), __builtin_fabsf(v0.y)),
                        __builtin_fmaxf(__builtin_fabsf(v0.z), __builtin_fabsf(v0.w))),
        __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v1.x), __builtin_fabsf(v1.y)),
                        __builtin_fmaxf(__builtin_fabsf(v1.z), __builtin_fabsf(v1.w))));
    amax = quad_max_nonneg(amax);
    if (on) {
        uint2 packed = make_uint2(0u, 0u);
        if (amax != 0.0f) {  // (one division for the eight values)
            const float inv = 127.0f / amax;
            packed.x = q8_0_pack4_scaled(v0, inv);
            packed.y = q8_0_pack4_scaled(v1, inv);
        }
        *reinterpret_cast<uint2 *>(qs + base) = packed;
        if ((tid & 3) == 0) d[base >> 5] = f2h_ref(amax / 127.0f);
    }
}
WD_DEV void lds_quantize_q8_0(const float *__restrict__ x, int n, int8_t *qs, uint16_t *d, int tid, int nthreads) {
    const int per_pass = nthreads * 8;
    for (int base0 = 0; base0 < n; base0 += per_pass) {
        const int base = base0 + tid * 8;
        const bool on = base < n;
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        if (on) {
            v0 = *reinterpret_cast<const float4 *>(x + base);
            v1 = *reinterpret_cast<const float4 *>(x + base + 4);
        }
        lds_quantize_q8_0_step(v0, v1, on, base, qs, d, tid);
    }
}

// Q8_K of one 256-value block by one wave (four values per lane).
WD_DEV void wave_quantize_q8_k_regs(const float4 &v, int8_t *qs256, float *d, int lane);
WD_DEV void wave_quantize_q8_k_block(const float *__restrict__ x256, int8_t *qs256, float *d, int lane) {
    wave_quantize_q8_k_regs(reinterpret_cast<const float4 *>(x256)[lane], qs256, d, lane);
}
// The same on four loaded values per lane (v = x256[4 * lane .. 4 * lane + 4)).
WD_DEV void wave_quantize_q8_k_regs(const float4 &v, int8_t *qs256, float *d, int lane) {
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    amax = wave_max_nonneg(amax);
    uint32_t packed = 0;
    float dv = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -127.0f / amax;
        const int q0 = min(127, static_cast<int>(__builtin_rintf(v.x * iscale)));
        const int q1 = min(127, static_cast<int>(__builtin_rintf(v.y * iscale)));
        const int q2 = min(127, static_cast<int>(__builtin_rintf(v.z * iscale)));
        const int q3 = min(127, static_cast<int>(__builtin_rintf(v.w * iscale)));
        packed = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
        dv = 1.0f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs256)[lane] = packed;
    if (lane == 0) *d = dv;
}

// ---- softmax + top-k by one wave, probabilities kept in registers --------------------------------
// Lane l owns the 8-expert groups l (and l + 64 when M == 2, i.e. more than 512 experts).
// Lanes 0..k-1 write ids/weights through the given pointers (LDS or global).
// src/qwen38_moe.cuh:711-818: softmax over all experts with the per-8 sums accumulated in a double in
// ascending order, k rungs of "largest remaining probability, lowest index on ties", renormalise.
// COHERENT: the logits were written by other workgroups of the same dispatch; they are read with
// device-scope atomic loads so that no stale cached copy can be seen.
// Wave-wide exact sum of doubles (any order gives the same bits when the caller has made sure that the sum is
// exact); the result is uniform.
WD_DEV double wave_sum_exact_f64(double v) {
    auto step = [](double x, auto mover) {
        const uint64_t b = __builtin_bit_cast(uint64_t, x);
        const int lo = mover(static_cast<int>(b & 0xffffffffu)), hi = mover(static_cast<int>(b >> 32));
        return x + __builtin_bit_cast(double, (static_cast<uint64_t>(static_cast<uint32_t>(hi)) << 32) | static_cast<uint32_t>(lo));
    };
    v = step(v, [](int w) { return dpp_i<kDppXor1>(0, w); });
    v = step(v, [](int w) { return dpp_i<kDppXor2>(0, w); });
    v = step(v, [](int w) { return dpp_i<0x141>(0, w); });                     // row_half_mirror: quads 0/1, 2/3 of a row
    v = step(v, [](int w) { return dpp_i<0x140>(0, w); });                     // row_mirror: the two halves of a row
    v = step(v, [](int w) { return dpp_i<kDppBcast15, 0xa, 0xf, true>(0, w); });  // rows 1, 3 += lane 15 of rows 0, 2
    v = step(v, [](int w) { return dpp_i<kDppBcast31, 0xc, 0xf, true>(0, w); });  // rows 2, 3 += lane 31
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(b & 0xffffffffu), 63));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), 63));
    return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}

// Sum of the group sums as the reference takes it (a double accumulated in ascending group order); gs[m] of lane
// l is the sum of group l + 64 m.  When every non-zero group sum is within a factor 2^20 of the largest, all of
// them are multiples of one power of two and every partial sum fits 53 bits, so the result is exact and the same
// in any order: a lane tree then replaces the chain of dependent double additions.
template <int M>
WD_DEV double sum_groups(const float (&gs)[M], int groups, int lane) {
    float gmax = 0.0f, gmin = INFINITY;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        gmax = __builtin_fmaxf(gmax, gs[m]);
        gmin = __builtin_fminf(gmin, gs[m] > 0.0f ? gs[m] : INFINITY);
    }
    gmax = wave_max(gmax);
    gmin = -wave_max(-gmin);
    double sum = 0.0;
    if (gmin >= gmax * 0x1p-20f && gmax < INFINITY) {
        double part = 0.0;
#pragma unroll
        for (int m = 0; m < M; ++m) part += static_cast<double>(gs[m]);
        sum = wave_sum_exact_f64(part);
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m) {
#pragma unroll
            for (int l = 0; l < 64; ++l) {
                const float gl = readlane_f(gs[m], l);
                if (l + 64 * m < groups) sum += static_cast<double>(gl);
            }
        }
    }
    return sum;
}

// Softmax of the row: lane l ends up with the probabilities of its 8-expert group(s) in v (or -inf everywhere
// when every exponential vanished: `dead`).
template <int M, bool COHERENT>
WD_DEV void softmax_probs(const float *logits, int n, int lane, float (&v)[8 * M], bool &dead) {
    const int groups = n >> 3;
    float mx = -INFINITY;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int g = lane + 64 * m;
        if (g < groups) {
            if (COHERENT) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    v[8 * m + i] = __hip_atomic_load(logits + g * 8 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                const float4 a = *reinterpret_cast<const float4 *>(logits + g * 8);
                const float4 b = *reinterpret_cast<const float4 *>(logits + g * 8 + 4);
                v[8 * m + 0] = a.x, v[8 * m + 1] = a.y, v[8 * m + 2] = a.z, v[8 * m + 3] = a.w;
                v[8 * m + 4] = b.x, v[8 * m + 5] = b.y, v[8 * m + 6] = b.z, v[8 * m + 7] = b.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[8 * m + i] = -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) mx = __builtin_fmaxf(mx, v[8 * m + i]);
    }
    mx = wave_max(mx);
    float gs[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const bool on = lane + 64 * m < groups;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[8 * m + i] = on ? exp_ggml(v[8 * m + i] - mx) : 0.0f;
        const float lo = v[8 * m + 0] + v[8 * m + 4], lh = v[8 * m + 2] + v[8 * m + 6];
        const float hi = v[8 * m + 1] + v[8 * m + 5], hh = v[8 * m + 3] + v[8 * m + 7];
        gs[m] = (lo + lh) + (hi + hh);
    }
    const double sum = sum_groups<M>(gs, groups, lane);
    dead = (sum == 0.0);
    const float inv = dead ? 0.0f : static_cast<float>(1.0 / sum);
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const bool on = lane + 64 * m < groups;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[8 * m + i] = (on && !dead) ? v[8 * m + i] * inv : -INFINITY;
    }
}

// k rungs of "largest remaining probability, lowest index on ties" over the probabilities held as by
// softmax_probs; lane j keeps the j-th selected probability and id.
// For a row whose exponentials all vanished every probability is -inf, nothing ever beats the running best of
// -inf, and the reference keeps expert 0 with the value read back from the row.
template <int M>
WD_DEV void rungs_on_probs(float (&v)[8 * M], int k, int lane, float &top_mine, int &id_mine) {
    top_mine = 0.0f;
    id_mine = 0;
    for (int j = 0; j < k; ++j) {
        // this lane's largest remaining probability; lowest slot on ties
        float bv = v[0];
#pragma unroll
        for (int i = 1; i < 8 * M; ++i) bv = __builtin_fmaxf(bv, v[i]);
        int slot = 8 * M - 1;
#pragma unroll
        for (int i = 8 * M - 2; i >= 0; --i) slot = (v[i] == bv) ? i : slot;
        const float best = wave_max(bv);
        int win = 0;
        if (best > -INFINITY) {
            // lowest expert index among the lanes holding `best`: slots of group l come before the
            // slots of group l + 64, and lower lanes before higher ones inside a group row
            const bool mine = bv == best;
            unsigned long long mask = __builtin_amdgcn_ballot_w64(mine && slot < 8);
            if (M == 2 && mask == 0ull) mask = __builtin_amdgcn_ballot_w64(mine);
            const int wl = __builtin_ctzll(mask);
            const int ws = __builtin_amdgcn_readlane(slot, wl);
            win = (wl + 64 * (ws >> 3)) * 8 + (ws & 7);
#pragma unroll
            for (int i = 0; i < 8 * M; ++i) v[i] = (lane == wl && ws == i) ? -INFINITY : v[i];
        }
        if (lane == j) {
            top_mine = best;
            id_mine = win;
        }
    }
}

// Renormalisation: the selected probabilities summed in selection order in a double, clamp, divide, optional
// scale; lanes 0..k-1 write ids/weights through the given pointers (LDS or global).
WD_DEV void finish_weights(float top_mine, int id_mine, int k, float w_scale, int32_t *ids, float *weights,
                           const int32_t *__restrict__ override_ids, int lane) {
    double wsum = 0.0;
    for (int j = 0; j < k; ++j) wsum += static_cast<double>(readlane_f(top_mine, j));
    const float denom = __builtin_fmaxf(static_cast<float>(wsum), 6.103515625e-5f);
    if (lane < k) {
        float wj = top_mine / denom;
        if (w_scale != 0.0f && w_scale != 1.0f) wj = wj * w_scale;
        weights[lane] = wj;
        ids[lane] = override_ids ? override_ids[lane] : id_mine;
    }
}

template <int M, bool COHERENT>
WD_DEV void topk_wave_m(const float *logits, int n, int k, float w_scale, int32_t *ids, float *weights,
                        const int32_t *__restrict__ override_ids, int lane) {
    float v[8 * M];
    bool dead;
    softmax_probs<M, COHERENT>(logits, n, lane, v, dead);
    float top_mine;
    int id_mine;
    rungs_on_probs<M>(v, k, lane, top_mine, id_mine);
    finish_weights(top_mine, id_mine, k, w_scale, ids, weights, override_ids, lane);
}

// The same selection by a workgroup of eight waves (every thread must call it; it contains barriers).
// Expert m * 512 + 64 * wave + lane belongs to (wave, lane): one or two logits per lane.  A wave instruction
// takes four cycles and a chain of k dependent arg-max steps costs about 0.2 us each, so the selection is made by
// thresholding and counting instead:
//   1. every row of 16 lanes publishes its largest logit (32 rows in the workgroup);
//   2. every wave finds T, the smallest of the row maxima that have fewer than k larger ones: at least k logits are
//      >= T, so the k largest are among the candidates {logit >= T} - a few dozen at most for any row that is not
//      nearly constant.  The candidates (logit, exponential, id) are compacted into one list in LDS (ballot, one
//      LDS atomic per wave); meanwhile the exponentials and the per-8 sums (a group is eight consecutive lanes)
//      are computed eight waves wide, and every wave notes its largest exponential outside the candidates;
//   3. wave 0 ranks the candidates by counting (one uniform read and a compare per candidate); rank r < k makes
//      a candidate the r-th selected.  exp is monotone only up to rounding and equal probabilities must go to the
//      lower id, so the result is checked: it is the reference's selection exactly when the probabilities are
//      strictly decreasing and the last one is strictly above every probability left.  The test is made on the
//      exponentials, with a margin that carries it over to the probabilities (see there), so that the ids go out
//      before the denominator is summed.  If it fails (ties - which also make the counted ranks collide -,
//      near-ties, rounding inversions, rows with -inf or NaN, a dead row, more than 64 candidates) wave 0 runs the
//      reference's rungs over the probabilities themselves.
// lds: 4 * (512 * M + 600) bytes of scratch.  The results are written by wave 0 (lanes 0..k-1).
// tagged != null: as soon as the ids are known - before the renormalisation, which only the weights need - id j
// goes to tagged[c * 16 + j] of the `copies` replicas with device-scope atomic stores (the readers poll them).
// Ids given by the caller (override_ids) are requested up front, so their round trip is not behind the selection.
// The three steps as functions of their own, so that a caller with the logits already in registers (or with waves
// that only keep the barriers company) can compose them.  LDS layout of the selection's scratch:
template <int M>
struct TopkLds {
    float *p, *gsum, *rmx, *cl, *ce, *rest, *selp;
    int *cid, *ncand, *sel;
    WD_DEV explicit TopkLds(uint8_t *lds) {
        p = reinterpret_cast<float *>(lds);        // [512 M] exponentials by expert id
        gsum = p + 512 * M;                        // [64 M] per-8 sums by group
        rmx = gsum + 64 * M;                       // [32] largest logit of every row of 16 lanes
        cl = rmx + 32;                             // [64] candidates: logit,
        ce = cl + 64;                              // [64] exponential,
        cid = reinterpret_cast<int *>(ce + 64);    // [64] id
        ncand = cid + 64;                          // [4] their number
        sel = ncand + 4;                           // [16] the r-th selected id
        selp = reinterpret_cast<float *>(sel + 16);  // [16] its exponential
        rest = selp + 16;                          // [8] largest exponential outside the candidates, by wave
    }
};
constexpr int kTopkLdsBytes1 = 4 * (512 + 600), kTopkLdsBytes2 = 4 * (1024 + 600);

// Step 1 (waves 0..7, before the first barrier): the row maxima of the logits held in l[] (expert m * 512 + 64 * wave + lane).
template <int M>
WD_DEV void topk_block_step1(const float (&l)[M], const TopkLds<M> &s, int lane, int wave) {
    if (wave == 0 && lane == 0) s.ncand[0] = 0;
    float lm = l[0];
#pragma unroll
    for (int m = 1; m < M; ++m) lm = __builtin_fmaxf(lm, l[m]);
    lm = __builtin_fmaxf(lm, dpp_f<kDppXor1>(lm, lm));
    lm = __builtin_fmaxf(lm, dpp_f<kDppXor2>(lm, lm));
    lm = __builtin_fmaxf(lm, dpp_f<kDppRor4>(lm, lm));
    lm = __builtin_fmaxf(lm, dpp_f<kDppRor8>(lm, lm));
    if ((lane & 15) == 0) s.rmx[wave * 4 + (lane >> 4)] = lm;
}

// Step 2 (waves 0..7, between the barriers): threshold, exponentials and per-8 sums, candidate list.
template <int M>
WD_DEV void topk_block_step2(const float (&l)[M], int n, int k, const TopkLds<M> &s, int lane, int wave) {
    auto nan_is_large = [](float v) { return v != v ? INFINITY : v; };
    const float r = s.rmx[lane & 31];
    const float mx = wave_max(r);
    float thr;
    {
        int larger = 0;
#pragma unroll
        for (int t = 0; t < 8; ++t) {  // the same 16 bytes for every lane: broadcast reads
            const float4 q = *reinterpret_cast<const float4 *>(s.rmx + 4 * t);
            larger += (q.x > r ? 1 : 0) + (q.y > r ? 1 : 0) + (q.z > r ? 1 : 0) + (q.w > r ? 1 : 0);
        }
        thr = -wave_max(larger < k ? -r : -INFINITY);
    }
    float rme = 0.0f;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int id = m * 512 + wave * 64 + lane;
        const float e = (id < n) ? exp_ggml(l[m] - mx) : 0.0f;
        const float gs = close_lanes8(e);
        if ((lane & 7) == 0) s.gsum[m * 64 + wave * 8 + (lane >> 3)] = gs;
        s.p[id] = e;
        const bool c = l[m] >= thr && l[m] > -INFINITY;
        const unsigned long long cm = __builtin_amdgcn_ballot_w64(c);
        if (cm != 0ull) {
            int base = 0;
            if (lane == 0) base = atomicAdd(s.ncand, static_cast<int>(__builtin_popcountll(cm)));
            base = __builtin_amdgcn_readfirstlane(base);
            const int pos = base + static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(cm >> 32),
                                                        __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(cm), 0u)));
            if (c && pos < 64) {
                s.cl[pos] = l[m];
                s.ce[pos] = e;
                s.cid[pos] = id;
            }
        }
        rme = __builtin_fmaxf(rme, c ? 0.0f : nan_is_large(e));
    }
    rme = wave_max(rme);
    if (lane == 0) s.rest[wave] = rme;
}

// Step 3 (wave 0, after the second barrier): ranks, check, publication of the ids, denominator, weights.
// id_given: the caller's id for lane j < k when the ids are replaced (override), requested before step 1.
template <int M>
WD_DEV void topk_block_step3(int n, int k, float w_scale, int32_t *ids, float *weights, bool override_ids, int id_given,
                             const TopkLds<M> &s, int lane, unsigned long long *stamps, uint32_t *tagged, int copies) {
#define WD_STAMP(i) do { if (stamps && lane == 0) stamps[i] = wall_clock64(); } while (0)
    auto nan_is_large = [](float v) { return v != v ? INFINITY : v; };
    const int groups = n >> 3;
    // ranks of the candidates
    const int nc = s.ncand[0];
    const float got_l = s.cl[lane], got_e = s.ce[lane];  // requested together with the count, not behind it
    const int got_id = s.cid[lane];
    const bool fits = nc <= 64;
    const bool mine = fits && lane < nc;
    const float my_l = mine ? got_l : -INFINITY;
    const float my_e = mine ? got_e : 0.0f;
    const int my_id = mine ? got_id : -1;
    if (lane < 16) s.sel[lane] = -1;
    int rk = 0;
    const int steps = fits ? (nc + 3) & ~3 : 0;  // lanes past the list hold -inf, which is ahead of nothing
    for (int src = 0; src < steps; src += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) rk += (readlane_f(my_l, src + u) > my_l) ? 1 : 0;
    }
    wave_lds_fence();
    if (mine && rk < k) {
        s.sel[rk] = my_id;  // equal logits collide here; the loser stays among the rest and fails the test below
        s.selp[rk] = my_e;
    }
    wave_lds_fence();
    const bool taken = mine && rk < k && s.sel[rk < k ? rk : 0] == my_id;
    float rest_all = wave_max((mine && !taken) ? nan_is_large(my_e) : 0.0f);
#pragma unroll
    for (int w = 0; w < 8; ++w) rest_all = __builtin_fmaxf(rest_all, s.rest[w]);
    if (!fits) rest_all = INFINITY;
    WD_STAMP(3);

    // The ids do not wait for the denominator: p = e * inv with one inv in [2^-10, 1] for the whole row is
    // monotone in e, and two exponentials that differ by more than a few units in the last place (and are not
    // tiny) cannot round to the same product, so this test on the exponentials implies the one on the
    // probabilities.  A NaN counts as larger than everything.
    const int idc = (lane < k) ? s.sel[lane] : -1;
    const bool have = idc >= 0 && idc < n;
    const float top_e = have ? s.selp[lane] : 0.0f;
    const float nxt = dpp_f<kDppShl1>(0.0f, top_e);  // k <= 16: the selected sit in one row of lanes
    const float below = (lane == k - 1 ? rest_all : nxt) * 1.000001f;
    const bool good = lane >= k || (have && top_e >= 0x1p-100f && top_e > below);
    const bool all_good = __builtin_amdgcn_ballot_w64(good) == ~0ull;
    int id_mine = override_ids ? id_given : idc;
    if (all_good && tagged) {
        // the ids (lanes 0..k-1, k <= 16) into every row of 16 lanes, then four replicas per store instruction: the last
        // replica goes out a quarter of the stores after the first
        const wd_uint2v t16 = __builtin_amdgcn_permlane16_swap(static_cast<uint32_t>(id_mine), static_cast<uint32_t>(id_mine), false, false);
        const wd_uint2v t32 = __builtin_amdgcn_permlane32_swap(t16.x, t16.x, false, false);
        const int j = lane & 15, c4 = lane >> 4;
#pragma unroll 4
        for (int c0 = 0; c0 < copies; c0 += 4)
            if (j < k && c0 + c4 < copies)
                __hip_atomic_store(tagged + (c0 + c4) * 16 + j, t32.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    WD_STAMP(6);

    // the denominator (only the weights and the slow path need it)
    float gs[M];
#pragma unroll
    for (int m = 0; m < M; ++m) gs[m] = (lane + 64 * m < groups) ? s.gsum[m * 64 + lane] : 0.0f;
    const double sum = sum_groups<M>(gs, groups, lane);
    const float inv = (sum == 0.0) ? 0.0f : static_cast<float>(1.0 / sum);
    const bool dead = sum == 0.0;
    float top_mine = top_e * inv;
    if (!all_good) {
        float v[8 * M];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int ix = (lane + 64 * m) * 8 + i;
                v[8 * m + i] = (ix < n && !dead) ? s.p[ix] * inv : -INFINITY;
            }
        rungs_on_probs<M>(v, k, lane, top_mine, id_mine);
        if (override_ids) id_mine = id_given;
        if (tagged && lane < k) {
#pragma unroll 4
            for (int c = 0; c < copies; ++c)
                __hip_atomic_store(tagged + c * 16 + lane, static_cast<uint32_t>(id_mine), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    finish_weights(top_mine, id_mine, k, w_scale, ids, weights, nullptr, lane);
    WD_STAMP(7);
#undef WD_STAMP
}

template <int M>
WD_DEV void topk_block_m(const float *logits, int n, int k, float w_scale, int32_t *ids, float *weights,
                         const int32_t *__restrict__ override_ids, uint8_t *lds, int lane, int wave,
                         unsigned long long *stamps = nullptr, uint32_t *tagged = nullptr, int copies = 0) {
#define WD_STAMP(i) do { if (stamps && wave == 0 && lane == 0) stamps[i] = wall_clock64(); } while (0)
    const TopkLds<M> s(lds);
    WD_STAMP(0);
    int id_given = 0;
    if (override_ids && wave == 0 && lane < k) id_given = override_ids[lane];
    float l[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int id = m * 512 + wave * 64 + lane;
        l[m] = (id < n) ? __hip_atomic_load(logits + id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -INFINITY;
    }
    topk_block_step1<M>(l, s, lane, wave);
    __syncthreads();
    WD_STAMP(1);
    topk_block_step2<M>(l, n, k, s, lane, wave);
    __syncthreads();
    WD_STAMP(2);
    if (wave == 0)
        topk_block_step3<M>(n, k, w_scale, ids, weights, override_ids != nullptr, id_given, s, lane, stamps, tagged, copies);
#undef WD_STAMP
}

WD_DEV void topk_block(const float *logits, int n, int k, float w_scale, int32_t *ids, float *weights,
                       const int32_t *__restrict__ override_ids, uint8_t *lds, int lane, int wave,
                       unsigned long long *stamps = nullptr, uint32_t *tagged = nullptr, int copies = 0) {
    if (n <= 512)
        topk_block_m<1>(logits, n, k, w_scale, ids, weights, override_ids, lds, lane, wave, stamps, tagged, copies);
    else
        topk_block_m<2>(logits, n, k, w_scale, ids, weights, override_ids, lds, lane, wave, stamps, tagged, copies);
}

template <bool COHERENT>
WD_DEV void topk_wave(const float *logits, int n, int k, float w_scale, int32_t *ids, float *weights,
                      const int32_t *__restrict__ override_ids, int lane) {
    if (n <= 512)
        topk_wave_m<1, COHERENT>(logits, n, k, w_scale, ids, weights, override_ids, lane);
    else
        topk_wave_m<2, COHERENT>(logits, n, k, w_scale, ids, weights, override_ids, lane);
}

// ---- the same selection by ONE wave that holds eight logits per lane ------------------------------------------------
// lv[j] is the logit of expert 64 j + lane (-inf at and beyond n; n <= 512, k <= 15).  A single wave pays for every trip
// through LDS or the scalar unit with hundreds of idle cycles, so step A stays in the vector registers: every logit
// becomes a 32-bit key - its bits mapped so that unsigned order is float order, the low nine bits replaced by
// 511 - expert - , every lane sorts its eight keys (a network of 19 exchanges), and k + 1 rounds of "largest head of any
// lane" (a DPP reduction; the lane that held it moves its keys up) give the k + 1 largest keys in order, key j in
// lane j.  The keys order the logits up to their low nine bits, so the result is accepted as the selection only when
//   * the keys' upper 23 bits are strictly decreasing over the k + 1 - any logit that was not taken then lies below
//     the grid point at or below the k-th taken logit -, and
//   * the exponentials e_0 > e_1 > ... > e_k of the k + 1 exact logits are strictly decreasing by a relative margin:
//     exp_ggml is within two units in the last place of the true exponential (relative error below 2^-22) on normal
//     results, so every logit not above the (k+1)-th has an exponential below e_k (1 + 2^-21), and
//     e_(k-1) > e_k (1 + 2^-18) puts the k-th selected strictly above everything left, also after the product with the
//     row's 1/sum has been rounded.
// Rows the test does not accept (ties, near-ties, NaN, +inf, fewer than k + 1 finite logits, selected exponentials below
// 2^-100) take the reference's rungs over all probabilities in step B.
struct SelWaveState {
    float mx;      // the row's largest logit
    float e;       // lane j <= k: exponential of the j-th largest logit (accepted rows)
    int id;        // lane j <= k: its expert
    bool fast;     // step A accepted the row (the same in every lane)
};

WD_DEV uint32_t wave_max_u32(uint32_t v) {  // the result is uniform
    // (umax_step: written so that the shuffle and the maximum become one instruction)
    v = umax_step<kDppXor1>(v);
    v = umax_step<kDppXor2>(v);
    v = umax_step<kDppRor4>(v);
    v = umax_step<kDppRor8>(v);  // every lane: its row's largest
    const wd_uint2v t = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    v = max(t.x, t.y);                                                                            // rows 0|2 and 1|3
    return max(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 0)),
               static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 16)));
}

// Step A.  Returns with st.fast, and for accepted rows the ids of the selection in lanes 0..k-1 of st.id.
// Registers and cross-lane moves only: no LDS is written or read.
WD_DEV void sel_wave_ids(const float (&lv)[8], int n, int k, int lane, SelWaveState &st) {
    uint32_t h[8];
    bool odd = false;
    float lm = lv[0];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int id = 64 * j + lane;
        odd = odd || lv[j] != lv[j];
        lm = __builtin_fmaxf(lm, lv[j]);
        const uint32_t b = f_bits(lv[j]);
        const uint32_t ord = b ^ ((b & 0x80000000u) ? 0xffffffffu : 0x80000000u);  // unsigned order = float order
        h[j] = id < n ? ((ord & ~0x1ffu) | static_cast<uint32_t>(511 - id)) : 0u;
    }
    const float mx = wave_max(lm);
    auto exchange = [&](int i, int j) {  // the larger key to the lower register
        const uint32_t hi = max(h[i], h[j]), lo = min(h[i], h[j]);
        h[i] = hi, h[j] = lo;
    };
    exchange(0, 1), exchange(2, 3), exchange(4, 5), exchange(6, 7);
    exchange(0, 2), exchange(1, 3), exchange(4, 6), exchange(5, 7);
    exchange(1, 2), exchange(5, 6);
    exchange(0, 4), exchange(1, 5), exchange(2, 6), exchange(3, 7);
    exchange(2, 4), exchange(3, 5);
    exchange(1, 2), exchange(3, 4), exchange(5, 6);
    uint32_t mine = 0u;  // lane j: the j-th largest key of the row
    for (int j = 0; j <= k; ++j) {
        const uint32_t m = wave_max_u32(h[0]);
        const bool won = h[0] == m;  // (keys are distinct: they end in the expert's number)
#pragma unroll
        for (int i = 0; i < 7; ++i) h[i] = won ? h[i + 1] : h[i];
        h[7] = won ? 0u : h[7];
        mine = lane == j ? m : mine;
    }
    // the exact logit behind key j: register idc / 64 of lane idc % 64
    const int idc = 511 - static_cast<int>(mine & 0x1ffu);
    const bool have = lane <= k && mine != 0u && idc < n;
    float l = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float from = __shfl(lv[j], idc & 63, kWave);
        l = (have && (idc >> 6) == j) ? from : l;
    }
    const float e = (have && l > -INFINITY) ? exp_ggml(l - mx) : 0.0f;
    const float nxt = dpp_f<kDppShl1>(0.0f, e);  // k + 1 <= 16: these lanes are one row
    const uint32_t grid = mine >> 9, grid_nxt = static_cast<uint32_t>(dpp_i<kDppShl1>(0, static_cast<int>(grid)));
    const bool good = lane > k || (have && l > -INFINITY &&
                                   (lane == k || (grid > grid_nxt && e >= 0x1p-100f && e > nxt * (lane == k - 1 ? 1.000004f : 1.000001f))));
    st.mx = mx, st.e = e, st.id = idc;
    st.fast = __builtin_amdgcn_ballot_w64(odd) == 0ull && mx < INFINITY && __builtin_amdgcn_ballot_w64(good) == ~0ull;
}

// Step B, first half (any wave that holds the logits; it need not be the wave of step A): every exponential into s.p,
// the per-8 sums, and the row's 1/sum as the reference takes it (0 for a row whose exponentials all vanished: `dead`).
WD_DEV float sel_wave_denominator(const float (&lv)[8], int n, const TopkLds<1> &s, int lane, bool &dead) {
    const int groups = n >> 3;
    float lm = lv[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) lm = __builtin_fmaxf(lm, lv[j]);
    const float mx = wave_max(lm);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int id = 64 * j + lane;
        const float e = (id < n) ? exp_ggml(lv[j] - mx) : 0.0f;
        const float gs = close_lanes8(e);
        if ((lane & 7) == 0) s.gsum[8 * j + (lane >> 3)] = gs;
        s.p[id] = e;
    }
    wave_lds_fence();
    const float g1[1] = {lane < groups ? s.gsum[lane] : 0.0f};
    const double sum = sum_groups<1>(g1, groups, lane);
    dead = sum == 0.0;
    return dead ? 0.0f : static_cast<float>(1.0 / sum);
}

// Step B, second half (the wave of step A; s.p and inv as the first half left them, which may have been another wave
// on the far side of a barrier): for rows step A did not accept the reference's rungs over the probabilities; then lanes
// 0..k-1 write the weights and the ids (ids_given: id_given instead).
WD_DEV void sel_wave_weights(int n, int k, float w_scale, const TopkLds<1> &s, int lane, SelWaveState &st, float inv, bool dead,
                             int32_t *ids, float *weights, bool ids_given, int id_given) {
    float top_mine = st.e * inv;
    int id_mine = st.id;
    if (!st.fast) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int ix = lane * 8 + i;
            v[i] = (ix < n && !dead) ? s.p[ix] * inv : -INFINITY;
        }
        rungs_on_probs<1>(v, k, lane, top_mine, id_mine);
        st.id = id_mine;
    }
    finish_weights(top_mine, ids_given ? id_given : id_mine, k, w_scale, ids, weights, nullptr, lane);
}

// Stand-alone softmax/top-k dispatch: one wave (src/qwen38_moe.cuh:711-818).
// If gate_logit != null, gate_logit[0] is replaced by sigmoid_ggml(gate_logit[0]) (shared expert gate).
// If override_ids != null the selected ids are replaced by override_ids[0..k) after the weights are formed.
__global__ __launch_bounds__(64) void k_topk_softmax(const float *__restrict__ logits, int n, int k, float w_scale,
                                                      int32_t *__restrict__ ids, float *__restrict__ weights,
                                                      float *__restrict__ gate_logit,
                                                      const int32_t *__restrict__ override_ids) {
    const int lane = threadIdx.x;
    if (gate_logit && lane == 0) gate_logit[0] = sigmoid_ggml(gate_logit[0]);
    if (n <= 512 && k <= 15) {  // threshold and ranks first, the reference's rungs for the rows that need them
        __shared__ __align__(16) uint8_t s_sel[kTopkLdsBytes1];
        const TopkLds<1> s(s_sel);
        float lv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) lv[j] = (64 * j + lane < n) ? logits[64 * j + lane] : -INFINITY;
        SelWaveState st;
        sel_wave_ids(lv, n, k, lane, st);
        int id_given = 0;
        if (override_ids && lane < k) id_given = override_ids[lane];
        bool dead;
        const float inv = sel_wave_denominator(lv, n, s, lane, dead);
        sel_wave_weights(n, k, w_scale, s, lane, st, inv, dead, ids, weights, override_ids != nullptr, id_given);
        return;
    }
    topk_wave<false>(logits, n, k, w_scale, ids, weights, override_ids, lane);
}

// ---- router rows: 32 lanes per row, 8 rows per 256-thread workgroup ---------------------------------
// All loads of a 2048-column span are issued before the first multiply-add, so one HBM round trip
// covers the span; the multiply-add chain of each accumulator still runs in ascending column order.
// COHERENT: results are published with device-scope atomic stores (another workgroup of the same
// dispatch reads them).
template <bool COHERENT>
WD_DEV void router_rows(const float *__restrict__ w, const float *__restrict__ x, float *logits, int rows, int cols,
                        const float *__restrict__ extra_w, float *extra_out, int wg) {
    const int t = threadIdx.x & 31;
    const int row = wg * static_cast<int>(blockDim.x >> 5) + (threadIdx.x >> 5);
    const int total = rows + (extra_w ? 1 : 0);
    const bool on = row < total;
    const float *wr = on ? (row < rows ? w + static_cast<size_t>(row) * cols : extra_w) : x;
    const int np = cols & ~31;
    float s = 0.0f;
    if (on) {
        for (int i0 = 0; i0 < np; i0 += 2048) {
            float wv[64], xv[64];
#pragma unroll
            for (int u = 0; u < 64; ++u) {
                const int i = i0 + 32 * u + t;
                if (i0 + 32 * u < np) {
                    wv[u] = wr[i];
                    xv[u] = x[i];
                }
            }
#pragma unroll
            for (int u = 0; u < 64; ++u)
                if (i0 + 32 * u < np) s = __builtin_fmaf(wv[u], xv[u], s);
        }
    }
    float o = __shfl_down(s, 16, 32);
    if (t < 16) s = s + o;
    o = __shfl_down(s, 8, 32);
    if (t < 8) s = s + o;
    o = __shfl_down(s, 4, 32);
    if (t < 4) s = s + o;
    o = __shfl_down(s, 1, 32);
    if (t == 0 || t == 2) s = s + o;
    o = __shfl_down(s, 2, 32);
    float acc = s + o;
    if (on && t == 0) {
        for (int c = np; c < cols; ++c) acc = acc + wr[c] * x[c];
        float *dst = (row < rows) ? logits + row : extra_out;
        if (COHERENT)
            __hip_atomic_store(dst, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            *dst = acc;
    }
}

// Router rows for the merged dispatch: one row per wave, x staged once per workgroup in LDS (f32 [cols]).
// Accumulator t (of ggml's 4 x 8) of the row lives in lanes t and t + 32: for every span of 2048 columns lane t
// runs the multiply-adds of columns [span, span + 1024) and hands the value to lane t + 32, which continues with
// [span + 1024, span + 2048) and hands it back for the next span, so each chain still sees its columns in
// ascending order while a lane holds only 32 weights (half the registers of the 32-lanes-per-row version,
// which lets three workgroups of the merged dispatch share a compute unit).
// Every thread of the workgroup must call it (it contains a barrier).
// SCALAR_ROW: keep the wave's row pointer in scalar registers (two vector registers fewer).
template <bool COHERENT, bool SCALAR_ROW = false>
WD_DEV void router_rows_wave(const float *__restrict__ w, const float *__restrict__ x, float *xs, float *logits, int rows,
                             int cols, const float *__restrict__ extra_w, float *extra_out, int wg) {
    const int lane = threadIdx.x & 63, t = lane & 31;
    const bool upper = lane >= 32;
    const int row = wg * static_cast<int>(blockDim.x >> 6) + static_cast<int>(threadIdx.x >> 6);
    const int total = rows + (extra_w ? 1 : 0);
    const bool on = row < total;
    const float *wr = on ? (row < rows ? w + static_cast<size_t>(row) * cols : extra_w) : x;
    if (SCALAR_ROW) {  // the row is the same for the whole wave
        const uintptr_t v = reinterpret_cast<uintptr_t>(wr);
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        wr = reinterpret_cast<const float *>((static_cast<uintptr_t>(hi) << 32) | lo);
    }
    const int np = cols & ~31;
    const int half_off = (upper ? 1024 : 0) + t;
    float wv[32];
    if (on) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            const int c = half_off + 32 * u;
            wv[u] = (c < np) ? wr[c] : 0.0f;
        }
    }
    for (int i = static_cast<int>(threadIdx.x) * 4; i < cols; i += static_cast<int>(blockDim.x) * 4) {
        if (i + 4 <= cols) {
            *reinterpret_cast<float4 *>(xs + i) = *reinterpret_cast<const float4 *>(x + i);
        } else {
            for (int c = i; c < cols; ++c) xs[c] = x[c];
        }
    }
    __syncthreads();
    float s = 0.0f;  // the chain value; valid in the half that ran last
    if (on) {
        for (int i0 = 0; i0 < np; i0 += 2048) {
            if (i0 > 0) {
#pragma unroll
                for (int u = 0; u < 32; ++u) {
                    const int c = i0 + half_off + 32 * u;
                    wv[u] = (c < np) ? wr[c] : 0.0f;
                }
            }
            // this lane's 32 multiply-adds of the span, continuing the chain from `start`
            auto run_half = [&](float start) {
                float v = start;
#pragma unroll
                for (int ub = 0; ub < 32; ub += 8) {
                    float xv[8];
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        const int c = i0 + half_off + 32 * (ub + q);
                        xv[q] = xs[c < np ? c : 0];
                    }
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        const int c = i0 + half_off + 32 * (ub + q);
                        const float nv = __builtin_fmaf(wv[ub + q], xv[q], v);
                        v = (c < np) ? nv : v;
                    }
                }
                return v;
            };
            // the lower half advances the chain (from the upper half's value of the previous span) ...
            const wd_uint2v back = __builtin_amdgcn_permlane32_swap(f_bits(s), f_bits(s), false, false);
            if (!upper) s = run_half(i0 == 0 ? 0.0f : bits_f(back.y));
            // ... and the upper half continues from its result
            const wd_uint2v fwd = __builtin_amdgcn_permlane32_swap(f_bits(s), f_bits(s), false, false);
            if (upper) s = run_half(bits_f(fwd.x));
        }
    }
    // the 32 accumulators are final in the upper half (lanes 32..63): ggml's closing tree
    float o = __shfl_down(s, 16, 32);
    if (t < 16) s = s + o;
    o = __shfl_down(s, 8, 32);
    if (t < 8) s = s + o;
    o = __shfl_down(s, 4, 32);
    if (t < 4) s = s + o;
    o = __shfl_down(s, 1, 32);
    if (t == 0 || t == 2) s = s + o;
    o = __shfl_down(s, 2, 32);
    float acc = s + o;
    if (on && lane == 32) {
        for (int c = np; c < cols; ++c) acc = acc + wr[c] * xs[c];
        float *dst = (row < rows) ? logits + row : extra_out;
        if (COHERENT)
            __hip_atomic_store(dst, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            *dst = acc;
    }
}

// The same for rows of 2049..4096 columns, two waves per row: wave 2 w takes the first 2048 columns of row (4 wg + w),
// wave 2 w + 1 the rest, both with every load of theirs in flight from the start - one trip to memory instead of one per
// span.  The chains still see their columns in ascending order: the second wave starts from the 32 accumulators the
// first one leaves in LDS (`hand`: 4 x 32 floats).  Every thread of the (512-thread) workgroup must call it.
WD_DEV void router_rows_wave_pair(const float *__restrict__ w, const float *__restrict__ x, float *xs, float *hand, float *logits,
                                  int rows, int cols, const float *__restrict__ extra_w, float *extra_out, int wg) {
    const int lane = threadIdx.x & 63, t = lane & 31, wave = static_cast<int>(threadIdx.x >> 6);
    const bool upper = lane >= 32, second = (wave & 1) != 0;
    const int row = wg * 4 + (wave >> 1);
    const int total = rows + (extra_w ? 1 : 0);
    const bool on = row < total;
    const float *wr = on ? (row < rows ? w + static_cast<size_t>(row) * cols : extra_w) : x;
    const int np = cols & ~31;
    const int c0 = (second ? 2048 : 0) + (upper ? 1024 : 0) + t;  // this lane's first column
    float wv[32];
    if (on) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            const int c = c0 + 32 * u;
            wv[u] = (c < np) ? wr[c] : 0.0f;
        }
    }
    for (int i = static_cast<int>(threadIdx.x) * 4; i < cols; i += static_cast<int>(blockDim.x) * 4) {
        if (i + 4 <= cols) {
            *reinterpret_cast<float4 *>(xs + i) = *reinterpret_cast<const float4 *>(x + i);
        } else {
            for (int c = i; c < cols; ++c) xs[c] = x[c];
        }
    }
    __syncthreads();
    auto run_half = [&](float start) {
        float v = start;
#pragma unroll
        for (int ub = 0; ub < 32; ub += 8) {
            float xv[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int c = c0 + 32 * (ub + q);
                xv[q] = xs[c < np ? c : 0];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int c = c0 + 32 * (ub + q);
                const float nv = __builtin_fmaf(wv[ub + q], xv[q], v);
                v = (c < np) ? nv : v;
            }
        }
        return v;
    };
    // one copy of the chain code for both waves of a pair: turn 0 is the first wave's, turn 1 the second's
    float s = 0.0f;
#pragma unroll 1
    for (int turn = 0; turn < 2; ++turn) {
        if (second == (turn == 1)) {
            const float start = s;
            if (on && !upper) s = run_half(start);
            const wd_uint2v fwd = __builtin_amdgcn_permlane32_swap(f_bits(s), f_bits(s), false, false);
            if (upper) s = on ? run_half(bits_f(fwd.x)) : bits_f(fwd.x);
        }
        if (turn == 0) {
            if (!second && upper) hand[(wave >> 1) * 32 + t] = s;
            __syncthreads();
            if (second) s = hand[(wave >> 1) * 32 + t];
        }
    }
    if (!second) return;
    // the 32 accumulators are final in the upper half (lanes 32..63): ggml's closing tree
    float o = __shfl_down(s, 16, 32);
    if (t < 16) s = s + o;
    o = __shfl_down(s, 8, 32);
    if (t < 8) s = s + o;
    o = __shfl_down(s, 4, 32);
    if (t < 4) s = s + o;
    o = __shfl_down(s, 1, 32);
    if (t == 0 || t == 2) s = s + o;
    o = __shfl_down(s, 2, 32);
    float acc = s + o;
    if (on && lane == 32) {
        for (int c = np; c < cols; ++c) acc = acc + wr[c] * xs[c];
        float *dst = (row < rows) ? logits + row : extra_out;
        __hip_atomic_store(dst, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- dispatch A -----------------------------------------------------------------------------------------
// grid = n_router_wgs + ceil(F / 8) (the second part only with a shared expert); 512 threads.
// Router workgroups: 16 rows each.  Shared-expert workgroups: 8 (gate, up) row pairs, one per wave.
// dynamic LDS: H bytes + H/32 halves for the Q8_0 copy of x.
//
// Hand-off to the selecting workgroup: logits are published with device-scope atomic stores, each
// workgroup then waits for its stores to complete and bumps a counter with a relaxed device-scope
// atomic; the workgroup that reads n_router_wgs - 1 knows every logit is complete and reads them
// with device-scope atomic loads.  No cache-wide release/acquire is needed for 2 KB of data.
__global__ __launch_bounds__(512) void k_layer_a(LayerArgs a) {
    extern __shared__ __align__(16) uint8_t lds_a[];
    __shared__ Q8RowTile tiles[8];
    __shared__ int s_last;
    const int wg = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (a.dry) return;
    mark(a, 0, 0);
    if (wg < a.n_router_wgs) {
        router_rows<true>(a.router, a.x, a.logits, a.preselected ? 0 : a.E, a.H, a.sh_inp, a.shared_gate, wg);
        mark(a, 0, 1);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0)
            s_last = (__hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      static_cast<unsigned>(a.n_router_wgs - 1));
        __syncthreads();
        if (s_last && wave == 0) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            if (a.trace && lane == 0) a.trace[(0 * 16 + 8) * 8 + 0] = wall_clock64();
            if (!a.preselected) topk_wave<true>(a.logits, a.E, a.k, a.w_scale, a.ids, a.weights, a.ids_override, lane);
            if (lane == 0) {
                if (a.sh_inp) {
                    const float g = __hip_atomic_load(a.shared_gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    a.shared_gate[0] = sigmoid_ggml(g);
                }
                a.arrive[0] = 0u;
            }
            if (a.trace && lane == 0) a.trace[(0 * 16 + 8) * 8 + 1] = wall_clock64();
        }
        mark(a, 0, 2);
        return;
    }
    int8_t *xq = reinterpret_cast<int8_t *>(lds_a);
    uint16_t *xd = reinterpret_cast<uint16_t *>(lds_a + a.H);
    const int r = (wg - a.n_router_wgs) * 8 + wave;
    const int nb = a.H >> 5;
    const size_t rb = static_cast<size_t>(nb) * 34;
    const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
    const uint8_t *const rows[2] = {a.sh_gate + off, a.sh_up + off};
    float gu[2];
    q8_row_wave<2>(rows, nb, xq, xd, tiles[wave], lane, gu, [&]() {
        lds_quantize_q8_0(a.x, a.H, xq, xd, threadIdx.x, 512);
        __syncthreads();
        mark(a, 0, 2);
    });
    if (lane == 0 && r < a.F) a.act[static_cast<size_t>(a.k) * a.F + r] = silu_ggml(gu[0]) * gu[1];
    mark(a, 0, 3);
}

// ---- dispatches A and B in one launch ---------------------------------------------------------------------
// Workgroups [0, n_router_wgs): router rows, the last one to finish selects the experts and publishes the ids;
// then ceil(F / 8) workgroups for the shared expert's gate/up; then k * ceil(F / 8) workgroups for the routed
// gate/up.  The routed workgroups are dispatched after the router ones (lower block index first), quantise x and
// stage the codebooks while the router runs, then poll the published ids; as soon as these appear they request
// their weights.  This removes a launch, a round trip for the ids and the serial activation set-up from the
// critical path of the layer.
//
// Publication: id j goes, as one 32-bit word, to ids_tagged[c][j] of every replica c with a device-scope atomic
// store; a word other than kTagInvalid is the id itself, so a reader needs no second flag.  The words are reset
// to kTagInvalid by dispatch C (or by the caller) before the next layer pass uses them.  The wait is bounded:
// when it runs out the workgroup sets status[0] and returns.
// COAL (IQ types): rows of eight super-blocks on 16-byte boundaries are fetched with one aligned 16-byte load per
// lane and parked in LDS (iq_rows8_coal); dynamic LDS then has 8 * 2 * kIqStageBytes more bytes behind the 4 * H + 16.
// NB (COAL only): super-blocks per row, 8 (hidden 2048) or 10 (hidden 2560).
// LOOP: the grid has fewer routed workgroups than there are (expert rung, group of eight rows) items; they walk them
// with the stride of their number.
template <int TYPE, bool COAL, int NB = 8, bool LOOP = false, bool PART = false, bool TRACE = false>
__global__ __launch_bounds__(512, 6) void k_layer_ab(LayerArgs a) {
    constexpr bool kIq = (TYPE == 21 || TYPE == 22);
    extern __shared__ __align__(16) uint8_t lds_ab[];
    __shared__ __align__(16) uint8_t s_union[sizeof(Q8RowTile) * 8 > sizeof(IqTables) ? sizeof(Q8RowTile) * 8 : sizeof(IqTables)];
    __shared__ int s_last;
    const int wg = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (a.dry) return;
    const int groups = (a.F + 7) / 8;
    const int n_shared_wgs = a.sh_inp ? groups : 0;

    mark<TRACE>(a, wg < a.n_router_wgs + n_shared_wgs ? 0 : 1, 0);
    if (wg < a.n_router_wgs) {
        if (COAL && NB == 10)  // rows of 2560 columns: two waves per row, four rows per workgroup (the host sizes the grid for it)
            router_rows_wave_pair(a.router, a.x, reinterpret_cast<float *>(lds_ab), reinterpret_cast<float *>(s_union), a.logits, a.E,
                                  a.H, a.sh_inp, a.shared_gate, wg);
        else
            router_rows_wave<true>(a.router, a.x, reinterpret_cast<float *>(lds_ab), a.logits, a.E, a.H, a.sh_inp,
                                   a.shared_gate, wg);
        mark<TRACE>(a, 0, 1);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0)
            s_last = (__hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      static_cast<unsigned>(a.n_router_wgs - 1));
        __syncthreads();
        if (s_last) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            if (TRACE && a.trace && threadIdx.x == 0) a.trace[(0 * 16 + 8) * 8 + 0] = wall_clock64();
            // results land behind the selection's own scratch
            static_assert(sizeof(s_union) >= kTopkLdsBytes2 + 128, "selection scratch, ids and weights must fit the shared area");
            int32_t *lds_ids = reinterpret_cast<int32_t *>(s_union + kTopkLdsBytes2);
            float *lds_w = reinterpret_cast<float *>(s_union + kTopkLdsBytes2 + 64);
            // the selection itself publishes the replicas that the routed workgroups wait for, ahead of the weights
            topk_block(a.logits, a.E, a.k, a.w_scale, lds_ids, lds_w, a.ids_override, s_union, lane, wave,
                       (TRACE && a.trace) ? a.trace + (0 * 16 + 9) * 8 : nullptr, a.ids_tagged, kTagCopies);
            if (wave == 0) {
                wave_lds_fence();
                // the plain copies for dispatch C
                if (lane < a.k) {
                    a.ids[lane] = lds_ids[lane];
                    a.weights[lane] = lds_w[lane];
                }
                if (TRACE && a.trace && lane == 0) a.trace[(0 * 16 + 8) * 8 + 1] = wall_clock64();
            } else if (wave == 5 && lane == 0) {
                // off the selection's path: the shared expert's gate, and the counter for the next layer pass
                if (a.sh_inp) {
                    const float g = __hip_atomic_load(a.shared_gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    a.shared_gate[0] = sigmoid_ggml(g);
                }
                a.arrive[0] = 0u;
            }
        }
        mark<TRACE>(a, 0, 2);
        return;
    }

    int8_t *xq = reinterpret_cast<int8_t *>(lds_ab);
    uint8_t *xscale = lds_ab + a.H;  // Q8_K: f32 [H/256]; Q8_0: f16 [H/32]
    if (wg < a.n_router_wgs + n_shared_wgs) {
        Q8RowTile *tiles = reinterpret_cast<Q8RowTile *>(s_union);
        const int r = (wg - a.n_router_wgs) * 8 + wave;
        const int nb = a.H >> 5;
        const size_t rb = static_cast<size_t>(nb) * 34;
        const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
        const uint8_t *const rows[2] = {uniform_ptr(a.sh_gate + off), uniform_ptr(a.sh_up + off)};  // one row pair per wave
        float gu[2];
        q8_row_wave<2>(rows, nb, xq, reinterpret_cast<const uint16_t *>(xscale), tiles[wave], lane, gu, [&]() {
            lds_quantize_q8_0(a.x, a.H, xq, reinterpret_cast<uint16_t *>(xscale), threadIdx.x, 512);
            __syncthreads();
        });
        if (lane == 0 && r < a.F) a.act[static_cast<size_t>(a.k) * a.F + r] = silu_ggml(gu[0]) * gu[1];
        return;
    }

    // routed gate/up: set-up that does not need the ids
    const int bw = wg - a.n_router_wgs - n_shared_wgs;
    IqTables &tables = *reinterpret_cast<IqTables *>(s_union);
    if (kIq) {
        stage_tables<TYPE == 21, TYPE == 22>(tables, threadIdx.x, 512);
        for (int b = wave; b < (a.H >> 8); b += 8)
            wave_quantize_q8_k_block(a.x + b * 256, xq + b * 256, reinterpret_cast<float *>(xscale) + b, lane);
    } else {
        lds_quantize_q8_0(a.x, a.H, xq, reinterpret_cast<uint16_t *>(xscale), threadIdx.x, 512);
    }
    mark<TRACE>(a, 1, 1);
    __shared__ int s_expert;
    const int n_routed_wgs = LOOP ? static_cast<int>(gridDim.x) - a.n_router_wgs - n_shared_wgs : 0;
    int item = bw;
    do {  // one item per workgroup unless the grid was capped (LOOP)
        const int j = item / groups;
        const int rg = item - j * groups;
        if (threadIdx.x == 0) {
            const uint32_t *src = a.ids_tagged + (bw & (kTagCopies - 1)) * 16 + j;
            uint32_t e = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned polls = 0;
            while (e == kTagInvalid && ++polls < a.spin_limit) {
                __builtin_amdgcn_s_sleep(4);
                e = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (e == kTagInvalid) __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_expert = static_cast<int>(e);
        }
        __syncthreads();
        mark<TRACE>(a, 1, 2);
        const int e = s_expert;
        if (e < 0 || e >= a.E) return;  // the wait ran out (status is set): leave without touching memory
        const uint8_t *gate = mat_ptr_expert<0>(a.gate_up, e);
        const uint8_t *up = mat_ptr_expert<1>(a.gate_up, e);
        float *act = a.act + static_cast<size_t>(j) * a.F;
        const int r = rg * 8 + wave;
        float gu[2];
        if (kIq) {
            const int nb = a.H >> 8;
            const size_t rb = static_cast<size_t>(nb) * (TYPE == 21 ? 110 : 82);
            const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
            const uint8_t *const rows[2] = {uniform_ptr(gate + off), uniform_ptr(up + off)};  // one row pair per wave
            // (PART) the chunk sums of the pair: gate row r of rung j, the up row F rows further on
            const size_t pg = static_cast<size_t>(nb) * 8;
            int32_t *pp = PART ? a.gup_part + (static_cast<size_t>(j) * 2 * a.F + min(r, a.F - 1)) * pg : nullptr;
            if (COAL && NB == 10)
                iq_rows10_coal<(kIq ? TYPE : 21), 2, PART>(rows, tables, xq, reinterpret_cast<const float *>(xscale), lane, gu,
                                                           lds_ab + ((4 * a.H + 16 + 15) & ~15) + wave * 2 * kIqStage10Bytes, pp, a.F * pg);
            else if (COAL)
                iq_rows8_coal<(kIq ? TYPE : 21), 2, PART>(rows, tables, xq, reinterpret_cast<const float *>(xscale), lane, gu,
                                                          lds_ab + ((4 * a.H + 16 + 15) & ~15) + wave * 2 * kIqStageBytes, pp, a.F * pg);
            else
                iq_rows_q8k<(kIq ? TYPE : 21), 2, PART>(rows, nb, tables, xq, reinterpret_cast<const float *>(xscale), lane, gu, pp,
                                                         a.F * pg);
        } else {
            Q8RowTile *tiles = reinterpret_cast<Q8RowTile *>(s_union);
            const int nb = a.H >> 5;
            const size_t rb = static_cast<size_t>(nb) * 34;
            const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
            const uint8_t *const rows[2] = {gate + off, up + off};
            q8_row_wave<2>(rows, nb, xq, reinterpret_cast<const uint16_t *>(xscale), tiles[wave], lane, gu);
        }
        if (lane == 0 && r < a.F) act[r] = silu_ggml(gu[0]) * gu[1];
        mark<TRACE>(a, 1, 3);
        if (LOOP) {
            item += n_routed_wgs;
            __syncthreads();  // s_expert is free for the next item
        }
    } while (LOOP && item < a.n_routed_items);
}

// ---- dispatch B -----------------------------------------------------------------------------------------
// TYPE: gate/up tensor type (21 IQ3_S, 22 IQ2_S, 8 Q8_0, 20 IQ4_NL).
// IQ types and Q8_0: 512-thread workgroups, one (gate,up) row pair per wave, grid = k * ceil(F / 8).
// IQ4_NL: 256-thread workgroups, four row pairs per wave, grid = k * ceil(F / 16).
// Every wave first requests its weight bytes; the workgroup then stages the codebooks and quantises x
// while they are in flight.  dynamic LDS: quantised x (H bytes + scales).
template <int TYPE, bool PART = false>
__global__ __launch_bounds__(TYPE == 20 ? 256 : 512) void k_layer_b(LayerArgs a) {
    constexpr bool kIq = (TYPE == 21 || TYPE == 22);
    constexpr int kThreads = (TYPE == 20) ? 256 : 512;
    constexpr int kRowsPerWg = (TYPE == 20) ? 16 : 8;
    extern __shared__ __align__(16) uint8_t lds_b[];
    __shared__ IqTables tables;
    __shared__ Q8TileN<4> tiles4[TYPE == 20 ? 4 : 1];
    __shared__ Q8RowTile tiles1[TYPE == 8 ? 8 : 1];
    int8_t *xq = reinterpret_cast<int8_t *>(lds_b);
    uint8_t *xscale = lds_b + a.H;  // f32 [H/256] or f16 [H/32]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (a.dry) return;
    mark(a, 1, 0);

    const int groups = (a.F + kRowsPerWg - 1) / kRowsPerWg;
    const int j = blockIdx.x / groups;
    const int rg = blockIdx.x - j * groups;
    const int e = a.ids[j];
    const uint8_t *gate = mat_ptr_expert<0>(a.gate_up, e);
    const uint8_t *up = mat_ptr_expert<1>(a.gate_up, e);
    float *act = a.act + static_cast<size_t>(j) * a.F;
    if (kIq) {
        const int nb = a.H >> 8;
        const size_t rb = static_cast<size_t>(nb) * (TYPE == 21 ? 110 : 82);
        const int r = rg * 8 + wave;
        const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
        const uint8_t *const rows[2] = {gate + off, up + off};
        float gu[2];
        const size_t pg = static_cast<size_t>(nb) * 8;
        int32_t *pp = PART ? a.gup_part + (static_cast<size_t>(j) * 2 * a.F + min(r, a.F - 1)) * pg : nullptr;
        iq_rows_q8k<(kIq ? TYPE : 21), 2, PART>(rows, nb, tables, xq, reinterpret_cast<const float *>(xscale), lane, gu,
                                                 pp, a.F * pg, [&]() {
            stage_tables<TYPE == 21, TYPE == 22>(tables, threadIdx.x, kThreads);
            for (int b = wave; b < (a.H >> 8); b += kThreads / 64)
                wave_quantize_q8_k_block(a.x + b * 256, xq + b * 256, reinterpret_cast<float *>(xscale) + b, lane);
            mark(a, 1, 1);
            __syncthreads();
            mark(a, 1, 2);
        });
        if (lane == 0 && r < a.F) act[r] = silu_ggml(gu[0]) * gu[1];
        mark(a, 1, 3);
    } else if (TYPE == 8) {
        const int nb = a.H >> 5;
        const size_t rb = static_cast<size_t>(nb) * 34;
        const int r = rg * 8 + wave;
        const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
        const uint8_t *const rows[2] = {gate + off, up + off};
        float gu[2];
        q8_row_wave<2>(rows, nb, xq, reinterpret_cast<const uint16_t *>(xscale), tiles1[TYPE == 8 ? wave : 0], lane, gu,
                       [&]() {
                           lds_quantize_q8_0(a.x, a.H, xq, reinterpret_cast<uint16_t *>(xscale), threadIdx.x, kThreads);
                           __syncthreads();
                       });
        if (lane == 0 && r < a.F) act[r] = silu_ggml(gu[0]) * gu[1];
    } else {
        const int nb = a.H >> 5;
        const size_t rb = static_cast<size_t>(nb) * 18;
        const int r0 = rg * 16 + wave * 4;
        const int nrows = max(0, min(4, a.F - r0));
        const size_t off = static_cast<size_t>(min(r0, a.F - 1)) * rb;
        const uint8_t *const rows[2] = {gate + off, up + off};
        float gu[2];
        q8_rows4_multi<1, 2, 4, false>(rows, nrows, nb, xq, reinterpret_cast<const uint16_t *>(xscale),
                                       tiles4[TYPE == 20 ? wave : 0], lane, gu, nullptr, 0, [&]() {
                                           lds_quantize_q8_0(a.x, a.H, xq, reinterpret_cast<uint16_t *>(xscale),
                                                             threadIdx.x, kThreads);
                                           __syncthreads();
                                       });
        const int r4 = lane >> 4;
        if ((lane & 15) == 0 && r4 < nrows) act[r0 + r4] = silu_ggml(gu[0]) * gu[1];
    }
    __syncthreads();
}

// ---- dispatch C -----------------------------------------------------------------------------------------
// KIND: down tensor kind (0 Q8_0, 1 IQ4_NL).  One workgroup per four output rows; wave m takes
// matrix m (the k routed down tensors, then the shared one), so every weight byte of the four rows
// is requested at once.  Each wave re-quantises the activation of its own matrix while its weights
// are in flight.  The first four lanes of wave 0 then fold the k+1 results in the reference order.
// grid = ceil(H / 4), block = 64 * min(k + 1, 16).
// dynamic LDS per wave: F bytes + F/32 halves (+ pad), then [k+1][4] floats.
// COAL: the rows are 16 blocks long, H is a multiple of 4 and every down tensor starts on a 16-byte boundary: the
// four rows of a wave are fetched as aligned 16-byte words (q8_rows4_coal).
// NB (COAL only): blocks per row, 16 or 20.  TWO (COAL only): the workgroup has half as many waves as matrices; a wave
// requests the rows and the activations of its two matrices together and parks all of it in LDS before the dot
// products, which keeps it within 80 registers: the waves of a workgroup go to the four SIMDs in turn, so three
// workgroups of six waves need six wave slots on two of them.  dynamic LDS per wave: two quantised activations and a
// staging area of 4 * NB * 34 bytes.
template <int KIND, bool COAL, int NB = 16, bool TWO = false, bool PART = false, bool TRACE = false>
__global__ __launch_bounds__(TWO ? 576 : 1024) __attribute__((amdgpu_waves_per_eu(TWO ? 6 : 4)))
void k_layer_c(LayerArgs a) {
    extern __shared__ __align__(16) uint8_t lds_c[];
    using Tile = typename std::conditional<COAL, Q8TileNB<NB>, Q8Tile>::type;
    __shared__ Tile tiles[TWO ? 9 : 16];
    const bool shared = a.sh_inp != nullptr;
    const int n_act = a.k + (shared ? 1 : 0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const size_t per_wave = (static_cast<size_t>(a.F) + a.F / 16 + 15) & ~static_cast<size_t>(15);
    int8_t *aq = reinterpret_cast<int8_t *>(lds_c + wave * per_wave);
    uint16_t *ad = reinterpret_cast<uint16_t *>(lds_c + wave * per_wave + a.F);
    float *ybuf = reinterpret_cast<float *>(lds_c + nwaves * per_wave);  // [n_act][4] (behind larger per-wave areas if TWO)
    const int r0 = blockIdx.x * 4;
    const int nrows = min(4, a.H - r0);
    const int nb = a.F >> 5;
    const int r4 = lane >> 4;
    if (a.dry) return;
    // every routed workgroup of this layer pass finished with the previous dispatch: make the ids published
    // for them invalid again (this dispatch reads the plain copy)
    if (a.clear_tagged && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kTagCopies * 16; i += blockDim.x)
            __hip_atomic_store(a.ids_tagged + i, kTagInvalid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    mark<TRACE>(a, 2, 0);
    // combine operands, requested early: lane m keeps router weight m, lane 16 the shared gate
    float wreg = 0.0f, res_pre = 0.0f, inject = 0.0f;
    unsigned bad = 0u;  // a bounded wait of this layer pass ran out: the results below are replaced by NaN
    if (wave == 0) {
        bad = __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane < a.k) wreg = a.weights[lane];
        if (lane == 16 && shared) wreg = a.shared_gate[0];
        // the residual values this workgroup updates at its end (nothing else writes them meanwhile): lane 4c + r
        // holds stream c of row r0 + r
        if (a.residual) {
            const int c = a.hc > 0 ? min(lane >> 2, a.hc - 1) : 0;
            res_pre = a.residual[static_cast<size_t>(c) * a.H + r0 + min(lane & 3, nrows - 1)];
            if (a.hc > 0) inject = a.hc_inject[c];
        }
    }
    // COAL: the activation of one matrix in registers, values 8 lane .. 8 lane + 8 and, with 20 blocks, 512 .. 639 in
    // lanes 0..15 (the others repeat them); its Q8_0 form into LDS
    constexpr int kActRegs = (COAL && NB == 20) ? 4 : 2;
    auto request_act = [&](int m, float4 (&v)[kActRegs]) {
        const float *act = a.act + static_cast<size_t>(m) * (NB * 32);
        v[0] = *reinterpret_cast<const float4 *>(act + lane * 8);
        v[1] = *reinterpret_cast<const float4 *>(act + lane * 8 + 4);
        if constexpr (kActRegs == 4) {
            v[2] = *reinterpret_cast<const float4 *>(act + 512 + (lane & 15) * 8);
            v[3] = *reinterpret_cast<const float4 *>(act + 512 + (lane & 15) * 8 + 4);
        }
    };
    auto quantise_act = [&](const float4 (&v)[kActRegs], int8_t *qs, uint16_t *d) {
        lds_quantize_q8_0_step(v[0], v[1], true, lane * 8, qs, d, lane);
        if constexpr (kActRegs == 4) lds_quantize_q8_0_step(v[2], v[3], lane < 16, 512 + (lane & 15) * 8, qs, d, lane);
    };
    if constexpr (COAL && TWO) {
        // Everything is requested at once; both activations are quantised and both row groups parked in LDS as they
        // arrive (loads return in order), so that no fetched word stays in a register while the dot products run.
        using RawQ8 = Q8CoalRaw<0, NB>;
        using RawW = Q8CoalRaw<KIND, NB>;
        constexpr size_t kStage = 4 * NB * 34;  // the larger of the two kinds
        const int uw = __builtin_amdgcn_readfirstlane(wave);
        uint8_t *const wbase = lds_c + wave * (2 * per_wave + kStage);
        int8_t *const aq2[2] = {reinterpret_cast<int8_t *>(wbase), reinterpret_cast<int8_t *>(wbase + per_wave)};
        uint16_t *const ad2[2] = {reinterpret_cast<uint16_t *>(wbase + a.F), reinterpret_cast<uint16_t *>(wbase + per_wave + a.F)};
        uint8_t *const stage2[2] = {reinterpret_cast<uint8_t *>(&tiles[wave]), wbase + 2 * per_wave};
        ybuf = reinterpret_cast<float *>(lds_c + nwaves * (2 * per_wave + kStage));
        const bool second = uw + nwaves < n_act;  // wave-uniform; a wave without a second matrix repeats its first (not used)
        RawQ8 raw[2];  // (the request of either kind: as many loads as Q8_0 rows need)
        float4 v[2][kActRegs];
        int mm[2], words[2];
        bool sh[2];
        // the activations first: their addresses need no expert id, and loads return in order - the quantisation
        // below then runs while the weights are still on their way
        int e[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            mm[q] = (q == 0 || second) ? uw + q * nwaves : uw;
            sh[q] = mm[q] == a.k;
            e[q] = sld_i32(a.ids + min(mm[q], a.k - 1));  // both ids asked for together (not used for the shared expert)
        }
#pragma unroll
        for (int q = 0; q < 2; ++q) request_act(mm[q], v[q]);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint8_t *w = sh[q] ? a.sh_down : mat_ptr_expert_uniform<0>(a.down, e[q]);
            const bool q8 = KIND == 0 || sh[q];  // wave-uniform
            words[q] = q8 ? RawQ8::kWords : RawW::kWords;
            raw[q] = q8_rows4_coal_request_any<NB>(w + static_cast<size_t>(r0) * NB * (q8 ? 34 : RawW::kBlk), words[q], lane);
        }
        mark<TRACE>(a, 2, 1);
        wave_lds_fence();
#pragma unroll
        for (int q = 0; q < 2; ++q) quantise_act(v[q], aq2[q], ad2[q]);
        mark<TRACE>(a, 2, 6);
#pragma unroll
        for (int q = 0; q < 2; ++q) q8_rows4_coal_stage_any<NB>(raw[q], stage2[q], words[q], lane);
        wave_lds_fence();
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if (q == 1 && !second) break;
            float y;
            if (PART && !sh[q]) {  // (the shared expert's sums are not part of the dump)
                int32_t *pp = a.down_part + (static_cast<size_t>(mm[q]) * a.H + r0) * (NB * 8);
                y = q8_rows4_coal_dots<KIND, NB, PART>(stage2[q], aq2[q], ad2[q], tiles[wave], lane, pp);
            } else {
                y = (KIND == 0 || sh[q]) ? q8_rows4_coal_dots<0, NB>(stage2[q], aq2[q], ad2[q], tiles[wave], lane)
                                         : q8_rows4_coal_dots<KIND, NB>(stage2[q], aq2[q], ad2[q], tiles[wave], lane);
            }
            if ((lane & 15) == 0) ybuf[mm[q] * 4 + r4] = y;
            mark<TRACE>(a, 2, q == 0 ? 2 : 5);
        }
    } else
    for (int m = wave; m < n_act; m += nwaves) {
        const bool is_shared = m == a.k;
        if constexpr (COAL) {
            // the activation first: its address needs no expert id, and loads return in order - it is quantised while
            // the weights are still on their way
            float4 v[kActRegs];
            request_act(m, v);
            const uint8_t *w = is_shared ? a.sh_down : mat_ptr_expert_uniform<0>(a.down, sld_i32(a.ids + m));
            float y;
            if (KIND == 0 || is_shared) {
                const auto raw = q8_rows4_coal_request<0, NB>(w + static_cast<size_t>(r0) * NB * 34, lane);
                wave_lds_fence();
                quantise_act(v, aq, ad);
                mark<TRACE>(a, 2, 1);
                if (PART && !is_shared)
                    y = q8_rows4_coal_finish<0, NB, PART>(raw, aq, ad, tiles[wave], lane, a.down_part + (static_cast<size_t>(m) * a.H + r0) * (NB * 8));
                else
                    y = q8_rows4_coal_finish<0, NB>(raw, aq, ad, tiles[wave], lane);
            } else {
                const auto raw = q8_rows4_coal_request<1, NB>(w + static_cast<size_t>(r0) * NB * 18, lane);
                wave_lds_fence();
                quantise_act(v, aq, ad);
                mark<TRACE>(a, 2, 1);
                y = q8_rows4_coal_finish<1, NB, PART>(raw, aq, ad, tiles[wave], lane,
                                                      PART ? a.down_part + (static_cast<size_t>(m) * a.H + r0) * (NB * 8) : nullptr);
            }
            if ((lane & 15) == 0) ybuf[m * 4 + r4] = y;
        } else {
            // m is the same for the whole wave: the id comes through the scalar path
            const uint8_t *w = is_shared ? a.sh_down : mat_ptr_expert_uniform<0>(a.down, sld_i32(a.ids + m));
            const size_t rb = static_cast<size_t>(nb) * ((KIND == 0 || is_shared) ? 34 : 18);
            const uint8_t *const rows[1] = {w + r0 * rb};
            float y[1];
            auto quantise = [&]() {
                wave_lds_fence();
                lds_quantize_q8_0(a.act + static_cast<size_t>(m) * a.F, a.F, aq, ad, lane, 64);
                wave_lds_fence();
                mark<TRACE>(a, 2, 1);
            };
            int32_t *pp = (PART && !is_shared) ? a.down_part + (static_cast<size_t>(m) * a.H + r0) * (static_cast<size_t>(nb) * 8) : nullptr;
            if (PART && !is_shared && KIND == 0)
                q8_rows4_multi<0, 1, 1, PART>(rows, nrows, nb, aq, ad, tiles[wave], lane, y, pp, 0, quantise);
            else if (KIND == 0 || is_shared)
                q8_rows4_multi<0, 1, 1, false>(rows, nrows, nb, aq, ad, tiles[wave], lane, y, nullptr, 0, quantise);
            else
                q8_rows4_multi<1, 1, 1, PART>(rows, nrows, nb, aq, ad, tiles[wave], lane, y, pp, 0, quantise);
            if ((lane & 15) == 0) ybuf[m * 4 + r4] = y[0];
        }
        mark<TRACE>(a, 2, 2);
    }
    __syncthreads();
    mark<TRACE>(a, 2, 3);
    if (wave == 0) {
        // every lane folds row r0 + (lane & 3); lanes 0..3 store it
        const int row = r0 + lane;
        const bool on = lane < nrows;
        float acc = 0.0f;
        for (int m = 0; m < a.k; ++m) {
            const float wm = lane_get(wreg, m);
            const float y = ybuf[m * 4 + (lane & 3)];
            const float prod = y * wm;
            acc = acc + prod;
            if (a.expert_out && on) a.expert_out[static_cast<size_t>(m) * a.H + row] = y;
        }
        const float gate = lane_get(wreg, 16);
        float o = acc;
        if (shared) {
            const float y = ybuf[a.k * 4 + (lane & 3)];
            const float prod = y * gate;
            o = acc + prod;
            if (on) a.down_f32[row] = y;
        }
        // an expert without a slot was reported by the waves above (or by the dispatch before)
        if (a.down.slot_of_expert) bad |= __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (bad) acc = o = __builtin_nanf("");  // the caller sees the failure in its data, without a synchronisation
        if (on) {
            a.accum[row] = acc;
            a.out[row] = o;
        }
        if (a.residual) {
            if (a.hc > 0) {
                const int c = lane >> 2;
                if (c < a.hc && (lane & 3) < nrows) {
                    const float weighted = o * hc_weight(inject, a.hc);
                    const float v = res_pre + weighted;
                    a.residual[static_cast<size_t>(c) * a.H + r0 + (lane & 3)] = a.hc_round_half ? round_half(v) : v;
                }
            } else if (on) {
                const float scaled = o * a.residual_scale;
                a.residual[row] = res_pre + scaled;
            }
        }
    }
    mark<TRACE>(a, 2, 4);
}

}  // namespace wd
