// M tokens through one MoE layer with every selected expert's weights read once.
//
// The reference batches M tokens as M*k (token, expert) pairs and re-reads an expert's weights for
// every pair that names it (src/qwen38_moe.cuh:1316-1437, :2743-3237).  Here a pass is three dispatches:
//   A  router, selection and shared gate/up of every token side by side (grid.y = token);
//   B  routed gate/up + SwiGLU over the union of the selected experts: a weight row is decoded once and applied to
//      the activation of every token that selected the expert;
//   C  down projections over the union (a member's rows are loaded once and applied to the activations of its
//      tokens) and the ordered combine per token.
// B and C each work the union out for themselves from the T*k ids (one wave per workgroup, in LDS); nothing about
// it goes through global memory.  Per token, the arithmetic and its order are those of the one-token kernels, so the
// results are bit-identical to M separate passes.
#pragma once

#include "wd_fused.cuh"

namespace wd {

constexpr int kMaxTokens = 8;

constexpr int kPairEntries = 128;  // entries of a pointer table (wd_moe_layer_tokens_pairs_f32)

// Tensor T of "expert" e when the pass was given a table of pointers instead of tensors that hold every expert: e is
// then an index into the table ([entry][tensors per entry]).  The host fills every one of the kPairEntries entries
// (those past the caller's with entry 0), and a number outside the table reads entry 0: a wrong id in the scratch gives
// a wrong result, never a load through a pointer nobody set.
template <int T>
WD_DEV const uint8_t *mat_ptr_entry(const MatSrc &s, int e) {
    if (s.table) return s.table[(static_cast<unsigned>(e) < static_cast<unsigned>(kPairEntries) ? e : 0) * s.per_expert + T];
    return mat_ptr_expert<T>(s, e);
}

struct TokenSlots {
    const float *x;
    float *logits;
    int32_t *ids;
    float *weights;
    float *act;          // [k+1][F]
    float *shared_gate;  // [1]
    unsigned *arrive;
    float *expert_out;   // null or [k][H]
    float *accum, *down_f32, *out;
};

struct TokenArgs {
    LayerArgs common;  // the layer; the per-token members are taken from tok[]
    int T;
    TokenSlots tok[kMaxTokens];
};

// ---- dispatch A for T tokens ----------------------------------------------------------------------------
// grid = T * (router_stride + shared_stride), 512 threads, the strides being the router and the shared workgroups of a
// token rounded up to a multiple of 8 (tokens_a_grid): first the router workgroups of every token, token by token, then
// the shared ones.  The router workgroups are on the pass's critical path and start first; and workgroup w of every
// token - the same weight rows - lands on the same XCD (workgroups go to the eight XCDs in turn), so its L2 serves the
// rows to the tokens after the first.  The padding workgroups return at once.  Per token this is the front of the
// one-token merged dispatch: router rows one per wave, the last router workgroup of the token selects its experts
// with the whole workgroup, the other workgroups run the shared expert's gate/up.
// dynamic LDS: 4 * H bytes (x as f32 for the router rows; the shared workgroups use H + H/16 of it).
struct TokensAGrid {
    int router_stride, shared_stride;
    __host__ __device__ int total(int tokens) const { return tokens * (router_stride + shared_stride); }
};
__host__ __device__ inline TokensAGrid tokens_a_grid(int n_router_wgs, int n_shared_wgs) {
    return TokensAGrid{(n_router_wgs + 7) & ~7, (n_shared_wgs + 7) & ~7};
}
__global__ __launch_bounds__(512, 4) void k_tokens_a(TokenArgs ta) {
    extern __shared__ __align__(16) uint8_t lds_ta[];
    __shared__ __align__(16) uint8_t s_work[sizeof(Q8RowTile) * 8];
    __shared__ int s_last;
    const LayerArgs &a = ta.common;
    const int n_shared_wgs = a.sh_inp ? (a.F + 7) / 8 : 0;
    const TokensAGrid gr = tokens_a_grid(a.n_router_wgs, n_shared_wgs);
    int token, wg;
    {
        const int b = blockIdx.x, router_part = ta.T * gr.router_stride;
        if (b < router_part) {
            token = b / gr.router_stride, wg = b - token * gr.router_stride;
            if (wg >= a.n_router_wgs) return;
        } else {
            token = (b - router_part) / gr.shared_stride;
            const int w = b - router_part - token * gr.shared_stride;
            if (w >= n_shared_wgs) return;
            wg = a.n_router_wgs + w;
        }
    }
    const TokenSlots &s = ta.tok[token];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (wg < a.n_router_wgs) {
        router_rows_wave<true, true>(a.router, s.x, reinterpret_cast<float *>(lds_ta), s.logits, a.preselected ? 0 : a.E, a.H,
                               a.sh_inp, s.shared_gate, wg);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0)
            s_last = (__hip_atomic_fetch_add(s.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      static_cast<unsigned>(a.n_router_wgs - 1));
        __syncthreads();
        if (!s_last) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (!a.preselected) {
            static_assert(sizeof(s_work) >= kTopkLdsBytes2 + 128, "selection scratch, ids and weights must fit the shared area");
            int32_t *lds_ids = reinterpret_cast<int32_t *>(s_work + kTopkLdsBytes2);  // behind the selection's own scratch
            float *lds_w = reinterpret_cast<float *>(s_work + kTopkLdsBytes2 + 64);
            topk_block(s.logits, a.E, a.k, a.w_scale, lds_ids, lds_w, nullptr, s_work, lane, wave);
            if (wave == 0) {
                wave_lds_fence();
                if (lane < a.k) {
                    s.ids[lane] = lds_ids[lane];
                    s.weights[lane] = lds_w[lane];
                }
            }
        }
        if (wave == 5 && lane == 0) {
            if (a.sh_inp) {
                const float g = __hip_atomic_load(s.shared_gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s.shared_gate[0] = sigmoid_ggml(g);
            }
            s.arrive[0] = 0u;
        }
        return;
    }
    int8_t *xq = reinterpret_cast<int8_t *>(lds_ta);
    uint16_t *xd = reinterpret_cast<uint16_t *>(lds_ta + a.H);
    Q8RowTile *tiles = reinterpret_cast<Q8RowTile *>(s_work);
    const int r = (wg - a.n_router_wgs) * 8 + wave;
    const int nb = a.H >> 5;
    const size_t rb = static_cast<size_t>(nb) * 34;
    const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
    const uint8_t *const rows[2] = {uniform_ptr(a.sh_gate + off), uniform_ptr(a.sh_up + off)};  // one row pair per wave
    float gu[2];
    q8_row_wave<2>(rows, nb, xq, xd, tiles[wave], lane, gu, [&]() {
        lds_quantize_q8_0(s.x, a.H, xq, xd, threadIdx.x, 512);
        __syncthreads();
    });
    if (lane == 0 && r < a.F) s.act[static_cast<size_t>(a.k) * a.F + r] = silu_ggml(gu[0]) * gu[1];
}

// The id of pair `pair` (= token * k + rank) for lane-parallel comparisons; pairs past the end get distinct
// negative values that match nothing.
WD_DEV int token_pair_id(const TokenArgs &ta, int pair) {
    const int k = ta.common.k, n = ta.T * k;
    const int pc = min(pair, n - 1);  // the load is unconditional (no branch, so that it can overlap with others)
    int t = 0;
    const int32_t *p = ta.tok[0].ids;
#pragma unroll
    for (int q = 1; q < kMaxTokens; ++q) {
        const bool past = pc >= q * k;
        t += past ? 1 : 0;
        p = past ? ta.tok[q].ids : p;
    }
    const int v = p[pc - t * k];
    return pair < n ? v : -1 - pair;
}

// The union of the T*k routed ids, in order of first appearance, with the rank at which every token selected
// each member (-1: not selected).  Lives in LDS; built by one full wave (T*k <= 128, expert ids < 1024).
struct TokenUnion {
    int count;
    int expert[128];
    int upos[128];                   // scratch of the build: union index of a first occurrence
    int8_t rank[128][kMaxTokens];
    int first_pair[1024];            // scratch of the build: lowest pair naming an expert
};

WD_DEV void token_union_build(const TokenArgs &ta, TokenUnion &un, int lane) {
    const int k = ta.common.k, n = ta.T * k;
    const int id_lo = token_pair_id(ta, lane), id_hi = token_pair_id(ta, lane + 64);
    const bool on_lo = lane < n, on_hi = lane + 64 < n;
    for (int i = lane; i < 128 * kMaxTokens / 4; i += 64) reinterpret_cast<uint32_t *>(&un.rank[0][0])[i] = 0xffffffffu;
    // lowest pair that names the same expert, through a table indexed by expert id
    if (on_lo) un.first_pair[id_lo] = 0x7fffffff;
    if (on_hi) un.first_pair[id_hi] = 0x7fffffff;
    wave_lds_fence();
    if (on_lo) atomicMin(&un.first_pair[id_lo], lane);
    if (on_hi) atomicMin(&un.first_pair[id_hi], lane + 64);
    wave_lds_fence();
    const int fq_lo = on_lo ? un.first_pair[id_lo] : -1, fq_hi = on_hi ? un.first_pair[id_hi] : -1;
    const bool first_lo = on_lo && fq_lo == lane, first_hi = on_hi && fq_hi == lane + 64;
    const unsigned long long m_lo = __builtin_amdgcn_ballot_w64(first_lo), m_hi = __builtin_amdgcn_ballot_w64(first_hi);
    const unsigned long long below = (1ull << lane) - 1ull;
    const int u_lo = __builtin_popcountll(m_lo & below);
    const int u_hi = __builtin_popcountll(m_lo) + __builtin_popcountll(m_hi & below);
    if (first_lo) {
        un.upos[lane] = u_lo;
        un.expert[u_lo] = id_lo;
    }
    if (first_hi) {
        un.upos[lane + 64] = u_hi;
        un.expert[u_hi] = id_hi;
    }
    if (lane == 0) un.count = __builtin_popcountll(m_lo) + __builtin_popcountll(m_hi);
    wave_lds_fence();
    // (token, rank) of a pair without a division: tokens are k pairs apart
    int t_lo = 0, t_hi = 0;
#pragma unroll
    for (int q = 1; q < kMaxTokens; ++q) {
        t_lo += (lane >= q * k) ? 1 : 0;
        t_hi += (lane + 64 >= q * k) ? 1 : 0;
    }
    if (on_lo) un.rank[un.upos[fq_lo]][t_lo] = static_cast<int8_t>(lane - t_lo * k);
    if (on_hi) un.rank[un.upos[fq_hi]][t_hi] = static_cast<int8_t>(lane + 64 - t_hi * k);
    wave_lds_fence();
}

// ---- dispatch B for T tokens ----------------------------------------------------------------------------
// Persistent form: grid = min(T * k * ceil(F / 8), a few workgroups per compute unit), 512 threads.  Every
// workgroup builds the union (wave 0), stages the codebooks and quantises the T inputs once, then walks the items
// (union member, group of 8 rows) blockIdx.x, blockIdx.x + gridDim.x, ...; a wave takes one (gate, up) row pair of
// the item, decodes it once and applies it to every token that selected the expert.
// MAXT: token capacity of the instantiation (4 or kMaxTokens).
// dynamic LDS: T * (H bytes + H/256 floats): the Q8_K copies of the T inputs.
// NB: 0, or the super-blocks per row (8 or 10) when the rows can be fetched as aligned words (IqRowFetch): the row pair of
// the wave's next item is then requested before the current one is worked on.  dynamic LDS then has
// 8 * 2 * (kIqStageBytes or kIqStage10Bytes) more bytes behind the activations (16-byte aligned).
template <int TYPE, int MAXT, int NB = 0>
__global__ __launch_bounds__(512, 4) void k_tokens_b(TokenArgs ta) {
    extern __shared__ __align__(16) uint8_t lds_tb[];
    __shared__ IqTables tables;
    __shared__ TokenUnion un;
    const LayerArgs &a = ta.common;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int groups = (a.F + 7) / 8;
    int8_t *xq = reinterpret_cast<int8_t *>(lds_tb);
    float *xd = reinterpret_cast<float *>(lds_tb + static_cast<size_t>(ta.T) * a.H);
    constexpr int kBlk = (TYPE == 21) ? 110 : 82;
    const int nb = a.H >> 8;
    const size_t rb = static_cast<size_t>(nb) * kBlk;
    mark(a, 1, 0);
    // the T inputs as Q8_K: a wave's blocks (wave, wave + 8, ...) are requested four at a time, the first four before
    // anything else so that the union build and the codebook staging run under their latency
    constexpr int kMaxBlocks = 4;
    float4 xv[kMaxBlocks];
    auto load_blocks = [&](int b0) {
#pragma unroll
        for (int i = 0; i < kMaxBlocks; ++i) {
            const int b = min(b0 + 8 * i, ta.T * nb - 1);
            const int t = __builtin_amdgcn_readfirstlane(b / nb), bb = b - t * nb;  // uniform index into the argument block
            xv[i] = reinterpret_cast<const float4 *>(ta.tok[t].x + bb * 256)[lane];
        }
    };
    auto quantise_blocks = [&](int b0) {
#pragma unroll
        for (int i = 0; i < kMaxBlocks; ++i) {
            const int b = b0 + 8 * i;
            if (b < ta.T * nb) {
                const int t = b / nb, bb = b - t * nb;
                wave_quantize_q8_k_regs(xv[i], xq + static_cast<size_t>(t) * a.H + bb * 256, xd + t * nb + bb, lane);
            }
        }
    };
    load_blocks(wave);
    if (wave == 0) token_union_build(ta, un, lane);
    mark(a, 1, 1);
    stage_tables<TYPE == 21, TYPE == 22>(tables, threadIdx.x, 512);
    quantise_blocks(wave);
    for (int b0 = wave + 8 * kMaxBlocks; b0 < ta.T * nb; b0 += 8 * kMaxBlocks) {
        load_blocks(b0);
        quantise_blocks(b0);
    }
    __syncthreads();
    mark(a, 1, 2);
    const int n_items = un.count * groups;
    // rows of eight super-blocks are one pass: the lane layout of iq_rows8_coal_dots then (a chain's lanes two apart inside
    // a row, no carry between passes, no lane excluded from a chain step)
    // (NB == 10: the same layout for super-blocks 0..7, and super-blocks 8 and 9 of both rows in one shared pass, as in
    // iq_rows10_coal)
    constexpr bool kPairs = NB == 8 || NB == 10;
    const int ib = kPairs ? ((lane >> 4) << 1) | (lane & 1) : lane >> 3, sbl = kPairs ? (lane >> 1) & 7 : lane & 7;
    const bool first = sbl == 0;
    constexpr int kStage = (NB == 10) ? kIqStage10Bytes : kIqStageBytes;
    uint8_t *stage = lds_tb + ((static_cast<size_t>(ta.T) * (a.H + sizeof(float) * nb) + 15) & ~static_cast<size_t>(15)) +
                     static_cast<size_t>(wave) * 2 * kStage;
    IqRowFetch<TYPE, NB == 0 ? 8 : NB> fetch[2];
    auto row_pair = [&](int item, const uint8_t *(&rows)[2]) {
        const int u = item / groups, rg = item - u * groups;
        const int e = un.expert[u];
        const size_t off = static_cast<size_t>(min(rg * 8 + wave, a.F - 1)) * rb;
        rows[0] = uniform_ptr(mat_ptr_entry<0>(a.gate_up, e) + off), rows[1] = uniform_ptr(mat_ptr_entry<1>(a.gate_up, e) + off);
    };
    if (NB != 0 && static_cast<int>(blockIdx.x) < n_items) {
        const uint8_t *rows[2];
        row_pair(blockIdx.x, rows);
        fetch[0].request(rows[0], lane), fetch[1].request(rows[1], lane);
    }
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int u = item / groups, rg = item - u * groups;
        int rank[MAXT];
#pragma unroll
        for (int t = 0; t < MAXT; ++t) rank[t] = __builtin_amdgcn_readfirstlane(static_cast<int>(un.rank[u][t]));
        const int r = rg * 8 + wave;
        const uint8_t *rows[2];  // one row pair per wave
        row_pair(item, rows);
        uint32_t lead[2] = {0, 0};
        if (NB != 0) {
            wave_lds_fence();  // the previous item's rows have been read
            fetch[0].store(stage, lane), fetch[1].store(stage + kStage, lane);
            lead[0] = fetch[0].lead, lead[1] = fetch[1].lead;
            wave_lds_fence();
            if (item + static_cast<int>(gridDim.x) < n_items) {  // the next item's rows, into the registers just written out
                const uint8_t *next[2];
                row_pair(item + gridDim.x, next);
                fetch[0].request(next[0], lane), fetch[1].request(next[1], lane);
            }
        }
        float acc[MAXT][2];
#pragma unroll
        for (int t = 0; t < MAXT; ++t) acc[t][0] = acc[t][1] = 0.0f;
        for (int base = 0; base < (NB == 10 ? 8 : nb); base += 8) {
            const int sb = base + sbl;
            const bool on = sb < nb;
            uint32_t w[2][8];
            int ls[2][2];
            float dw[2] = {0.0f, 0.0f};
            if (on) {
                IqFields f[2];
                if (NB != 0) {
                    f[0] = iq_fields_lds<TYPE>(stage + lead[0] + sb * kBlk, ib, sb);
                    f[1] = iq_fields_lds<TYPE>(stage + kStage + lead[1] + sb * kBlk, ib, sb);
                } else {
                    f[0] = iq_load<TYPE>(rows[0] + static_cast<size_t>(sb) * kBlk, ib);
                    f[1] = iq_load<TYPE>(rows[1] + static_cast<size_t>(sb) * kBlk, ib);
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    iq_decode<TYPE>(f[i], ib, tables, w[i], ls[i]);
                    dw[i] = h2f(f[i].d);
                }
            }
#pragma unroll
            for (int t = 0; t < MAXT; ++t) {
                if (rank[t] < 0) continue;  // uniform
                uint32_t av[8];
                float dx = 0.0f;
                if (on) {
                    const int8_t *aq = xq + static_cast<size_t>(t) * a.H + sb * 256 + ib * 32;
                    const uint4 a0 = *reinterpret_cast<const uint4 *>(aq);
                    const uint4 a1 = *reinterpret_cast<const uint4 *>(aq + 16);
                    av[0] = a0.x, av[1] = a0.y, av[2] = a0.z, av[3] = a0.w, av[4] = a1.x, av[5] = a1.y, av[6] = a1.z, av[7] = a1.w;
                    dx = xd[t * nb + sb];
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    int p[8];
                    float ds = 0.0f;
                    if (on) {
                        iq_dot_decoded(w[i], ls[i], av, p);
                        ds = dw[i] * dx;
                    } else {
#pragma unroll
                        for (int c = 0; c < 8; ++c) p[c] = 0;
                    }
                    if (kPairs) {
                        const float pf = static_cast<float>(reduce_scatter_ib_pairs(p, lane));
                        float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
                        for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
                        acc[t][i] = v;
                        continue;
                    }
                    const float pf = static_cast<float>(reduce_scatter_ib(p, lane));
                    const float carry = dpp_f<kDppShl7>(0.0f, acc[t][i]);
                    float v = __builtin_fmaf(ds, pf, base == 0 ? 0.0f : carry);
#pragma unroll
                    for (int s = 1; s < 8; ++s) {
                        const float up = dpp_f<kDppShr1>(0.0f, v);
                        const float nxt = __builtin_fmaf(ds, pf, up);
                        v = first ? v : nxt;
                    }
                    acc[t][i] = v;
                }
            }
        }
        if (NB == 10) {
            // super-blocks 8 and 9: position 0/1 of the pass = row 0, position 2/3 = row 1 (positions 4..7 idle)
            const int ri = min(sbl >> 1, 1), sb = 8 + (sbl & 1);
            const bool on = sbl < 4;
            const IqFields f = iq_fields_lds<TYPE>(stage + ri * kStage + (ri ? lead[1] : lead[0]) + sb * kBlk, ib, sb);
            uint32_t w[8];
            int ls[2];
            iq_decode<TYPE>(f, ib, tables, w, ls);
            const float dw = h2f(f.d);
#pragma unroll
            for (int t = 0; t < MAXT; ++t) {
                if (rank[t] < 0) continue;  // uniform
                const int8_t *aq = xq + static_cast<size_t>(t) * a.H + sb * 256 + ib * 32;
                const uint4 a0 = *reinterpret_cast<const uint4 *>(aq);
                const uint4 a1 = *reinterpret_cast<const uint4 *>(aq + 16);
                const uint32_t av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                int p[8];
                iq_dot_decoded(w, ls, av, p);
                const float ds = on ? dw * xd[t * nb + sb] : 0.0f;
                const int P = reduce_scatter_ib_pairs(p, lane);
                const float pf = on ? static_cast<float>(P) : 0.0f;
                float carry = dpp_f<0x10E, 0xf, 0x1>(0.0f, acc[t][0]);  // row 0's chain: position 7 -> position 0
                carry = dpp_f<0x10A, 0xf, 0x2>(carry, acc[t][1]);       // row 1's chain: position 7 -> position 2
                const float v8 = __builtin_fmaf(ds, pf, carry);
                const float v9 = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v8));
                acc[t][0] = dpp_f<0x11C>(0.0f, v9);  // back to position 7 for the closing tree
                acc[t][1] = dpp_f<0x118>(0.0f, v9);
            }
        }
#pragma unroll
        for (int t = 0; t < MAXT; ++t) {
            if (rank[t] < 0) continue;
            float g = kPairs ? close_chains_pairs(acc[t][0]) : close_lanes8_strided(acc[t][0]);
            float up = kPairs ? close_chains_pairs(acc[t][1]) : close_lanes8_strided(acc[t][1]);
            if (TYPE == 22) {
                g = 0.125f * g;
                up = 0.125f * up;
            }
            if (lane == 0 && r < a.F) ta.tok[t].act[static_cast<size_t>(rank[t]) * a.F + r] = silu_ggml(g) * up;
        }
        mark(a, 1, item == static_cast<int>(blockIdx.x) ? 3 : 4);
    }
    mark(a, 1, 5);
}

// ---- dispatch C for T tokens ----------------------------------------------------------------------------
// grid = ceil(H / 8), 1024 threads: a workgroup owns eight output rows (two groups of four).  Work items are
// (token, matrix) with matrix = the token's k routed down tensors, then the shared one; wave w takes items w,
// w + 16, w + 32 of a round of 48: it requests the activations and (as soon as the ids are in) the eight rows of all
// its items together (F <= 512: one block per lane and row group), then quantises each item's activation once and
// runs the one-token row code on both row groups.  Items that name the same expert read the same rows within one
// workgroup, so memory sees them once.  Waves 0..T-1 finally fold token t's results in its own top-k order.
// dynamic LDS: per wave F bytes + F/32 halves (+pad), then [T][k+1][8] floats.
__global__ __launch_bounds__(1024) void k_tokens_c(TokenArgs ta) {
    extern __shared__ __align__(16) uint8_t lds_tc[];
    __shared__ Q8Tile tiles[16];
    const LayerArgs &a = ta.common;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int kWaves = 16, kItems = 3;
    const size_t per_wave = (static_cast<size_t>(a.F) + a.F / 16 + 15) & ~static_cast<size_t>(15);
    int8_t *aq = reinterpret_cast<int8_t *>(lds_tc + wave * per_wave);
    uint16_t *ad = reinterpret_cast<uint16_t *>(lds_tc + wave * per_wave + a.F);
    float *ybuf = reinterpret_cast<float *>(lds_tc + kWaves * per_wave);  // [T][k+1][8]
    const bool shared = a.sh_down != nullptr;
    const int per_token = a.k + (shared ? 1 : 0);
    const int n_items = ta.T * per_token;
    const int r0 = blockIdx.x * 8;
    const int nb = a.F >> 5;  // <= 16
    const int r4 = lane >> 4, b = lane & 15, c = lane & 7;
    const bool act_on = lane * 8 < a.F;
    mark(a, 2, 0);
    // every routed id of the pass, one vector load per wave; an item's id is then a lane read
    const int id_lo = token_pair_id(ta, lane), id_hi = token_pair_id(ta, lane + 64);
    // combine operands of token `wave`, requested early: lane j keeps router weight j, lane 16 the shared gate
    const int tw = __builtin_amdgcn_readfirstlane(wave);  // uniform index into the argument block
    float wreg;
    {
        const TokenSlots &s = ta.tok[min(tw, ta.T - 1)];
        const float *src = (lane == 16 && shared) ? s.shared_gate : s.weights + min(lane, a.k - 1);
        wreg = *src;
    }
    Q8Tile &tile = tiles[wave];
    for (int item0 = 0; item0 < n_items; item0 += kWaves * kItems) {
        int it_t[kItems], it_j[kItems];
        bool it_on[kItems];
        float4 v0[kItems], v1[kItems];
        Q8Block wb[kItems][2];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {  // unconditional loads: an item past the end repeats the last one
            const int item = item0 + tw + kWaves * i;
            it_on[i] = item < n_items;
            const int ic = min(item, n_items - 1);
            it_t[i] = ic / per_token, it_j[i] = ic - it_t[i] * per_token;
            const float *act = ta.tok[it_t[i]].act + static_cast<size_t>(it_j[i]) * a.F + min(lane * 8, a.F - 8);
            v0[i] = *reinterpret_cast<const float4 *>(act);
            v1[i] = *reinterpret_cast<const float4 *>(act + 4);
        }
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const bool is_shared = it_j[i] == a.k;
            const int pair = it_t[i] * a.k + (is_shared ? 0 : it_j[i]);
            const int e = pair < 64 ? __builtin_amdgcn_readlane(id_lo, pair) : __builtin_amdgcn_readlane(id_hi, pair - 64);
            const uint8_t *w = is_shared ? a.sh_down : mat_ptr_entry<0>(a.down, e);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const int row = min(r0 + 4 * g + r4, a.H - 1);
                wb[i][g] = q8_load<0>(w + (static_cast<size_t>(row) * nb + min(b, nb - 1)) * 34);
            }
        }
        mark(a, 2, 1);
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if (!it_on[i]) continue;  // uniform
            wave_lds_fence();
            lds_quantize_q8_0_step(v0[i], v1[i], act_on, lane * 8, aq, ad, lane);
            wave_lds_fence();
            uint32_t av[8];
            float dxa = 0.0f;
            if (b < nb) {
                const uint4 a0 = *reinterpret_cast<const uint4 *>(aq + b * 32);
                const uint4 a1 = *reinterpret_cast<const uint4 *>(aq + b * 32 + 16);
                av[0] = a0.x, av[1] = a0.y, av[2] = a0.z, av[3] = a0.w, av[4] = a1.x, av[5] = a1.y, av[6] = a1.z, av[7] = a1.w;
                dxa = h2f(ad[b]);
            }
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const bool on = r0 + 4 * g + r4 < a.H && b < nb;
                int p[8];
                float ds = 0.0f;
                if (on) {
                    q8_chunks<0>(wb[i][g], av, p);
                    ds = h2f(wb[i][g].d) * dxa;
                } else {
#pragma unroll
                    for (int q = 0; q < 8; ++q) p[q] = 0;
                }
                wave_lds_fence();  // earlier reads of the tile are done before it is overwritten
                float4 *dst = reinterpret_cast<float4 *>(&tile.pf[0][r4 * 136 + b * 8]);
                dst[0] = make_float4(static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]),
                                     static_cast<float>(p[3]));
                dst[1] = make_float4(static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]),
                                     static_cast<float>(p[7]));
                tile.ds[0][lane] = ds;
                wave_lds_fence();
                float acc = 0.0f;
#pragma unroll
                for (int s = 0; s < 16; ++s)  // slots past the row's end hold zeros: fma(0, 0, acc) == acc
                    acc = __builtin_fmaf(tile.ds[0][r4 * 16 + s], tile.pf[0][r4 * 136 + s * 8 + c], acc);
                const float y = close_lanes8(acc);
                if ((lane & 15) == 0) ybuf[(it_t[i] * (a.k + 1) + it_j[i]) * 8 + 4 * g + r4] = y;
            }
            mark(a, 2, 2 + i);
        }
    }
    __syncthreads();
    mark(a, 2, 5);
    if (tw < ta.T) {
        const TokenSlots &s = ta.tok[tw];
        const int t = tw;
        const int row = r0 + lane;
        const bool row_on = lane < 8 && row < a.H;
        float acc = 0.0f;
        for (int j = 0; j < a.k; ++j) {
            const float wj = lane_get(wreg, j);
            const float y = ybuf[(t * (a.k + 1) + j) * 8 + (lane & 7)];
            const float prod = y * wj;
            acc = acc + prod;
            if (s.expert_out && row_on) s.expert_out[static_cast<size_t>(j) * a.H + row] = y;
        }
        const float gate = lane_get(wreg, 16);
        if (row_on) {
            float o = acc;
            if (shared) {
                const float y = ybuf[(t * (a.k + 1) + a.k) * 8 + lane];
                const float prod = y * gate;
                o = acc + prod;
                s.down_f32[row] = y;
            }
            s.accum[row] = acc;
            s.out[row] = o;
        }
    }
    mark(a, 2, 6);
}

// The same for IQ4_NL (KIND 1) or Q8_0 (KIND 0) rows of NB = 16 or 20 blocks in 16-byte aligned groups of four, fetched as
// aligned words (q8_rows4_coal): preferred over k_tokens_c where both apply (aligned Q8_0 rows of 16 blocks).  Eight rows per workgroup, 16 waves, an
// item is (token, matrix) with the shared expert (always Q8_0) as matrix k; a wave has the two row groups of two items
// in flight.  dynamic LDS per wave: F bytes + F/32 halves (+ pad), then [T][k+1][8] floats.
template <int KIND, int NB>
__global__ __launch_bounds__(1024) void k_tokens_c_nb(TokenArgs ta) {
    extern __shared__ __align__(16) uint8_t lds_tn[];
    __shared__ Q8TileNB<NB> tiles[16];
    const LayerArgs &a = ta.common;
    const int lane = threadIdx.x & 63;
    constexpr int kWaves = 16, kItems = 2, kF = NB * 32;
    using RawQ8 = Q8CoalRaw<0, NB>;
    using RawW = Q8CoalRaw<KIND, NB>;
    const int tw = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const size_t per_wave = (static_cast<size_t>(kF) + kF / 16 + 15) & ~static_cast<size_t>(15);
    int8_t *aq = reinterpret_cast<int8_t *>(lds_tn + tw * per_wave);
    uint16_t *ad = reinterpret_cast<uint16_t *>(lds_tn + tw * per_wave + kF);
    float *ybuf = reinterpret_cast<float *>(lds_tn + kWaves * per_wave);  // [T][k+1][8]
    const bool shared = a.sh_down != nullptr;
    const int per_token = a.k + (shared ? 1 : 0);
    const int n_items = ta.T * per_token;
    const int r0 = blockIdx.x * 8;  // hidden is a multiple of 8
    const int r4 = lane >> 4;
    const int id_lo = token_pair_id(ta, lane), id_hi = token_pair_id(ta, lane + 64);
    float wreg;
    {
        const TokenSlots &s = ta.tok[min(tw, ta.T - 1)];
        const float *src = (lane == 16 && shared) ? s.shared_gate : s.weights + min(lane, a.k - 1);
        wreg = *src;
    }
    Q8TileNB<NB> &tile = tiles[tw];
    for (int item0 = 0; item0 < n_items; item0 += kWaves * kItems) {
        int it_t[kItems], it_j[kItems];
        bool it_on[kItems];
        float4 v0[kItems], v1[kItems], v2[kItems], v3[kItems];
        uint4 raw[kItems][2][RawQ8::kLoads];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {  // unconditional loads: an item past the end repeats the last one
            const int item = item0 + tw + kWaves * i;
            it_on[i] = item < n_items;
            const int ic = min(item, n_items - 1);
            it_t[i] = ic / per_token, it_j[i] = ic - it_t[i] * per_token;
            const float *act = ta.tok[it_t[i]].act + static_cast<size_t>(it_j[i]) * kF;
            v0[i] = *reinterpret_cast<const float4 *>(act + lane * 8);
            v1[i] = *reinterpret_cast<const float4 *>(act + lane * 8 + 4);
            if (NB == 20) {  // values 512..639: lanes 0..15 (the others repeat them)
                v2[i] = *reinterpret_cast<const float4 *>(act + 512 + (lane & 15) * 8);
                v3[i] = *reinterpret_cast<const float4 *>(act + 512 + (lane & 15) * 8 + 4);
            }
        }
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const bool is_shared = it_j[i] == a.k;
            const int pair = it_t[i] * a.k + (is_shared ? 0 : it_j[i]);
            const int e = pair < 64 ? __builtin_amdgcn_readlane(id_lo, pair) : __builtin_amdgcn_readlane(id_hi, pair - 64);
            const uint8_t *w = is_shared ? a.sh_down : mat_ptr_entry<0>(a.down, e);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                if (KIND == 0 || is_shared) {  // wave-uniform
                    const RawQ8 r = q8_rows4_coal_request<0, NB>(w + static_cast<size_t>(r0 + 4 * g) * NB * 34, lane);
#pragma unroll
                    for (int q = 0; q < RawQ8::kLoads; ++q) raw[i][g][q] = r.u[q];
                } else {
                    const RawW r = q8_rows4_coal_request<KIND, NB>(w + static_cast<size_t>(r0 + 4 * g) * NB * RawW::kBlk, lane);
#pragma unroll
                    for (int q = 0; q < RawW::kLoads; ++q) raw[i][g][q] = r.u[q];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if (!it_on[i]) continue;  // uniform
            const bool is_shared = it_j[i] == a.k;
            wave_lds_fence();
            lds_quantize_q8_0_step(v0[i], v1[i], true, lane * 8, aq, ad, lane);
            if (NB == 20) lds_quantize_q8_0_step(v2[i], v3[i], lane < 16, 512 + (lane & 15) * 8, aq, ad, lane);
            wave_lds_fence();
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                float y;
                if (KIND == 0 || is_shared) {
                    RawQ8 r;
#pragma unroll
                    for (int q = 0; q < RawQ8::kLoads; ++q) r.u[q] = raw[i][g][q];
                    y = q8_rows4_coal_finish<0, NB>(r, aq, ad, tile, lane);
                } else {
                    RawW r;
#pragma unroll
                    for (int q = 0; q < RawW::kLoads; ++q) r.u[q] = raw[i][g][q];
                    y = q8_rows4_coal_finish<KIND, NB>(r, aq, ad, tile, lane);
                }
                if ((lane & 15) == 0) ybuf[(it_t[i] * (a.k + 1) + it_j[i]) * 8 + 4 * g + r4] = y;
            }
        }
    }
    __syncthreads();
    if (tw < ta.T) {
        const TokenSlots &s = ta.tok[tw];
        const int row = r0 + lane;
        const bool row_on = lane < 8;
        float acc = 0.0f;
        for (int j = 0; j < a.k; ++j) {
            const float wj = lane_get(wreg, j);
            const float y = ybuf[(tw * (a.k + 1) + j) * 8 + (lane & 7)];
            const float prod = y * wj;
            acc = acc + prod;
            if (s.expert_out && row_on) s.expert_out[static_cast<size_t>(j) * a.H + row] = y;
        }
        const float gate = lane_get(wreg, 16);
        if (row_on) {
            float o = acc;
            if (shared) {
                const float y = ybuf[(tw * (a.k + 1) + a.k) * 8 + lane];
                const float prod = y * gate;
                o = acc + prod;
                s.down_f32[row] = y;
            }
            s.accum[row] = acc;
            s.out[row] = o;
        }
    }
}

}  // namespace wd
