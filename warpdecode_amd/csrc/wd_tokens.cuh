// M tokens through one MoE layer with every selected expert's weights read once.
//
// The reference batches M tokens as M*k (token, expert) pairs and re-reads an expert's weights for
// every pair that names it (src/qwen38_moe.cuh:1316-1437, :2743-3237).  Here the pairs are first
// folded into the union of selected experts; a workgroup loads a weight row once and applies it to
// the activation of every token that routed to that expert.  Per token, the arithmetic and its order
// are those of the one-token kernels, so the results are bit-identical to M separate passes.
#pragma once

#include "wd_fused.cuh"

namespace wd {

constexpr int kMaxTokens = 8;

struct TokenArgs {
    int T, H, F, k;
    const float *x[kMaxTokens];
    int32_t *ids[kMaxTokens];
    float *weights[kMaxTokens];
    float *act[kMaxTokens];          // [k+1][F]
    float *shared_gate[kMaxTokens];
    float *expert_out[kMaxTokens];   // null or [k][H]
    float *accum[kMaxTokens], *down_f32[kMaxTokens], *out[kMaxTokens];
    MatSrc gate_up, down;
    const uint8_t *sh_down;          // null = no shared expert
    int32_t *union_count;            // [1]
    int32_t *union_ids;              // [T*k]
    int32_t *union_slot;             // [T*k][kMaxTokens]: position j of the expert in token t's list, or -1
};

// One wave: folds the T*k routed ids (T*k <= 128) into their union, in order of first appearance.
__global__ __launch_bounds__(64) void k_tokens_union(TokenArgs a) {
    __shared__ int32_t s_id[128];
    __shared__ int32_t s_upos[128];
    const int lane = threadIdx.x;
    const int n = a.T * a.k;
    for (int i = lane; i < 128; i += 64) s_id[i] = (i < n) ? a.ids[i / a.k][i % a.k] : -1;
    for (int i = lane; i < n * kMaxTokens; i += 64) a.union_slot[i] = -1;
    __syncthreads();
    int first[2], is_first[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int i = lane + 64 * h;
        first[h] = i;
        if (i < n) {
            for (int q = 0; q < i; ++q)
                if (s_id[q] == s_id[i]) {
                    first[h] = q;
                    break;
                }
        }
        is_first[h] = (i < n) && first[h] == i;
    }
    const unsigned long long m0 = __builtin_amdgcn_ballot_w64(is_first[0] != 0);
    const unsigned long long m1 = __builtin_amdgcn_ballot_w64(is_first[1] != 0);
    const unsigned long long below = (1ull << lane) - 1ull;
    const int up0 = __builtin_popcountll(m0 & below);
    const int up1 = __builtin_popcountll(m0) + __builtin_popcountll(m1 & below);
    if (is_first[0]) {
        s_upos[lane] = up0;
        a.union_ids[up0] = s_id[lane];
    }
    if (is_first[1]) {
        s_upos[lane + 64] = up1;
        a.union_ids[up1] = s_id[lane + 64];
    }
    if (lane == 0) a.union_count[0] = __builtin_popcountll(m0) + __builtin_popcountll(m1);
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int i = lane + 64 * h;
        if (i < n) a.union_slot[s_upos[first[h]] * kMaxTokens + i / a.k] = i % a.k;
    }
}

// gate/up + SwiGLU of the union experts.  grid = (T*k) * ceil(F/8), 512 threads: one (gate, up) row
// pair per wave, loaded once, applied to every token that selected the expert.
// dynamic LDS: T * (H bytes + H/256 floats).
template <int TYPE>
__global__ __launch_bounds__(512) void k_tokens_b(TokenArgs a) {
    extern __shared__ __align__(16) uint8_t lds_tb[];
    __shared__ IqTables tables;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int groups = (a.F + 7) / 8;
    const int u = blockIdx.x / groups, rg = blockIdx.x - u * groups;
    if (u >= a.union_count[0]) return;
    const int e = a.union_ids[u];
    int slot[kMaxTokens];
#pragma unroll
    for (int t = 0; t < kMaxTokens; ++t) slot[t] = (t < a.T) ? a.union_slot[u * kMaxTokens + t] : -1;
    int8_t *xq = reinterpret_cast<int8_t *>(lds_tb);
    float *xd = reinterpret_cast<float *>(lds_tb + static_cast<size_t>(a.T) * a.H);
    constexpr int kBlk = (TYPE == 21) ? 110 : 82;
    const int nb = a.H >> 8;
    const size_t rb = static_cast<size_t>(nb) * kBlk;
    const int r = rg * 8 + wave;
    const size_t off = static_cast<size_t>(min(r, a.F - 1)) * rb;
    const uint8_t *const rows[2] = {mat_ptr_ids(a.gate_up, 0, e) + off, mat_ptr_ids(a.gate_up, 1, e) + off};
    const int ib = lane >> 3, sbl = lane & 7;
    const bool first = sbl == 0;
    float acc[kMaxTokens][2];
#pragma unroll
    for (int t = 0; t < kMaxTokens; ++t) acc[t][0] = acc[t][1] = 0.0f;
    for (int base = 0; base < nb; base += 8) {
        const int sb = base + sbl;
        const bool on = sb < nb;
        IqFields f[2];
        if (on) {
            f[0] = iq_load<TYPE>(rows[0] + static_cast<size_t>(sb) * kBlk, ib);
            f[1] = iq_load<TYPE>(rows[1] + static_cast<size_t>(sb) * kBlk, ib);
        }
        if (base == 0) {
            stage_tables<TYPE == 21, TYPE == 22>(tables, threadIdx.x, 512);
            for (int b = wave; b < a.T * nb; b += 8) {
                const int t = b / nb, bb = b - t * nb;
                wave_quantize_q8_k_block(a.x[t] + bb * 256, xq + static_cast<size_t>(t) * a.H + bb * 256, xd + t * nb + bb, lane);
            }
            __syncthreads();
        }
#pragma unroll
        for (int t = 0; t < kMaxTokens; ++t) {
            if (slot[t] < 0) continue;  // uniform
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
                    iq_chunks<TYPE>(f[i], ib, tables, av, p);
                    ds = h2f(f[i].d) * dx;
                } else {
#pragma unroll
                    for (int c = 0; c < 8; ++c) p[c] = 0;
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
#pragma unroll
    for (int t = 0; t < kMaxTokens; ++t) {
        if (slot[t] < 0) continue;
        float g = close_lanes8_strided(acc[t][0]), up = close_lanes8_strided(acc[t][1]);
        if (TYPE == 22) {
            g = 0.125f * g;
            up = 0.125f * up;
        }
        if (lane == 0 && r < a.F) a.act[t][static_cast<size_t>(slot[t]) * a.F + r] = silu_ggml(g) * up;
    }
}

// Down projections + ordered combine for T tokens.  grid = ceil(H/4), block = 64 * waves.
// Wave w walks the union entries w, w + waves, ... and then (entry U) the shared expert; it loads
// its four rows of the entry's down tensor once (F <= 512: one block per lane) and applies them to
// the Q8_0 activation of every token that uses the entry.  Waves 0..T-1 then fold token t's results
// in its own top-k order.  dynamic LDS: per wave F bytes + F/32 halves (+pad), then [T][k+1][4] floats.
__global__ __launch_bounds__(1024) void k_tokens_c(TokenArgs a) {
    extern __shared__ __align__(16) uint8_t lds_tc[];
    __shared__ Q8Tile tiles[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const size_t per_wave = (static_cast<size_t>(a.F) + a.F / 16 + 15) & ~static_cast<size_t>(15);
    int8_t *aq = reinterpret_cast<int8_t *>(lds_tc + wave * per_wave);
    uint16_t *ad = reinterpret_cast<uint16_t *>(lds_tc + wave * per_wave + a.F);
    float *ybuf = reinterpret_cast<float *>(lds_tc + nwaves * per_wave);  // [T][k+1][4]
    const bool shared = a.sh_down != nullptr;
    const int U = a.union_count[0];
    const int n_entries = U + (shared ? 1 : 0);
    const int r0 = blockIdx.x * 4;
    const int nrows = min(4, a.H - r0);
    const int nb = a.F >> 5;  // <= 16
    const int r4 = lane >> 4, b = lane & 15, c = lane & 7;
    const bool on = r4 < nrows && b < nb;
    Q8Tile &tile = tiles[wave];
    for (int u = wave; u < n_entries; u += nwaves) {
        const bool is_shared = u == U;
        const uint8_t *w = is_shared ? a.sh_down : mat_ptr_ids(a.down, 0, a.union_ids[u]);
        Q8Block wb;
        if (on) wb = q8_load<0>(w + (static_cast<size_t>(r0 + r4) * nb + b) * 34);
        for (int t = 0; t < a.T; ++t) {
            const int j = is_shared ? a.k : a.union_slot[u * kMaxTokens + t];
            if (j < 0) continue;  // uniform
            wave_lds_fence();
            lds_quantize_q8_0(a.act[t] + static_cast<size_t>(j) * a.F, a.F, aq, ad, lane, 64);
            wave_lds_fence();
            int p[8];
            float ds = 0.0f;
            if (on) {
                const uint4 a0 = *reinterpret_cast<const uint4 *>(aq + b * 32);
                const uint4 a1 = *reinterpret_cast<const uint4 *>(aq + b * 32 + 16);
                const uint32_t av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                q8_chunks<0>(wb, av, p);
                ds = h2f(wb.d) * h2f(ad[b]);
            } else {
#pragma unroll
                for (int q = 0; q < 8; ++q) p[q] = 0;
            }
            float4 *dst = reinterpret_cast<float4 *>(&tile.pf[0][r4 * 136 + b * 8]);
            dst[0] = make_float4(static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]),
                                 static_cast<float>(p[3]));
            dst[1] = make_float4(static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]),
                                 static_cast<float>(p[7]));
            tile.ds[0][lane] = ds;
            wave_lds_fence();
            float acc = 0.0f;
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < nb) acc = __builtin_fmaf(tile.ds[0][r4 * 16 + s], tile.pf[0][r4 * 136 + s * 8 + c], acc);
            const float y = close_lanes8(acc);
            if ((lane & 15) == 0) ybuf[(t * (a.k + 1) + j) * 4 + r4] = y;
        }
    }
    __syncthreads();
    for (int t = wave; t < a.T; t += nwaves) {
        if (lane >= nrows) continue;
        const int row = r0 + lane;
        float acc = 0.0f;
        for (int j = 0; j < a.k; ++j) {
            const float y = ybuf[(t * (a.k + 1) + j) * 4 + lane];
            const float prod = y * a.weights[t][j];
            acc = acc + prod;
            if (a.expert_out[t]) a.expert_out[t][static_cast<size_t>(j) * a.H + row] = y;
        }
        float o = acc;
        if (shared) {
            const float y = ybuf[(t * (a.k + 1) + a.k) * 4 + lane];
            const float prod = y * a.shared_gate[t][0];
            o = acc + prod;
            a.down_f32[t][row] = y;
        }
        a.accum[t][row] = acc;
        a.out[t][row] = o;
    }
}

}  // namespace wd
