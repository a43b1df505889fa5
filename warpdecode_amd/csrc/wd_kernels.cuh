// __global__ kernels of the stand-alone operators (64-wide wavefronts, 256-thread workgroups).
#pragma once

#include "wd_rows.cuh"

namespace wd {

// Where the weight matrices of a grouped dispatch live.
//   table != null      matrix m = table[m]                       (expert pointer table)
//   ids   != null      matrix m belongs to expert ids[m / per_expert], tensor m % per_expert:
//                        resident:  base[t] + expert * stride[t]
//                        slot pool: pool + slot_of_expert[expert] * slot_bytes + slot_off[t]
//   otherwise          the single matrix `single`
struct MatSrc {
    const uint8_t *single;
    const uint8_t *const *table;
    const int32_t *ids;
    int per_expert;
    const uint8_t *base[2];
    size_t stride[2];
    const int32_t *slot_of_expert;
    const uint8_t *pool;
    size_t slot_bytes;
    size_t slot_off[2];
    unsigned *slot_status;  // set to 2 when an expert without a slot is asked for (may be null)
};

// The slot of an expert that is not in the pool is -1: such a request is reported through the status word and reads
// slot 0 (memory that exists, values that mean nothing) instead of an address before the pool.
WD_DEV size_t checked_slot(const MatSrc &s, int slot) {
    if (slot < 0) {
        if (s.slot_status) __hip_atomic_store(s.slot_status, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        slot = 0;
    }
    return static_cast<size_t>(slot);
}

WD_DEV const uint8_t *mat_ptr(const MatSrc &s, int m) {
    if (s.table) return s.table[m];
    if (s.ids) {
        const int j = m / s.per_expert, t = m - j * s.per_expert;
        const int e = s.ids[j];
        if (s.slot_of_expert) return s.pool + checked_slot(s, s.slot_of_expert[e]) * s.slot_bytes + s.slot_off[t];
        return s.base[t] + static_cast<size_t>(e) * s.stride[t];
    }
    return s.single;
}

// Tensor T (0 = the first, 1 = the second of an expert's tensors in this source) of expert e.  T is a template
// argument so that base, stride and slot offset are fixed members of the argument block (scalar registers, loaded
// without waiting for e) instead of a lookup by a computed index.
template <int T>
WD_DEV const uint8_t *mat_ptr_expert(const MatSrc &s, int e) {
    if (s.slot_of_expert) return s.pool + checked_slot(s, s.slot_of_expert[e]) * s.slot_bytes + s.slot_off[T];
    return s.base[T] + static_cast<size_t>(e) * s.stride[T];
}

// The same for an e that is the same in every lane: the slot comes through the scalar path, so the lookup neither
// waits for nor is counted among the wave's vector loads.
template <int T>
WD_DEV const uint8_t *mat_ptr_expert_uniform(const MatSrc &s, int e) {
    if (s.slot_of_expert) return s.pool + checked_slot(s, sld_i32(s.slot_of_expert + e)) * s.slot_bytes + s.slot_off[T];
    return s.base[T] + static_cast<size_t>(e) * s.stride[T];
}

__global__ void k_fill_u32(uint32_t *dst, uint32_t v, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = v;
}

// ---- Q8_K quantiser: one wave per 256-value block, four values per lane -------------------
__global__ __launch_bounds__(256) void k_q8_k_quantize(const float *__restrict__ x, int blocks,
                                                        int8_t *__restrict__ qs, float *__restrict__ scales,
                                                        int16_t *__restrict__ bsums) {
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= blocks) return;
    const float4 v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(blk) * 256)[lane];
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    amax = wave_max_nonneg(amax);
    uint32_t packed = 0;
    int part = 0;
    float d = 0.0f;
    if (amax != 0.0f) {
        // always-negative inverse scale (reference convention): quants carry the sign of -x
        const float iscale = -127.0f / amax;
        const int q0 = min(127, static_cast<int>(__builtin_rintf(v.x * iscale)));
        const int q1 = min(127, static_cast<int>(__builtin_rintf(v.y * iscale)));
        const int q2 = min(127, static_cast<int>(__builtin_rintf(v.z * iscale)));
        const int q3 = min(127, static_cast<int>(__builtin_rintf(v.w * iscale)));
        packed = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
        part = q0 + q1 + q2 + q3;
        d = 1.0f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs + static_cast<size_t>(blk) * 256)[lane] = packed;
    part = quad_sum_i(part);
    if ((lane & 3) == 0) bsums[static_cast<size_t>(blk) * 16 + (lane >> 2)] = static_cast<int16_t>(part);
    if (lane == 0) scales[blk] = d;
}

// ---- Q8_0 quantiser: eight lanes per 32-value block, four values per lane -----------------
// (inv: 127 / amax, for a caller that packs more than four values of a block)
WD_DEV uint32_t q8_0_pack4_scaled(float4 v, float inv) {
    const int q0 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.x * inv))));
    const int q1 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.y * inv))));
    const int q2 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.z * inv))));
    const int q3 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.w * inv))));
    return (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
}
WD_DEV uint32_t q8_0_pack4(float4 v, float amax) {
    if (amax == 0.0f) return 0u;
    const float inv = 127.0f / amax;
    const int q0 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.x * inv))));
    const int q1 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.y * inv))));
    const int q2 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.z * inv))));
    const int q3 = max(-128, min(127, static_cast<int>(__builtin_rintf(v.w * inv))));
    return (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
}

__global__ __launch_bounds__(256) void k_q8_0_quantize(const float *__restrict__ x, int blocks,
                                                        int8_t *__restrict__ qs, uint16_t *__restrict__ scales) {
    const int sub = threadIdx.x & 7;
    const int blk = blockIdx.x * 32 + (threadIdx.x >> 3);
    const bool on = blk < blocks;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (on) v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(blk) * 32)[sub];
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    amax = oct_max_nonneg(amax);
    if (!on) return;
    reinterpret_cast<uint32_t *>(qs + static_cast<size_t>(blk) * 32)[sub] = q8_0_pack4(v, amax);
    if (sub == 0) scales[blk] = f2h_ref(amax / 127.0f);
}

// ---- the reference's plain Q8_0 x Q8_1 path and its half-input quantiser ----------------------------------------
// IEEE float -> half bits (the reference's __float2half), unlike f2h_ref.
WD_DEV uint16_t f2h_rn(float v) {
    const _Float16 f = static_cast<_Float16>(v);
    uint16_t h;
    __builtin_memcpy(&h, &f, 2);
    return h;
}
// The largest |v| of the block of 32 values held four per lane by eight consecutive lanes.
WD_DEV float block32_amax(const float4 &v) {
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    return oct_max_nonneg(amax);
}
// q8_1_quantize_f32_kernel, src/lowbit.cuh:287-308: d = amax / 127, q = roundf(x / d) (a division; halves away from
// zero), scale = half(d).  Eight lanes per block, four values per lane.
__global__ __launch_bounds__(256) void k_q8_1_quantize(const float *__restrict__ x, int blocks, int8_t *__restrict__ qs,
                                                        uint16_t *__restrict__ scales) {
    const int sub = threadIdx.x & 7;
    const int blk = blockIdx.x * 32 + (threadIdx.x >> 3);
    const bool on = blk < blocks;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (on) v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(blk) * 32)[sub];
    const float amax = block32_amax(v);
    if (!on) return;
    const float d = amax / 127.0f;
    auto q = [&](float t) { return amax == 0.0f ? 0 : static_cast<int>(__builtin_roundf(t / d)); };
    const int q0 = q(v.x), q1 = q(v.y), q2 = q(v.z), q3 = q(v.w);
    reinterpret_cast<uint32_t *>(qs + static_cast<size_t>(blk) * 32)[sub] =
        (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
    if (sub == 0) scales[blk] = f2h_rn(d);
}
// q8_0_quantize_half_kernel, src/warodecode.cu:1504-1520: half input, inv = 127 / amax, q = lrintf(v * inv) clamped to
// +-127, scale = half(amax / 127).
__global__ __launch_bounds__(256) void k_q8_0_quantize_f16(const uint16_t *__restrict__ x, int blocks, int8_t *__restrict__ qs,
                                                            uint16_t *__restrict__ scales) {
    const int sub = threadIdx.x & 7;
    const int blk = blockIdx.x * 32 + (threadIdx.x >> 3);
    const bool on = blk < blocks;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (on) {
        const uint2 h = reinterpret_cast<const uint2 *>(x + static_cast<size_t>(blk) * 32)[sub];
        v = make_float4(h2f(static_cast<uint16_t>(h.x)), h2f(static_cast<uint16_t>(h.x >> 16)), h2f(static_cast<uint16_t>(h.y)),
                        h2f(static_cast<uint16_t>(h.y >> 16)));
    }
    const float amax = block32_amax(v);
    if (!on) return;
    const float inv = amax == 0.0f ? 0.0f : 127.0f / amax;
    auto q = [&](float t) { return max(-127, min(127, static_cast<int>(__builtin_rintf(t * inv)))); };
    const int q0 = q(v.x), q1 = q(v.y), q2 = q(v.z), q3 = q(v.w);
    reinterpret_cast<uint32_t *>(qs + static_cast<size_t>(blk) * 32)[sub] =
        (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | (static_cast<uint32_t>(q3 & 0xff) << 24);
    if (sub == 0) scales[blk] = f2h_rn(amax / 127.0f);
}
// q8_0_q8_1_gemv_f32_kernel, src/lowbit.cuh:310-341: one wave per row, lane = block (64 blocks a pass); the row's sum
// runs over the blocks in ascending order, one rounded multiply of the two scales, one with the integer sum, one add.
// block_sums (optional): int32 [rows][cols / 32].
__global__ __launch_bounds__(256) void k_gemv_q8_0_q8_1(const uint8_t *__restrict__ w, int rows, int cols,
                                                         const int8_t *__restrict__ qs, const uint16_t *__restrict__ scales,
                                                         float *__restrict__ y, int32_t *__restrict__ block_sums) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nb = cols >> 5;
    const uint8_t *wr = w + static_cast<size_t>(row) * nb * 34;
    float sum = 0.0f;
    for (int base = 0; base < nb; base += 64) {
        const int b = base + lane;
        float prod = 0.0f;
        if (b < nb) {
            const uint8_t *blk = wr + static_cast<size_t>(b) * 34;
            int dot = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t wq = static_cast<uint32_t>(ldu<uint16_t>(blk + 2 + 4 * i)) | (static_cast<uint32_t>(ldu<uint16_t>(blk + 4 + 4 * i)) << 16);
                dot = sdot4(wq, *reinterpret_cast<const uint32_t *>(qs + b * 32 + 4 * i), dot);
            }
            if (block_sums) block_sums[static_cast<size_t>(row) * nb + b] = dot;
            const float scale = h2f(ldu<uint16_t>(blk)) * h2f(scales[b]);
            prod = scale * static_cast<float>(dot);
        }
        const int n = min(64, nb - base);
        for (int i = 0; i < n; ++i) sum = sum + readlane_f(prod, i);
    }
    if (lane == 0) y[row] = sum;
}
// Element-wise half <-> float (IEEE rounding on the way down).
__global__ void k_f16_to_f32(const uint16_t *__restrict__ src, float *__restrict__ dst, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = h2f(src[i]);
}
__global__ void k_f32_to_f16(const float *__restrict__ src, uint16_t *__restrict__ dst, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = f2h_rn(src[i]);
}

// ---- router GEMV: 32 lanes per row, lane t owns accumulator t of the 4x8 scheme --------------
// (src/qwen38_moe.cuh:198-245).  Optional extra row (the shared expert's gate vector).
__global__ __launch_bounds__(256) void k_router_gemv(const float *__restrict__ w, const float *__restrict__ x,
                                                      float *__restrict__ logits, int rows, int cols,
                                                      const float *__restrict__ extra_w,
                                                      float *__restrict__ extra_out) {
    const int t = threadIdx.x & 31;
    const int row = blockIdx.x * 8 + (threadIdx.x >> 5);
    const int total = rows + (extra_w ? 1 : 0);
    const bool on = row < total;
    const float *wr = on ? (row < rows ? w + static_cast<size_t>(row) * cols : extra_w) : w;
    const int np = cols & ~31;
    float s = 0.0f;
    if (on) {
#pragma unroll 16
        for (int i = 0; i < np; i += 32) s = __builtin_fmaf(wr[i + t], x[i + t], s);
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
        if (row < rows)
            logits[row] = acc;
        else
            extra_out[0] = acc;
    }
}

// ---- IQ3_S / IQ2_S x Q8_K GEMV: 16 rows per workgroup, 4 per wave, grid.y = matrix -----------
template <int TYPE, bool PART>
__global__ __launch_bounds__(256) void k_gemv_iq(MatSrc src, int rows, int cols, const int8_t *__restrict__ act_qs,
                                                  const float *__restrict__ act_d, float *__restrict__ out,
                                                  int32_t *__restrict__ partials, int ppr) {
    __shared__ IqTables tables;
    stage_tables<TYPE == 21, TYPE == 22>(tables, threadIdx.x, 256);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = blockIdx.y;
    const uint8_t *w = mat_ptr(src, m);
    const int nb = cols >> 8;
    const size_t rb = static_cast<size_t>(nb) * (TYPE == 21 ? 110 : 82);
    const int r0 = blockIdx.x * 16 + wave * 4;
    for (int r = r0; r < min(rows, r0 + 4); ++r) {
        int32_t *pp = PART ? partials + (static_cast<size_t>(m) * rows + r) * ppr : nullptr;
        const float y = iq_row_q8k<TYPE, PART>(w + static_cast<size_t>(r) * rb, nb, tables, act_qs, act_d, lane, pp);
        if (lane == 0) out[static_cast<size_t>(m) * rows + r] = y;
    }
}

// ---- Q8_0 / IQ4_NL / Q4_0 x Q8_0 GEMV: 16 rows per workgroup, 4 per wave ----------------------
// act_stride: elements between the activations of consecutive matrices (0 = one shared activation).
template <int KIND, bool PART>
__global__ __launch_bounds__(256) void k_gemv_q8(MatSrc src, int rows, int cols, const int8_t *__restrict__ act_qs,
                                                  const uint16_t *__restrict__ act_d, int act_stride,
                                                  float *__restrict__ out, int32_t *__restrict__ partials, int ppr) {
    __shared__ Q8Tile tiles[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = blockIdx.y;
    const uint8_t *w = mat_ptr(src, m);
    const int nb = cols >> 5;
    const int8_t *aq = act_qs + static_cast<size_t>(m) * act_stride;
    const uint16_t *ad = act_d + static_cast<size_t>(m) * (act_stride >> 5);
    const int r0 = blockIdx.x * 16 + wave * 4;
    if (r0 >= rows) return;
    const int nrows = min(4, rows - r0);
    const size_t rb = static_cast<size_t>(nb) * (KIND == 0 ? 34 : 18);
    int32_t *pp = PART ? partials + (static_cast<size_t>(m) * rows + r0) * ppr : nullptr;
    float y;
    if (KIND == 2)
        y = q4_0_rows4<PART>(w + r0 * rb, nrows, nb, aq, ad, lane, pp);
    else
        y = q8_rows4<(KIND == 1 ? 1 : 0), PART>(w + r0 * rb, nrows, nb, aq, ad, tiles[wave], lane, pp);
    const int r4 = lane >> 4;
    if ((lane & 15) == 0 && r4 < nrows) out[static_cast<size_t>(m) * rows + r0 + r4] = y;
}

// ---- Q4_0 x Q8_0 GEMV, streaming form ---------------------------------------------------------------------
// For matrices whose rows are a whole number of 8-block groups (144 bytes = nine 16-byte words) and whose group
// count per row (lpr) divides 64.  A wave owns 64 consecutive groups per pass (64 * 144 = 9216 contiguous bytes,
// 64 / lpr rows): nine fully coalesced 16-byte loads per lane bring them in, LDS turns the lane-interleaved words
// into one group per lane (both sides conflict-free: stride 16 in, stride 144 out), and the 18-byte blocks are cut
// out of the 36 dwords in registers (even blocks with four byte-align ops, odd blocks are dword aligned).  Lane l
// always works on column group l % lpr.  The workgroup keeps the activation in LDS (each group's 256 bytes padded
// to 272 so that the 16-byte reads of neighbouring groups fall on different banks), with the per-block scale as a
// float and 8 * sum(a) beside it; Block sums are exact; the float side adds a lane's
// eight blocks in order and folds the row's lanes with an xor tree (Q4_0 has no canonical float order).
// A wave takes NP consecutive passes and requests all of them before it touches the first.
// grid.x * WPB waves * NP passes cover ceil(rows / (64 / lpr)) passes.
// dynamic LDS: lpr * 272 bytes of quants, then nb floats, then nb ints.
// (the body: `block` is the workgroup's number among those of its matrix)
template <bool PART, int NP, int WPB>
WD_DEV void gemv_q4_stream_body(const uint8_t *__restrict__ w, int rows, int nb, const int8_t *__restrict__ act_qs,
                                const uint16_t *__restrict__ act_d, float *__restrict__ out, int32_t *__restrict__ partials,
                                int block) {
    __shared__ uint4 stage[WPB][9 * 64];
    extern __shared__ __align__(16) uint8_t q4_act[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lpr = nb >> 3, lpr_shift = __builtin_ctz(lpr), rpp = 64 >> lpr_shift;
    const int col = lane & (lpr - 1), rsub = lane >> lpr_shift;
    float *ad = reinterpret_cast<float *>(q4_act + lpr * 272);
    int *corr = reinterpret_cast<int *>(ad + nb);
    const size_t rb = static_cast<size_t>(nb) * 18;
    const long long pass0 = (static_cast<long long>(block) * WPB + wave) * NP;
    uint4 v[NP][9];
    auto fetch = [&](long long pass, int slot) {
        const long long row0 = pass * rpp;
        const long long left = static_cast<long long>(rows) - row0;
        const size_t valid = left <= 0 ? 0 : static_cast<size_t>(left < rpp ? left : rpp) * rb;
        const uint8_t *base = w + static_cast<size_t>(row0) * rb;
#pragma unroll
        for (int k = 0; k < 9; ++k) {
            const size_t off = static_cast<size_t>(k) * 1024 + static_cast<size_t>(lane) * 16;
            v[slot][k] = off < valid ? gld_u128_aligned(base + off) : make_uint4(0, 0, 0, 0);
        }
    };
    // activation into LDS: thread t takes 16-byte pieces t, t + blockDim.x, ...; a block's two pieces give its sum.  The
    // first piece is requested before the weights so that it can be consumed while they are still in flight.
    const int n_pieces = nb * 2;
    uint4 q0 = make_uint4(0, 0, 0, 0);
    uint16_t d0 = 0;
    if (static_cast<int>(threadIdx.x) < n_pieces) {
        q0 = *reinterpret_cast<const uint4 *>(act_qs + threadIdx.x * 16);
        d0 = act_d[threadIdx.x >> 1];
    }
#pragma unroll
    for (int p = 0; p < NP; ++p) fetch(pass0 + p, p);
    for (int i = threadIdx.x; i < n_pieces; i += WPB * 64) {
        const bool first = i == static_cast<int>(threadIdx.x);
        const uint4 q = first ? q0 : *reinterpret_cast<const uint4 *>(act_qs + i * 16);
        *reinterpret_cast<uint4 *>(q4_act + (i >> 4) * 272 + (i & 15) * 16) = q;
        int s = sdot4(0x01010101u, q.x, 0);
        s = sdot4(0x01010101u, q.y, s);
        s = sdot4(0x01010101u, q.z, s);
        s = sdot4(0x01010101u, q.w, s);
        s += lane_xor(s, 1);
        if ((i & 1) == 0) {
            corr[i >> 1] = 8 * s;
            ad[i >> 1] = h2f(first ? d0 : act_d[i >> 1]);
        }
    }
    __syncthreads();
    const uint8_t *my_act = q4_act + col * 272;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const long long row0 = (pass0 + p) * rpp;
        if (row0 >= rows) break;  // wave-uniform
#pragma unroll
        for (int k = 0; k < 9; ++k) stage[wave][k * 64 + lane] = v[p][k];
        wave_lds_fence();
        uint32_t d[36];
#pragma unroll
        for (int k = 0; k < 9; ++k) {
            const uint4 u = stage[wave][lane * 9 + k];
            d[4 * k] = u.x, d[4 * k + 1] = u.y, d[4 * k + 2] = u.z, d[4 * k + 3] = u.w;
        }
        wave_lds_fence();
        const int row = static_cast<int>(row0) + rsub;
        float sumf = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = j >> 1;
            uint32_t n[4], dw;
            if ((j & 1) == 0) {
                dw = d[9 * m] & 0xffffu;
#pragma unroll
                for (int l = 0; l < 4; ++l) n[l] = __builtin_amdgcn_alignbyte(d[9 * m + l + 1], d[9 * m + l], 2);
            } else {
                dw = d[9 * m + 4] >> 16;
#pragma unroll
                for (int l = 0; l < 4; ++l) n[l] = d[9 * m + 5 + l];
            }
            const uint4 lo = *reinterpret_cast<const uint4 *>(my_act + j * 32), hi = *reinterpret_cast<const uint4 *>(my_act + j * 32 + 16);
            const uint32_t al[4] = {lo.x, lo.y, lo.z, lo.w}, ah[4] = {hi.x, hi.y, hi.z, hi.w};
            int sumi = -corr[col * 8 + j];  // sum (nibble - 8) * a = sum nibble * a - 8 * sum a
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                sumi = sdot4(n[l] & 0x0f0f0f0fu, al[l], sumi);
                sumi = sdot4((n[l] >> 4) & 0x0f0f0f0fu, ah[l], sumi);
            }
            if (PART && row < rows) partials[static_cast<size_t>(row) * nb + col * 8 + j] = sumi;
            sumf += h2f(static_cast<uint16_t>(dw)) * ad[col * 8 + j] * static_cast<float>(sumi);
        }
        for (int mask = lpr >> 1; mask >= 1; mask >>= 1) sumf += lane_xor(sumf, mask);
        if (col == 0 && row < rows) out[row] = sumf;
    }
}
template <bool PART, int NP, int WPB>
__global__ __launch_bounds__(WPB * 64) void k_gemv_q4_stream(const uint8_t *__restrict__ w, int rows, int nb,
                                                         const int8_t *__restrict__ act_qs,
                                                         const uint16_t *__restrict__ act_d, float *__restrict__ out,
                                                         int32_t *__restrict__ partials) {
    gemv_q4_stream_body<PART, NP, WPB>(w, rows, nb, act_qs, act_d, out, partials, static_cast<int>(blockIdx.x));
}
// Several matrices of one row length in one launch (see k_gemv_q8_rows8_split_batch): workgroup b belongs to the item
// whose range of workgroups holds b and does there what k_gemv_q4_stream does for that item alone.
constexpr int kGemvBatchMax = 16;
struct GemvBatch {
    const uint8_t *w[kGemvBatchMax];
    const int8_t *act_qs[kGemvBatchMax];
    const uint16_t *act_d[kGemvBatchMax];
    float *out[kGemvBatchMax];
    int rows[kGemvBatchMax];
    int first_group[kGemvBatchMax + 1];  // the item's first workgroup; first_group[n]: all workgroups
    int n;
};
WD_DEV int gemv_batch_item(const GemvBatch &b) {
    int item = 0;
    for (int i = 1; i < b.n; ++i)
        if (static_cast<int>(blockIdx.x) >= b.first_group[i]) item = i;
    return __builtin_amdgcn_readfirstlane(item);
}
template <int WPB>
__global__ __launch_bounds__(WPB * 64) void k_gemv_q4_stream_batch(GemvBatch b, int nb) {
    const int item = gemv_batch_item(b);
    gemv_q4_stream_body<false, 1, WPB>(b.w[item], b.rows[item], nb, b.act_qs[item], b.act_d[item], b.out[item], nullptr,
                                       static_cast<int>(blockIdx.x) - b.first_group[item]);
}

// ---- dense Q8_0 x Q8_0 GEMV, streaming: one lane per (row, chain) ----------------------------------------------
// The reference order of a Q8_0 row (src/qwen38_cpu_moe.cuh:690-722) is eight chains, chain c over bytes 4c..4c+3 of
// every block, each one fma(d_w d_a, float(dot4), acc) per block in block order: the chains of a row are as long as
// the row, and nothing shortens them.  A wave therefore takes eight rows and gives every (row, chain) pair a lane
// (lane = 8 row + chain): each fma instruction then advances 64 chains, no value crosses lanes until the closing tree,
// and the cost per block and row is under one vector instruction.
// The eight rows are fetched KB blocks at a time (34 KB bytes per row, whole 16-byte words because KB is a multiple of
// 8 and rows start on 16-byte boundaries) with lane-contiguous 16-byte loads, one chunk ahead in a second register set,
// and copied to LDS with a row stride that spreads the eight rows over the banks.  Blocks are 34 bytes, so the four
// bytes of a lane are dword aligned in the odd blocks of a chunk and two bytes off in the even ones (two dwords and a
// v_alignbyte); the parity is the same for every lane, so the unrolled loop knows it at compile time.
// The activation's quants and its scales (as floats) are staged in LDS once per workgroup.
// dynamic LDS: cols bytes, cols/32 floats, then one stage of 8 * kQ8sRowStride<KB> bytes per wave.
template <int KB>
constexpr int kQ8sRowStride = KB == 64 ? 2208 : (KB == 32 ? 1184 : 544);  // 34 KB + padding, 8 (mod 32) dwords

template <int KB>
struct Q8sFetch {
    static constexpr int kWordsPerRow = 34 * KB / 16;                 // 16-byte words of a row's chunk
    static constexpr int kWords = 8 * kWordsPerRow;                    // of the eight rows
    static constexpr int kLoads = (kWords + 63) / 64;
    uint4 u[kLoads];
};

// Eight blocks of a lane's row (lane = 8 row + chain) out of a staged chunk: the lane's four bytes of every block, the
// blocks' scales, the activation's four bytes and scales.  The LDS reads are issued as one group, so that a caller can put
// the next group's before the arithmetic of this one.
struct Q8sBatch {
    uint32_t w[12];  // blocks 0 2 4 6 of the batch: two dwords each (w[3i], w[3i+1]); blocks 1 3 5 7: w[3i+2]
    uint32_t dw[8], a[8];
    float4 da[2];
    // my: the lane's bytes of the chunk's first block; row_blocks: the row's first block in the stage; my_a / ad: the
    // activation's quants at the lane's chain and its scales; b0: the chunk's first block in the row; s: batch in the chunk.
    WD_DEV void load(const uint8_t *my, const uint8_t *row_blocks, const int8_t *my_a, const float *ad, int b0, int s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint8_t *blk = my + 34 * (8 * s + 2 * i);
            w[3 * i] = *reinterpret_cast<const uint32_t *>(blk);
            w[3 * i + 1] = *reinterpret_cast<const uint32_t *>(blk + 4);
            w[3 * i + 2] = *reinterpret_cast<const uint32_t *>(blk + 36);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            dw[i] = *reinterpret_cast<const uint16_t *>(row_blocks + 34 * (8 * s + i));
            a[i] = *reinterpret_cast<const uint32_t *>(my_a + 32 * (b0 + 8 * s + i));
        }
        da[0] = *reinterpret_cast<const float4 *>(ad + b0 + 8 * s);
        da[1] = *reinterpret_cast<const float4 *>(ad + b0 + 8 * s + 4);
    }
    // block i of the batch: its scale product and its chunk sum
    WD_DEV float scale(int i) const {
        const float d[8] = {da[0].x, da[0].y, da[0].z, da[0].w, da[1].x, da[1].y, da[1].z, da[1].w};
        return h2f(static_cast<uint16_t>(dw[i])) * d[i];
    }
    WD_DEV int dot(int i) const {
        const uint32_t q = (i & 1) ? w[3 * (i >> 1) + 2] : __builtin_amdgcn_alignbyte(w[3 * (i >> 1) + 1], w[3 * (i >> 1)], 2);
        return sdot4(q, a[i], 0);
    }
};

// SETS: register sets of fetched chunks in flight per wave (2 for grids of single waves, which have nothing else to
// hide the memory latency with).
template <int KB, bool PART, int WAVES, int SETS>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(WAVES == 1 ? 1 : 4))) void k_gemv_q8_rows8(const uint8_t *__restrict__ w, int rows, int nb,
                                                              const int8_t *__restrict__ act_qs, const uint16_t *__restrict__ act_d,
                                                              float *__restrict__ out, int32_t *__restrict__ partials) {
    using Fetch = Q8sFetch<KB>;
    constexpr int RS = kQ8sRowStride<KB>;
    extern __shared__ __align__(16) uint8_t q8s_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cols = nb * 32;
    int8_t *aq = reinterpret_cast<int8_t *>(q8s_lds);
    float *ad = reinterpret_cast<float *>(q8s_lds + cols);
    uint8_t *stage = q8s_lds + cols + nb * 4 + wave * (8 * RS);
    const size_t rb = static_cast<size_t>(nb) * 34;
    // the waves of the grid take the groups of eight rows in turn (rows >= 8)
    const int n_groups = (rows + 7) >> 3, n_waves = gridDim.x * WAVES, first = blockIdx.x * WAVES + wave;
    const int my_groups = first < n_groups ? (n_groups - first + n_waves - 1) / n_waves : 0;
    const int nchunks = nb / KB;
    // where the lane's words of a chunk lie: in memory (relative to the chunk of the group's first row) and in the stage
    const int row = lane >> 3, c = lane & 7;
    uint32_t goff[Fetch::kLoads], loff[Fetch::kLoads];
#pragma unroll
    for (int i = 0; i < Fetch::kLoads; ++i) {
        const int u = min(i * 64 + lane, Fetch::kWords - 1);
        const int r = u / Fetch::kWordsPerRow, within = u - r * Fetch::kWordsPerRow;
        goff[i] = static_cast<uint32_t>(r * rb + 16 * within);
        loff[i] = static_cast<uint32_t>(r * RS + 16 * within);
    }
    // the fetch runs SETS chunks ahead of the arithmetic, over the group boundaries
    int f_group = min(first, n_groups - 1), f_chunk = 0, fetched = 0;
    const int items = my_groups * nchunks;
    Fetch fs[SETS];
    auto fetch = [&](Fetch &f) {
        // a last group of fewer than eight rows is moved up to end with the matrix: it then repeats rows of the group
        // before it, which come out the same
        const uint8_t *p = uniform_ptr(w + static_cast<size_t>(min(8 * f_group, rows - 8)) * rb + static_cast<size_t>(f_chunk) * (34 * KB));
#pragma unroll
        for (int i = 0; i < Fetch::kLoads; ++i) f.u[i] = gld_u128_aligned(p + goff[i]);
        // past the wave's last chunk the same chunk is requested again (and not used), so that every turn issues the
        // same number of requests
        if (++fetched < items) {
            if (++f_chunk == nchunks) f_chunk = 0, f_group += n_waves;
        }
    };
#pragma unroll
    for (int i = 0; i < SETS; ++i) fetch(fs[i]);
    for (int i = threadIdx.x; i < cols / 16; i += 64 * WAVES) reinterpret_cast<uint4 *>(aq)[i] = reinterpret_cast<const uint4 *>(act_qs)[i];
    for (int i = threadIdx.x; i < nb; i += 64 * WAVES) ad[i] = h2f(act_d[i]);
    __syncthreads();
    if (my_groups == 0) return;  // wave-uniform
    const uint8_t *my = stage + row * RS + 4 * c;
    const int8_t *my_a = aq + 4 * c;
    float acc = 0.0f;
    int group = first, chunk = 0;
    auto turn = [&](Fetch &f) {
        wave_lds_fence();  // the previous chunk has been read
#pragma unroll
        for (int i = 0; i < Fetch::kLoads; ++i) *reinterpret_cast<uint4 *>(stage + loff[i]) = f.u[i];
        wave_lds_fence();
        fetch(f);  // a later chunk, into the registers just written out
        const int b0 = chunk * KB;
        const int out_row = min(8 * group, rows - 8) + row;
        int32_t *pp = PART ? partials + (static_cast<size_t>(out_row) * nb) * 8 + c : nullptr;
        const uint8_t *row_blocks = stage + row * RS;
        auto compute_batch = [&](const Q8sBatch &bt, int s) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int p = bt.dot(i);
                if (PART) pp[(b0 + 8 * s + i) * 8] = p;
                acc = __builtin_fmaf(bt.scale(i), static_cast<float>(p), acc);
            }
        };
        // eight blocks at a time, the next eight requested from LDS before the arithmetic of these
        Q8sBatch t0, t1;
        t0.load(my, row_blocks, my_a, ad, b0, 0);
#pragma unroll
        for (int s = 0; s < KB / 8; s += 2) {
            t1.load(my, row_blocks, my_a, ad, b0, s + 1);
            __builtin_amdgcn_sched_barrier(0);
            compute_batch(t0, s);
            if (s + 2 < KB / 8) t0.load(my, row_blocks, my_a, ad, b0, s + 2);
            __builtin_amdgcn_sched_barrier(0);
            compute_batch(t1, s + 1);
        }
        if (++chunk == nchunks) {
            const float y = close_lanes8(acc);
            if (c == 0) out[out_row] = y;
            acc = 0.0f, chunk = 0, group += n_waves;
        }
    };
    for (int t = 0; t < items; t += SETS) {
#pragma unroll
        for (int i = 0; i < SETS; ++i) {
            if (t + i >= items) break;
            turn(fs[i]);
        }
    }
}

// ---- dense Q8_0 x Q8_0 GEMV, few rows: the waves of a workgroup share the eight rows of a group --------------------
// With few row groups a group's wave runs alone on its SIMD and the time is the length of its chains (about 40 cycles
// per block: one wave issues an instruction every four cycles and a block is ten of them).  Only the fma itself has to
// run in block order.  So wave v of a workgroup takes blocks [v NCH*KB, (v+1) NCH*KB) of the eight rows, requests all
// of them at once, turns them into (d_w d_a, float(dot4)) pairs in registers at its own pace, and then the waves run
// their parts of the chains one after the other, handing the 64 accumulators on through LDS: NCH*KB dependent fma per
// wave, nothing else.  Lane = 8 row + chain as in k_gemv_q8_rows8; nb = KB NCH WAVES blocks per row (KB = 16 or 32).
// dynamic LDS: cols bytes, cols/32 floats, 256 bytes of accumulators, then one stage of 8 * kQ8sRowStride<KB> per wave.
// (the body: `group` is the workgroup's group of eight rows)
template <int KB, int NCH, int WAVES, bool PART>
WD_DEV void gemv_q8_rows8_split_body(const uint8_t *__restrict__ w, int rows, int nb, const int8_t *__restrict__ act_qs,
                                     const uint16_t *__restrict__ act_d, float *__restrict__ out, int32_t *__restrict__ partials,
                                     int group) {
    constexpr int SEG = NCH * KB;
    using Fetch = Q8sFetch<KB>;
    constexpr int RS = kQ8sRowStride<KB>;
    extern __shared__ __align__(16) uint8_t q8p_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cols = nb * 32;
    int8_t *aq = reinterpret_cast<int8_t *>(q8p_lds);
    float *ad = reinterpret_cast<float *>(q8p_lds + cols);
    float *carry = reinterpret_cast<float *>(q8p_lds + cols + nb * 4);
    uint8_t *stage = q8p_lds + cols + nb * 4 + 256 + wave * (8 * RS);
    const size_t rb = static_cast<size_t>(nb) * 34;
    const int row = lane >> 3, c = lane & 7;
    // a last group of fewer than eight rows is moved up to end with the matrix (rows >= 8)
    const int base_row = min(8 * group, rows - 8);
    const uint8_t *src = uniform_ptr(w + static_cast<size_t>(base_row) * rb + static_cast<size_t>(wave) * (34 * SEG));
    uint32_t loff[Fetch::kLoads];
    Fetch f[NCH];
#pragma unroll
    for (int i = 0; i < Fetch::kLoads; ++i) {
        const int u = min(i * 64 + lane, Fetch::kWords - 1);
        const int r = u / Fetch::kWordsPerRow, within = u - r * Fetch::kWordsPerRow;
        loff[i] = static_cast<uint32_t>(r * RS + 16 * within);
        const uint32_t goff = static_cast<uint32_t>(r * rb + 16 * within);
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) f[ch].u[i] = gld_u128_aligned(src + goff + ch * (34 * KB));
    }
    for (int i = threadIdx.x; i < cols / 16; i += 64 * WAVES) reinterpret_cast<uint4 *>(aq)[i] = reinterpret_cast<const uint4 *>(act_qs)[i];
    for (int i = threadIdx.x; i < nb; i += 64 * WAVES) ad[i] = h2f(act_d[i]);
    __syncthreads();
    const uint8_t *my = stage + row * RS + 4 * c;
    const int8_t *my_a = aq + 4 * c;
    const int first_block = wave * SEG;
    int32_t *pp = PART ? partials + (static_cast<size_t>(base_row + row) * nb) * 8 + c : nullptr;
    float dv[SEG], pv[SEG];
    const uint8_t *row_blocks = stage + row * RS;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
        wave_lds_fence();  // the previous chunk has been read
#pragma unroll
        for (int i = 0; i < Fetch::kLoads; ++i) *reinterpret_cast<uint4 *>(stage + loff[i]) = f[ch].u[i];
        wave_lds_fence();
        const int b0 = first_block + ch * KB;
        auto pairs = [&](const Q8sBatch &bt, int s) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int p = bt.dot(i);
                if (PART) pp[(b0 + 8 * s + i) * 8] = p;
                dv[ch * KB + 8 * s + i] = bt.scale(i);
                pv[ch * KB + 8 * s + i] = static_cast<float>(p);
            }
        };
        Q8sBatch t0, t1;
        t0.load(my, row_blocks, my_a, ad, b0, 0);
#pragma unroll
        for (int s = 0; s < KB / 8; s += 2) {
            t1.load(my, row_blocks, my_a, ad, b0, s + 1);
            __builtin_amdgcn_sched_barrier(0);
            pairs(t0, s);
            if (s + 2 < KB / 8) t0.load(my, row_blocks, my_a, ad, b0, s + 2);
            __builtin_amdgcn_sched_barrier(0);
            pairs(t1, s + 1);
        }
    }
    // the chains, one wave after the other in block order
    float acc = 0.0f;
#pragma unroll
    for (int turn = 0; turn < WAVES; ++turn) {
        if (wave == turn) {
            if (turn > 0) acc = carry[lane];
#pragma unroll
            for (int i = 0; i < SEG; ++i) acc = __builtin_fmaf(dv[i], pv[i], acc);
            if (turn < WAVES - 1) carry[lane] = acc;
        }
        if (turn < WAVES - 1) __syncthreads();
    }
    if (wave == WAVES - 1) {
        const float y = close_lanes8(acc);
        if (c == 0) out[base_row + row] = y;
    }
}
template <int KB, int NCH, int WAVES, bool PART>
__global__ __launch_bounds__(64 * WAVES) void k_gemv_q8_rows8_split(const uint8_t *__restrict__ w, int rows, int nb,
                                                              const int8_t *__restrict__ act_qs, const uint16_t *__restrict__ act_d,
                                                              float *__restrict__ out, int32_t *__restrict__ partials) {
    gemv_q8_rows8_split_body<KB, NCH, WAVES, PART>(w, rows, nb, act_qs, act_d, out, partials, static_cast<int>(blockIdx.x));
}
// Several matrices of the same row length in ONE launch (the projections a block applies to one or a few activations:
// each of them alone is bound by its launch, not by its bytes).  Workgroup b belongs to the item whose range of row
// groups holds b; what it computes is what k_gemv_q8_rows8_split computes for that item alone.
template <int KB, int NCH, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void k_gemv_q8_rows8_split_batch(GemvBatch b, int nb) {
    const int item = gemv_batch_item(b);
    gemv_q8_rows8_split_body<KB, NCH, WAVES, false>(b.w[item], b.rows[item], nb, b.act_qs[item], b.act_d[item], b.out[item], nullptr,
                                                   static_cast<int>(blockIdx.x) - b.first_group[item]);
}

// ---- Q6_K x Q8_K GEMV: the waves of the grid take the rows in turn, pass by pass, one pass fetched ahead -------
// The activation (quants, scales, 16-value sums) is staged in LDS once per workgroup.
// dynamic LDS: kQ6ActStride bytes per super-block, then cols/256 floats, then cols/16 int16 (each part 16-byte
// aligned), then four wave stages of kQ6StageBytes.
// FULL: rows are a whole number of passes.
template <bool FULL>
struct Q6Walk {  // the passes of a wave's rows, in memory order
    const uint8_t *src;
    size_t row_skip;  // bytes from the end of one of the wave's rows to the start of its next
    int pass, npass, last_bytes;
    Q6Pieces full, last;
    WD_DEV bool is_last() const { return pass == npass - 1; }
    WD_DEV const Q6Pieces &pieces() const { return (FULL || !is_last()) ? full : last; }
    WD_DEV void advance() {
        src = uniform_ptr(src + ((FULL || !is_last()) ? 1680 : last_bytes) + (is_last() ? row_skip : 0));
        pass = is_last() ? 0 : pass + 1;
    }
};

template <bool PART, bool ALIGNED, bool FULL>
__global__ __launch_bounds__(256) void k_gemv_q6k(const uint8_t *__restrict__ w, int rows, int cols,
                                                   const int8_t *__restrict__ act_qs, const float *__restrict__ act_d,
                                                   const int16_t *__restrict__ act_bsums, float *__restrict__ out,
                                                   int32_t *__restrict__ partials) {
    extern __shared__ __align__(16) uint8_t q6_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nb = cols >> 8, npass = (nb + 7) >> 3;
    const int aq_bytes = nb * kQ6ActStride;
    int8_t *aq = reinterpret_cast<int8_t *>(q6_lds);
    float *ad = reinterpret_cast<float *>(q6_lds + aq_bytes);
    int16_t *ab = reinterpret_cast<int16_t *>(q6_lds + aq_bytes + ((nb * 4 + 15) & ~15));
    uint8_t *stage = q6_lds + aq_bytes + ((nb * 4 + 15) & ~15) + nb * 32 + wave * kQ6StageBytes;
    const size_t rb = static_cast<size_t>(nb) * 210;
    // the waves of the grid take the rows in turn, so that the waves running together read neighbouring rows
    const int n_waves = gridDim.x * 4;
    const int r0 = blockIdx.x * 4 + wave;
    const int n_rows = r0 < rows ? (rows - r0 + n_waves - 1) / n_waves : 0;
    Q6Walk<FULL> fetch;  // runs one pass ahead of `work`
    fetch.src = uniform_ptr(w + static_cast<size_t>(min(r0, rows - 1)) * rb);  // a wave without rows asks for the last one
    fetch.row_skip = static_cast<size_t>(n_waves - 1) * rb;
    fetch.pass = 0, fetch.npass = npass, fetch.last_bytes = (nb - 8 * (npass - 1)) * 210;
    fetch.full = q6k_pieces(1680, lane), fetch.last = q6k_pieces(fetch.last_bytes, lane);
    Q6Walk<FULL> work = fetch;
    Q6Fetch fa = q6k_fetch<ALIGNED>(fetch.src, fetch.pieces()), fb;
    for (int i = threadIdx.x; i < cols / 16; i += 256)  // 16 words of 16 bytes per super-block
        reinterpret_cast<uint4 *>(aq + (i >> 4) * kQ6ActStride)[i & 15] = reinterpret_cast<const uint4 *>(act_qs)[i];
    for (int i = threadIdx.x; i < nb; i += 256) ad[i] = act_d[i];
    for (int i = threadIdx.x; i < nb * 8; i += 256) reinterpret_cast<uint32_t *>(ab)[i] = reinterpret_cast<const uint32_t *>(act_bsums)[i];
    __syncthreads();
    if (n_rows <= 0) return;  // wave-uniform
    const int items = n_rows * npass;
    long long r = r0;
    float acc = 0.0f;
    auto step = [&](const Q6Fetch &cur) {
        wave_lds_fence();  // the previous pass has been read
        q6k_stage(stage, cur, work.pieces());
        wave_lds_fence();
        acc = q6k_pass<PART, FULL>(stage, 8 * work.pass, nb, aq, ad, ab, lane, acc, PART ? partials + static_cast<size_t>(r) * nb * 8 : nullptr);
        if (work.is_last()) {
            const float y = q6k_close(acc);
            if (lane == 15) out[r] = y;
            r += n_waves;
        }
        work.advance();
    };
    // Two register sets take turns, so that the request for the next pass stays in flight while this one is worked on.
    // Every turn issues its three requests (after the wave's last pass: the same pass again, not used), so that the
    // count of requests in flight does not depend on the path taken.
    for (int t = 0; t < items; t += 2) {
        if (t + 1 < items) fetch.advance();
        fb = q6k_fetch<ALIGNED>(fetch.src, fetch.pieces());
        step(fa);
        if (t + 1 >= items) break;
        if (t + 2 < items) fetch.advance();
        fa = q6k_fetch<ALIGNED>(fetch.src, fetch.pieces());
        step(fb);
    }
}

// ---- elementwise ---------------------------------------------------------------------------------
__global__ void k_silu_mul_experts(const float *__restrict__ gate_up, float *__restrict__ act, int ffn) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= ffn) return;
    const float *g = gate_up + static_cast<size_t>(2) * blockIdx.y * ffn;
    act[static_cast<size_t>(blockIdx.y) * ffn + i] = silu_ggml(g[i]) * g[ffn + i];
}

__global__ void k_weighted_accum(const float *__restrict__ experts, const float *__restrict__ weights,
                                 float *__restrict__ accum, int n, int k) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float a = accum[i];
    for (int j = 0; j < k; ++j) {
        const float prod = experts[static_cast<size_t>(j) * n + i] * weights[j];
        a = a + prod;
    }
    accum[i] = a;
}

// out may alias routed
__global__ void k_add_shared(const float *routed, const float *__restrict__ shared,
                             const float *__restrict__ gate, float *out, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float prod = shared[i] * gate[0];
    out[i] = routed[i] + prod;
}

// gate[0] = sigmoid_ggml(gate[0])
__global__ void k_sigmoid1(float *gate) {
    if (threadIdx.x == 0 && blockIdx.x == 0) gate[0] = sigmoid_ggml(gate[0]);
}

// accum[i] = ordered weighted sum of the k expert outputs (product rounded, then sum rounded);
// out[i] = accum[i] + shared[i] * gate[0] when a shared expert is present, else accum[i].
// residual (optional): residual[i] += out[i] * residual_scale.
__global__ void k_combine(const float *__restrict__ experts, const float *__restrict__ weights, int k,
                          const float *__restrict__ shared, const float *__restrict__ gate,
                          float *__restrict__ accum, float *__restrict__ out, float *__restrict__ residual,
                          float residual_scale, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float a = 0.0f;
    for (int j = 0; j < k; ++j) {
        const float prod = experts[static_cast<size_t>(j) * n + i] * weights[j];
        a = a + prod;
    }
    accum[i] = a;
    if (shared) {
        const float prod = shared[i] * gate[0];
        a = a + prod;
    }
    out[i] = a;
    if (residual) {  // next layer's input in a layer stack
        const float scaled = a * residual_scale;
        residual[i] = residual[i] + scaled;
    }
}

// Hyper-connection combine of the FFN branch: residual[c][h] += branch[h] * (2 sigmoid(inject[c] / hc)) for the hc
// residual streams, product rounded, then sum rounded (src/qwen38_hc.cuh:2530-2547).  SHARED: 0 = branch is block_out,
// 1 / 2 = branch = routed + shared * gate[0] with the shared expert's output as float / as half bits (:2241-2263).
template <int SHARED>
__global__ void k_hc_combine(float *__restrict__ residual, const float *__restrict__ block_out, const void *__restrict__ shared,
                             const float *__restrict__ gate, const float *__restrict__ inject, int hidden, int hc, int round) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden * hc) return;
    const int c = i / hidden, h = i - c * hidden;
    float branch = block_out[h];
    if (SHARED != 0) {
        const float sh = SHARED == 1 ? static_cast<const float *>(shared)[h] : h2f(static_cast<const uint16_t *>(shared)[h]);
        const float weighted = sh * gate[0];
        branch = branch + weighted;
    }
    const float weighted = branch * hc_weight(inject[c], hc);
    const float v = residual[i] + weighted;
    residual[i] = round ? round_half(v) : v;
}

}  // namespace wd
