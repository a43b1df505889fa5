// Wave-level row decoders: one (or four) weight rows in raw GGUF block bytes against a
// quantised activation, with the float accumulation order of the reference CPU path
// (src/qwen38_cpu_moe.cuh:298-440): eight chunk-lane accumulators, one fused multiply-add
// per super-block (IQ2_S/IQ3_S) or per 32-value block (Q8_0), closing tree
// ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)).  Integer sums are exact, so their order is free.
#pragma once

#include "wd_device.cuh"
#include "wd_codebooks.inc"

namespace wd {

// ---- codebooks, expanded at compile time ------------------------------------------
struct Grid3 {
    uint32_t v[512];
};
struct Grid2 {
    uint64_t v[1024];
};
struct SignMask {
    uint2 v[16];  // .x: 0xff in every byte whose sign bit is set, .y: 0x01 in the same bytes
};

constexpr Grid3 make_grid3() {
    Grid3 g{};
    const char *s = WD_IQ3S_GRID_DIGITS;
    for (int e = 0; e < 512; ++e) {
        uint32_t v = 0;
        for (int j = 0; j < 4; ++j) v |= (2u * static_cast<uint32_t>(s[e * 4 + j] - '0') + 1u) << (8 * j);
        g.v[e] = v;
    }
    return g;
}
constexpr Grid2 make_grid2() {
    Grid2 g{};
    const char *s = WD_IQ2S_GRID_DIGITS;
    for (int e = 0; e < 1024; ++e) {
        uint64_t v = 0;
        for (int j = 0; j < 8; ++j) {
            const uint64_t t = static_cast<uint64_t>(s[e * 8 + j] - '0');
            v |= (8u + 17u * t + (t == 2 ? 1u : 0u)) << (8 * j);
        }
        g.v[e] = v;
    }
    return g;
}
constexpr SignMask make_signmask() {
    SignMask m{};
    for (int s = 0; s < 16; ++s) {
        uint32_t ones = 0;
        for (int j = 0; j < 4; ++j) ones |= ((s >> j) & 1u) << (8 * j);
        m.v[s].x = ones * 0xffu;
        m.v[s].y = ones;
    }
    return m;
}

__device__ const Grid3 k_grid3 = make_grid3();
__device__ const Grid2 k_grid2 = make_grid2();
__device__ const SignMask k_signmask = make_signmask();

// LDS copies staged once per workgroup.
struct IqTables {
    uint32_t grid3[512];
    uint64_t grid2[1024];
    uint2 sign[16];
};

template <bool NEED3, bool NEED2>
WD_DEV void stage_tables(IqTables &t, int tid, int nthreads) {
    if (NEED3)
        for (int i = tid; i < 512; i += nthreads) t.grid3[i] = k_grid3.v[i];
    if (NEED2)
        for (int i = tid; i < 1024; i += nthreads) t.grid2[i] = k_grid2.v[i];
    if (tid < 16) t.sign[tid] = k_signmask.v[tid];
}

// Four codebook magnitudes with the four sign bits applied, as packed int8.
// Magnitudes are >= 1, so (m ^ 0xff) + 1 never carries out of its byte.
WD_DEV uint32_t apply_signs(uint32_t mags, uint2 sm) { return (mags ^ sm.x) + sm.y; }

// Sum over the eight lanes of a group of p[c], delivered to the lane with (lane & 7) == c.
WD_DEV int reduce_scatter8(const int (&p)[8], int lane) {
    const bool h4 = (lane & 4) != 0;
    int r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int keep = h4 ? p[j + 4] : p[j];
        const int send = h4 ? p[j] : p[j + 4];
        r[j] = keep + lane_xor(send, 4);
    }
    const bool h2 = (lane & 2) != 0;
    int s[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int keep = h2 ? r[j + 2] : r[j];
        const int send = h2 ? r[j] : r[j + 2];
        s[j] = keep + lane_xor(send, 2);
    }
    const bool h1 = (lane & 1) != 0;
    const int keep = h1 ? s[1] : s[0];
    const int send = h1 ? s[0] : s[1];
    return keep + lane_xor(send, 1);
}

// ---- IQ3_S / IQ2_S x Q8_K ------------------------------------------------------------
// Lane (sb = lane >> 3, ib = lane & 7) decodes 32-value block ib of super-block 8*pass + sb.
// chunk sums p[c] = ls * dot4(signed magnitudes of chunk c, activations 4c..4c+3 of the block).
WD_DEV void iq3s_block_chunks(const uint8_t *blk, int ib, const IqTables &t, const uint32_t (&a)[8],
                              int (&p)[8]) {
    const uint2 qs = ldu<uint2>(blk + 2 + ib * 8);
    const uint32_t qh = blk[66 + ib];
    const uint32_t sg = ldu<uint32_t>(blk + 74 + ib * 4);
    const uint32_t sc = blk[106 + (ib >> 1)];
    const int ls = 1 + 2 * static_cast<int>((sc >> (4 * (ib & 1))) & 15u);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t q = ((c < 4 ? qs.x : qs.y) >> (8 * (c & 3))) & 0xffu;
        const uint32_t idx = q | ((qh << (8 - c)) & 0x100u);
        const uint32_t sbits = (sg >> (4 * c)) & 15u;  // byte c>>1, nibble c&1
        const uint32_t w4 = apply_signs(t.grid3[idx], t.sign[sbits]);
        p[c] = ls * sdot4(w4, a[c], 0);
    }
}

WD_DEV void iq2s_block_chunks(const uint8_t *blk, int ib, const IqTables &t, const uint32_t (&a)[8],
                              int (&p)[8]) {
    const uint32_t qs = ldu<uint32_t>(blk + 2 + ib * 4);
    const uint32_t sg = ldu<uint32_t>(blk + 34 + ib * 4);
    const uint32_t qh = blk[66 + ib];
    const uint32_t sc = blk[74 + ib];
    const int ls_lo = 1 + 2 * static_cast<int>(sc & 15u);
    const int ls_hi = 1 + 2 * static_cast<int>(sc >> 4);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t idx = ((qs >> (8 * g)) & 0xffu) | ((qh << (8 - 2 * g)) & 0x300u);
        const uint64_t mags = t.grid2[idx];
        const uint32_t s8 = (sg >> (8 * g)) & 0xffu;
        const int ls = (g < 2) ? ls_lo : ls_hi;  // chunks 0..3 low nibble, 4..7 high nibble
        p[2 * g] = ls * sdot4(apply_signs(static_cast<uint32_t>(mags), t.sign[s8 & 15u]), a[2 * g], 0);
        p[2 * g + 1] = ls * sdot4(apply_signs(static_cast<uint32_t>(mags >> 32), t.sign[s8 >> 4]), a[2 * g + 1], 0);
    }
}

// One row.  act_qs / act_d: Q8_K activation (global or LDS).  Result valid in lane 0.
// `partials` (PART only): int32 [nb][8] for this row.
template <int TYPE, bool PART>
WD_DEV float iq_row_q8k(const uint8_t *row, int nb, const IqTables &t, const int8_t *act_qs, const float *act_d,
                        int lane, int32_t *partials) {
    constexpr int kBlk = (TYPE == 21) ? 110 : 82;
    const int sbl = lane >> 3, ib = lane & 7;
    float acc = 0.0f;
    for (int base = 0; base < nb; base += 8) {
        const int sb = base + sbl;
        const bool on = sb < nb;
        int p[8];
        float ds = 0.0f;
        if (on) {
            uint32_t a[8];
            const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
            const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
            a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
            const uint8_t *blk = row + static_cast<size_t>(sb) * kBlk;
            if (TYPE == 21)
                iq3s_block_chunks(blk, ib, t, a, p);
            else
                iq2s_block_chunks(blk, ib, t, a, p);
            ds = h2f(ldu<uint16_t>(blk)) * act_d[sb];
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) p[c] = 0;
        }
        const int P = reduce_scatter8(p, lane);  // lane (sbl, c): chunk c of super-block sb
        if (PART && on) partials[sb * 8 + ib] = P;
        const float pf = static_cast<float>(P);
        const int cnt = min(8, nb - base);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            if (s < cnt) {
                const float pv = lane_get(pf, s * 8 + ib);
                const float dv = lane_get(ds, s * 8 + ib);
                acc = __builtin_fmaf(dv, pv, acc);
            }
        }
    }
    float r = close_lanes8(acc);
    if (TYPE == 22) r = 0.125f * r;
    return r;
}

// ---- Q8_0 (and Q4_0 / IQ4_NL codes) x Q8_0 ------------------------------------------------
// Four rows per wave step: lane (r4 = lane >> 4, b = lane & 15) takes blocks b, b+16, ... of row r4.
// The per-block chunk sums are handed to the chain lanes through a per-wave LDS tile so that every
// chunk accumulator sees its blocks in ascending order.
struct Q8Tile {
    float pf[4 * 136];  // [r4][b][c], row stride padded to 136 floats (bank spread)
    float ds[64];       // [r4][b]
};

// kind: 0 = Q8_0 (34-byte blocks), 1 = IQ4_NL (18-byte blocks, codebook values)
template <int KIND>
WD_DEV void q8ish_block_chunks(const uint8_t *blk, const uint32_t (&a)[8], int (&p)[8]) {
    if (KIND == 0) {
        const uint4 q0 = ldu<uint4>(blk + 2);
        const uint4 q1 = ldu<uint4>(blk + 18);
        p[0] = sdot4(q0.x, a[0], 0), p[1] = sdot4(q0.y, a[1], 0), p[2] = sdot4(q0.z, a[2], 0);
        p[3] = sdot4(q0.w, a[3], 0), p[4] = sdot4(q1.x, a[4], 0), p[5] = sdot4(q1.y, a[5], 0);
        p[6] = sdot4(q1.z, a[6], 0), p[7] = sdot4(q1.w, a[7], 0);
    } else {
        // chunk l < 4: low nibbles of bytes 4l..4l+3; chunk l >= 4: high nibbles of bytes 4(l-4)..
        const uint4 n = ldu<uint4>(blk + 2);
        const uint32_t w[4] = {n.x, n.y, n.z, n.w};
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            int lo = 0, hi = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t byte = (w[l] >> (8 * j)) & 0xffu;
                constexpr int8_t lut[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
                lo += static_cast<int>(lut[byte & 15u]) * static_cast<int>(static_cast<int8_t>(a[l] >> (8 * j)));
                hi += static_cast<int>(lut[byte >> 4]) * static_cast<int>(static_cast<int8_t>(a[l + 4] >> (8 * j)));
            }
            p[l] = lo;
            p[l + 4] = hi;
        }
    }
}

// rows: pointer to the first of up to four consecutive rows (row stride = nb * block bytes);
// nrows (1..4) rows are valid.  Result for row r4 valid in lane r4*16.
// partials (PART): int32 [4][nb][8] starting at the first row.
template <int KIND, bool PART>
WD_DEV float q8_rows4(const uint8_t *rows, int nrows, int nb, const int8_t *act_qs, const uint16_t *act_d,
                      Q8Tile &tile, int lane, int32_t *partials) {
    constexpr int kBlk = (KIND == 0) ? 34 : 18;
    const int r4 = lane >> 4, b = lane & 15, c = lane & 7;
    const bool row_on = r4 < nrows;
    const uint8_t *row = rows + static_cast<size_t>(r4) * nb * kBlk;
    float acc = 0.0f;
    // IQ4_NL pairs blocks into an even and an odd accumulator and treats a trailing unpaired block
    // apart (src/qwen38_cpu_moe.cuh:377-422).
    float acc_odd = 0.0f;
    const int paired = (KIND == 1) ? (nb & ~1) : nb;
    for (int base = 0; base < nb; base += 16) {
        const int bi = base + b;
        const bool on = row_on && bi < nb;
        int p[8];
        float ds = 0.0f;
        if (on) {
            uint32_t a[8];
            const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32);
            const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32 + 16);
            a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
            const uint8_t *blk = row + static_cast<size_t>(bi) * kBlk;
            q8ish_block_chunks<KIND>(blk, a, p);
            ds = h2f(ldu<uint16_t>(blk)) * h2f(act_d[bi]);
            if (PART) {
#pragma unroll
                for (int j = 0; j < 8; ++j) partials[(static_cast<size_t>(r4) * nb + bi) * 8 + j] = p[j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) p[j] = 0;
        }
        wave_lds_fence();  // previous pass's reads are done before the tile is overwritten
        float4 *dst = reinterpret_cast<float4 *>(&tile.pf[r4 * 136 + b * 8]);
        dst[0] = make_float4(static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]),
                             static_cast<float>(p[3]));
        dst[1] = make_float4(static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]),
                             static_cast<float>(p[7]));
        tile.ds[lane] = ds;
        wave_lds_fence();
        const int cnt = min(16, nb - base);
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            if (s < cnt) {
                const float pv = tile.pf[r4 * 136 + s * 8 + c];
                const float dv = tile.ds[r4 * 16 + s];
                if (KIND == 1) {
                    const int blk_i = base + s;
                    if (blk_i < paired) {
                        if (blk_i & 1)
                            acc_odd = __builtin_fmaf(dv, pv, acc_odd);
                        else
                            acc = __builtin_fmaf(dv, pv, acc);
                    }
                } else {
                    acc = __builtin_fmaf(dv, pv, acc);
                }
            }
        }
    }
    if (KIND == 1) acc = acc + acc_odd;
    float r = close_lanes8(acc);
    if (KIND == 1 && (nb & 1)) {
        // trailing block: one rounded product with the whole-block integer sum, added after the tree.
        // The tile still holds the last pass; every chunk value is an exact integer < 2^24.
        const int s = (nb - 1) & 15;
        float tot = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) tot += tile.pf[r4 * 136 + s * 8 + j];
        r = r + tile.ds[r4 * 16 + s] * tot;
    }
    return r;
}

// ---- dense Q4_0 x Q8_0 (src/warodecode.cu:1534-1562; no canonical float order) ------------
// One row per 16 lanes, lane b takes blocks b, b+16, ...; block sums are exact, the float side is
// sum over blocks of (d_w * d_x) * (float)sumi folded with a fixed 16-lane tree.
template <bool PART>
WD_DEV float q4_0_rows4(const uint8_t *rows, int nrows, int nb, const int8_t *act_qs, const uint16_t *act_d,
                        int lane, int32_t *partials) {
    const int r4 = lane >> 4, b = lane & 15;
    const uint8_t *row = rows + static_cast<size_t>(r4) * nb * 18;
    float sumf = 0.0f;
    if (r4 < nrows) {
        for (int bi = b; bi < nb; bi += 16) {
            const uint8_t *blk = row + static_cast<size_t>(bi) * 18;
            const uint4 n = ldu<uint4>(blk + 2);
            const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32);
            const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32 + 16);
            const uint32_t w[4] = {n.x, n.y, n.z, n.w};
            const uint32_t lo_a[4] = {a0.x, a0.y, a0.z, a0.w};
            const uint32_t hi_a[4] = {a1.x, a1.y, a1.z, a1.w};
            // sum (nibble - 8) * a  =  sum nibble * a  -  8 * sum a
            int sumi = 0, asum = 0;
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                sumi = sdot4(w[l] & 0x0f0f0f0fu, lo_a[l], sumi);
                sumi = sdot4((w[l] >> 4) & 0x0f0f0f0fu, hi_a[l], sumi);
                asum = sdot4(0x01010101u, lo_a[l], asum);
                asum = sdot4(0x01010101u, hi_a[l], asum);
            }
            sumi -= 8 * asum;
            if (PART) partials[static_cast<size_t>(r4) * nb + bi] = sumi;
            sumf += h2f(ldu<uint16_t>(blk)) * h2f(act_d[bi]) * static_cast<float>(sumi);
        }
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) sumf += lane_xor(sumf, m);
    return sumf;
}

}  // namespace wd
