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
    WD_DEV uint32_t grid3_at(uint32_t idx) const { return grid3[idx]; }
    WD_DEV uint32_t grid3_bytes(uint32_t off) const { return *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint8_t *>(grid3) + off); }  // off = 4 idx
    WD_DEV uint64_t grid2_at(uint32_t idx) const { return grid2[idx]; }
    WD_DEV uint2 sign_at(uint32_t nibble) const { return sign[nibble]; }
};
// The same tables for a kernel that knows their LDS byte address when it is compiled (BASE: the address of an IqTables
// in the workgroup's LDS): a lookup's address is then the scaled index alone, the rest goes into the load's offset field.
template <unsigned BASE>
struct IqTablesAt {
    typedef const __attribute__((address_space(3))) uint32_t *Lds32;
    typedef const __attribute__((address_space(3))) uint64_t *Lds64;
    WD_DEV uint32_t grid3_at(uint32_t idx) const {
        return *(Lds32)(uintptr_t)(BASE + static_cast<unsigned>(offsetof(IqTables, grid3)) + 4u * idx);
    }
    WD_DEV uint32_t grid3_bytes(uint32_t off) const { return *(Lds32)(uintptr_t)(BASE + static_cast<unsigned>(offsetof(IqTables, grid3)) + off); }
    WD_DEV uint64_t grid2_at(uint32_t idx) const {
        return *(Lds64)(uintptr_t)(BASE + static_cast<unsigned>(offsetof(IqTables, grid2)) + 8u * idx);
    }
    WD_DEV uint2 sign_at(uint32_t nibble) const {
        const uint64_t v = *(Lds64)(uintptr_t)(BASE + static_cast<unsigned>(offsetof(IqTables, sign)) + 8u * nibble);
        return make_uint2(static_cast<uint32_t>(v), static_cast<uint32_t>(v >> 32));
    }
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

typedef unsigned wd_uint2v __attribute__((ext_vector_type(2)));

// Lane layout of the IQ decoders: lane = 8 * ib + sb (ib = 32-value block inside the super-block,
// sb = super-block of the current pass).  The eight lanes that share sb are 8 apart, so their
// chunk sums are folded with a half swap (ib bit 2), a row-pair swap (ib bit 1) and a rotate by 8
// inside the row (ib bit 0).  Returns, in lane (ib, sb), the sum over the eight ib-lanes of p[ib].
WD_DEV int reduce_scatter_ib(const int (&p)[8], int lane) {
    int q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // .x = (own low half, partner-low's p[j+4]);  .y = (partner-high's p[j], own high half)
        const wd_uint2v r = __builtin_amdgcn_permlane32_swap(static_cast<unsigned>(p[j]), static_cast<unsigned>(p[j + 4]),
                                                            false, false);
        q[j] = static_cast<int>(r.x + r.y);  // lanes < 32: chunk j, lanes >= 32: chunk j + 4
    }
    int s2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const wd_uint2v r = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(q[j]), static_cast<unsigned>(q[j + 2]),
                                                            false, false);
        s2[j] = static_cast<int>(r.x + r.y);  // even rows: q[j] family, odd rows: q[j + 2] family
    }
    const bool odd = (lane & 8) != 0;
    const int keep = odd ? s2[1] : s2[0];
    const int send = odd ? s2[0] : s2[1];
    return keep + dpp_i<kDppRor8>(0, send);
}

// ---- IQ3_S / IQ2_S x Q8_K ------------------------------------------------------------
// Lane (sb = lane >> 3, ib = lane & 7) decodes 32-value block ib of super-block 8*pass + sb.
// chunk sums p[c] = ls * dot4(signed magnitudes of chunk c, activations 4c..4c+3 of the block).
// Loading and decoding are separate steps so that a wave can put the loads of several rows in
// flight before it starts to decode the first one.
struct IqFields {
    uint2 qs;       // IQ3_S: 8 index bytes; IQ2_S: .x = 4 index bytes, .y = 4 sign bytes
    uint32_t sg;    // IQ3_S: 4 sign bytes
    uint32_t qh, sc;
    uint16_t d;
};

template <int TYPE>
WD_DEV IqFields iq_load(const uint8_t *blk, int ib) {
    IqFields f;
    if (TYPE == 21) {
        f.qs = gld_u64(blk + 2 + ib * 8);
        f.qh = gld_u8(blk + 66 + ib);
        f.sg = gld_u32(blk + 74 + ib * 4);
        f.sc = gld_u8(blk + 106 + (ib >> 1));
    } else {
        f.qs.x = gld_u32(blk + 2 + ib * 4);
        f.qs.y = gld_u32(blk + 34 + ib * 4);
        f.sg = 0;
        f.qh = gld_u8(blk + 66 + ib);
        f.sc = gld_u8(blk + 74 + ib);
    }
    f.d = gld_u16(blk);
    return f;
}

template <int TYPE, typename Tables>
WD_DEV void iq_chunks(const IqFields &f, int ib, const Tables &t, const uint32_t (&a)[8], int (&p)[8]) {
    if (TYPE == 21) {
        const int ls = 1 + 2 * static_cast<int>((f.sc >> (4 * (ib & 1))) & 15u);
        // all sixteen lookups first, the arithmetic after: a lane's block then waits for the LDS once, not eight times
        uint32_t g[8];
        uint2 sm[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            // (the entry's byte offset, 4 (q | high bit << 8), put together from parts that are one instruction each)
            const uint32_t q4 = (((c < 4 ? f.qs.x : f.qs.y) >> (8 * (c & 3))) & 0xffu) << 2;
            const uint32_t off = q4 | ((f.qh << (10 - c)) & 0x400u);
            const uint32_t sbits = (f.sg >> (4 * c)) & 15u;  // sign byte c>>1, nibble c&1
            g[c] = t.grid3_bytes(off);
            sm[c] = t.sign_at(sbits);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) p[c] = __mul24(ls, sdot4(apply_signs(g[c], sm[c]), a[c], 0));
    } else {
        const int ls_lo = 1 + 2 * static_cast<int>(f.sc & 15u);
        const int ls_hi = 1 + 2 * static_cast<int>(f.sc >> 4);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint32_t idx = ((f.qs.x >> (8 * g)) & 0xffu) | ((f.qh << (8 - 2 * g)) & 0x300u);
            const uint64_t mags = t.grid2_at(idx);
            const uint32_t s8 = (f.qs.y >> (8 * g)) & 0xffu;
            const int ls = (g < 2) ? ls_lo : ls_hi;  // chunks 0..3 low nibble, 4..7 high nibble
            p[2 * g] = __mul24(ls, sdot4(apply_signs(static_cast<uint32_t>(mags), t.sign_at(s8 & 15u)), a[2 * g], 0));
            p[2 * g + 1] = __mul24(ls, sdot4(apply_signs(static_cast<uint32_t>(mags >> 32), t.sign_at(s8 >> 4)), a[2 * g + 1], 0));
        }
    }
}

// The same in two steps, for callers that apply one decoded sub-block to several activations: the 32 signed
// weights (eight packed dwords) and the odd sub-scale of every chunk first, the chunk sums per activation after.
template <int TYPE, typename Tables>
WD_DEV void iq_decode(const IqFields &f, int ib, const Tables &t, uint32_t (&w)[8], int (&ls)[2]) {
    if (TYPE == 21) {
        ls[0] = ls[1] = 1 + 2 * static_cast<int>((f.sc >> (4 * (ib & 1))) & 15u);
        uint32_t g[8];
        uint2 sm[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t q4 = (((c < 4 ? f.qs.x : f.qs.y) >> (8 * (c & 3))) & 0xffu) << 2;
            const uint32_t off = q4 | ((f.qh << (10 - c)) & 0x400u);
            const uint32_t sbits = (f.sg >> (4 * c)) & 15u;
            g[c] = t.grid3_bytes(off);
            sm[c] = t.sign_at(sbits);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) w[c] = apply_signs(g[c], sm[c]);
    } else {
        ls[0] = 1 + 2 * static_cast<int>(f.sc & 15u);  // chunks 0..3
        ls[1] = 1 + 2 * static_cast<int>(f.sc >> 4);   // chunks 4..7
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint32_t idx = ((f.qs.x >> (8 * g)) & 0xffu) | ((f.qh << (8 - 2 * g)) & 0x300u);
            const uint64_t mags = t.grid2_at(idx);
            const uint32_t s8 = (f.qs.y >> (8 * g)) & 0xffu;
            w[2 * g] = apply_signs(static_cast<uint32_t>(mags), t.sign_at(s8 & 15u));
            w[2 * g + 1] = apply_signs(static_cast<uint32_t>(mags >> 32), t.sign_at(s8 >> 4));
        }
    }
}
WD_DEV void iq_dot_decoded(const uint32_t (&w)[8], const int (&ls)[2], const uint32_t (&a)[8], int (&p)[8]) {
    // (The sub-scales pass through a statement the compiler cannot look into.  It knows that they are small, drops
    // __mul24's sign extension of them as redundant and moves what is left out of the caller's loop - and then selects,
    // for a factor that is just some register, the full 32-bit multiply: a quarter-rate instruction, sixteen times per
    // pair of rows.  With the extension in place both factors are visibly 24 bits wide and the multiply is v_mul_i32_i24.)
    int l[2] = {ls[0], ls[1]};
    asm("" : "+v"(l[0]), "+v"(l[1]));
#pragma unroll
    for (int c = 0; c < 8; ++c) p[c] = __mul24(l[c >> 2], sdot4(w[c], a[c], 0));
}

// NR rows against one Q8_K activation (act_qs / act_d in global memory or LDS).  y[i] is uniform
// across the wave.  `partials` (PART only): int32 [nb][8] per row, rows `pstride` ints apart.
//
// Float order: chunk lane c accumulates fma(d_w * d_x, (float)sum, acc) over ascending super-blocks.
// After the integer fold, lane (c, sb) holds chunk c of super-block sb, so the eight lanes of one
// group form the chain of chunk c: the accumulator moves one lane up per step (row_shr:1) and the
// finished chain sits in the group's last lane.
struct NoPre {
    WD_DEV void operator()() const {}
};

// `pre` runs once, after the weight loads of the first pass have been issued and before the
// activation is read: the place to produce the activation (quantise into LDS, barrier) while the
// weights are in flight.
template <int TYPE, int NR, bool PART, typename Pre = NoPre>
WD_DEV void iq_rows_q8k(const uint8_t *const (&rows)[NR], int nb, const IqTables &t, const int8_t *act_qs,
                        const float *act_d, int lane, float (&y)[NR], int32_t *partials, size_t pstride,
                        Pre pre = Pre()) {
    constexpr int kBlk = (TYPE == 21) ? 110 : 82;
    const int ib = lane >> 3, sbl = lane & 7;
    const bool first = sbl == 0;
    float acc[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[i] = 0.0f;
    for (int base = 0; base < nb; base += 8) {
        const int sb = base + sbl;
        const bool on = sb < nb;
        IqFields f[NR];
        uint32_t a[8];
        float dx = 0.0f;
        if (on) {
#pragma unroll
            for (int i = 0; i < NR; ++i) f[i] = iq_load<TYPE>(rows[i] + static_cast<size_t>(sb) * kBlk, ib);
        }
        if (base == 0) pre();
        if (on) {
            const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
            const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
            a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
            dx = act_d[sb];
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            int p[8];
            float ds = 0.0f;
            if (on) {
                iq_chunks<TYPE>(f[i], ib, t, a, p);
                ds = h2f(f[i].d) * dx;
            } else {
#pragma unroll
                for (int c = 0; c < 8; ++c) p[c] = 0;
            }
            const int P = reduce_scatter_ib(p, lane);  // lane (c = ib, sb): chunk c of super-block sb
            if (PART && on) partials[i * pstride + sb * 8 + ib] = P;
            const float pf = static_cast<float>(P);
            // carry of the previous pass: last lane of the group -> first lane (lanes past the row's
            // end pass the accumulator through unchanged, fma(0, 0, acc) == acc)
            const float carry = dpp_f<kDppShl7>(0.0f, acc[i]);
            float v = __builtin_fmaf(ds, pf, base == 0 ? 0.0f : carry);
#pragma unroll
            for (int s = 1; s < 8; ++s) {
                const float up = dpp_f<kDppShr1>(0.0f, v);
                const float nxt = __builtin_fmaf(ds, pf, up);
                v = first ? v : nxt;
            }
            acc[i] = v;
        }
    }
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const float r = close_lanes8_strided(acc[i]);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}

// ---- IQ3_S / IQ2_S rows of exactly eight super-blocks, coalesced ------------------------------------------
// Such a row is 880 (IQ3_S) or 656 (IQ2_S) contiguous bytes, a whole number of 16-byte words.  When it starts on a
// 16-byte boundary the wave fetches it with one aligned 16-byte load per lane (55 or 41 lanes) instead of five
// narrow loads per lane, parks it in LDS and picks the fields of (super-block, 32-value block) from there.
// Blocks are only 2-byte aligned: fields wider than two bytes are read as aligned dwords and shifted by two bytes in
// the even super-blocks (block offset 110 sb or 82 sb is 0 mod 4 there, and every such field sits at 2 mod 4).
constexpr int kIqStageBytes = 896;  // per row, 16-byte multiple >= 880

template <int TYPE>
WD_DEV IqFields iq_fields_lds(const uint8_t *blk, int ib, int sb) {
    const uint32_t sh = (sb & 1) ? 0u : 2u;
    IqFields f;
    f.d = *reinterpret_cast<const uint16_t *>(blk);
    if (TYPE == 21) {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(blk + 2 + ib * 8 - sh);
        const uint32_t r0 = q[0], r1 = q[1], r2 = q[2];
        f.qs.x = __builtin_amdgcn_alignbyte(r1, r0, sh);
        f.qs.y = __builtin_amdgcn_alignbyte(r2, r1, sh);
        const uint32_t *g = reinterpret_cast<const uint32_t *>(blk + 74 + ib * 4 - sh);
        f.sg = __builtin_amdgcn_alignbyte(g[1], g[0], sh);
        f.qh = blk[66 + ib];
        f.sc = blk[106 + (ib >> 1)];
    } else {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(blk + 2 + ib * 4 - sh);
        f.qs.x = __builtin_amdgcn_alignbyte(q[1], q[0], sh);
        const uint32_t *g = reinterpret_cast<const uint32_t *>(blk + 34 + ib * 4 - sh);
        f.qs.y = __builtin_amdgcn_alignbyte(g[1], g[0], sh);
        f.sg = 0;
        f.qh = blk[66 + ib];
        f.sc = blk[74 + ib];
    }
    return f;
}

// iq_rows_q8k<TYPE, NR, false> for nb == 8 and 16-byte aligned rows.  stage: NR * kIqStageBytes bytes of LDS owned by
// the wave, 16-byte aligned.
// The fetch and the rest apart, for callers that put other requests in flight between the two.
template <int TYPE, int NR>
struct IqRows8Raw {
    static constexpr int kBlk = (TYPE == 21) ? 110 : 82, kWords = 8 * kBlk / 16;
    uint4 u[NR];
};
template <int TYPE, int NR>
WD_DEV IqRows8Raw<TYPE, NR> iq_rows8_coal_request(const uint8_t *const (&rows)[NR], int lane) {
    IqRows8Raw<TYPE, NR> raw;
#pragma unroll
    for (int i = 0; i < NR; ++i) raw.u[i] = gld_u128_aligned(rows[i] + 16 * min(lane, IqRows8Raw<TYPE, NR>::kWords - 1));
    return raw;
}
template <int TYPE, int NR>
WD_DEV void iq_rows8_coal_park(const IqRows8Raw<TYPE, NR> &raw, int lane, uint8_t *stage) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
        if (lane < IqRows8Raw<TYPE, NR>::kWords) reinterpret_cast<uint4 *>(stage + i * kIqStageBytes)[lane] = raw.u[i];
    wave_lds_fence();
}
// The dot products of the NR rows parked in `stage`.
// PART: the int32 chunk sums go out as well ([8 super-blocks][8 chunk lanes] per row, rows `pstride` ints apart).
//
// Lane layout (differs from iq_rows_q8k): super-block sb = (lane >> 1) & 7, 32-value block ib = 2 (lane >> 4) + (lane & 1).
// The integer fold over the eight ib-lanes is a half swap (ib bit 2), a row-pair swap (ib bit 1) and a swap of
// neighbours (ib bit 0); it leaves chunk c of super-block sb in the lane that decoded (ib = c, sb).  The eight lanes of
// one chain then sit two apart inside one row of 16 lanes, in super-block order, so a chain step is row_shr:2 in place:
// the first lane of a chain has no source there and reads zero, which makes its fma the chain's first term again -
// no lane has to be excluded from a step - and the finished chains sit in lanes 14, 15 of every row, where two swaps
// and one shifted add form ggml's closing tree.
WD_DEV int reduce_scatter_ib_pairs(const int (&p)[8], int lane) {
    int q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const wd_uint2v r = __builtin_amdgcn_permlane32_swap(static_cast<unsigned>(p[j]), static_cast<unsigned>(p[j + 4]),
                                                            false, false);
        q[j] = static_cast<int>(r.x + r.y);  // lanes < 32: chunk j, lanes >= 32: chunk j + 4
    }
    int s2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const wd_uint2v r = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(q[j]), static_cast<unsigned>(q[j + 2]),
                                                            false, false);
        s2[j] = static_cast<int>(r.x + r.y);  // even rows: q[j] family, odd rows: q[j + 2] family
    }
    const bool odd = (lane & 1) != 0;
    const int keep = odd ? s2[1] : s2[0];
    const int send = odd ? s2[0] : s2[1];
    return keep + dpp_i<kDppXor1>(0, send);
}
// ((l0 + l4) + (l2 + l6)) + ((l1 + l5) + (l3 + l7)) with chain c in lane 16 (c >> 1) + 14 + (c & 1); uniform result.
WD_DEV float close_chains_pairs(float v) {
    const wd_uint2v h = __builtin_amdgcn_permlane32_swap(f_bits(v), f_bits(v), false, false);
    const float a = bits_f(h.x) + bits_f(h.y);  // lanes 14, 15, 30, 31: l0 + l4, l1 + l5, l2 + l6, l3 + l7
    const wd_uint2v w = __builtin_amdgcn_permlane16_swap(f_bits(a), f_bits(a), false, false);
    const float b = bits_f(w.x) + bits_f(w.y);  // lane 14: (l0 + l4) + (l2 + l6), lane 15: (l1 + l5) + (l3 + l7)
    const float c = b + dpp_f<kDppShr1>(0.0f, b);
    return readlane_f(c, 15);
}
template <int TYPE, int NR, bool PART = false, typename Tables = IqTables>
WD_DEV void iq_rows8_coal_dots(const Tables &t, const int8_t *act_qs, const float *act_d, int lane, float (&y)[NR],
                               const uint8_t *stage, int32_t *partials = nullptr, size_t pstride = 0) {
    constexpr int kBlk = IqRows8Raw<TYPE, NR>::kBlk;
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
    const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
    const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float dx = act_d[sb];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const IqFields f = iq_fields_lds<TYPE>(stage + i * kIqStageBytes + sb * kBlk, ib, sb);
        int p[8];
        iq_chunks<TYPE>(f, ib, t, a, p);
        const float ds = h2f(f.d) * dx;
        const int P = reduce_scatter_ib_pairs(p, lane);  // lane (c = ib, sb): chunk c of super-block sb
        if (PART) partials[i * pstride + sb * 8 + ib] = P;
        const float pf = static_cast<float>(P);
        float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
        for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
        const float r = close_chains_pairs(v);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}
// iq_rows8_coal_dots in two steps, for a caller that has the rows long before it has the activation: the decode (fields
// from the stage, codebook and sign lookups, signs applied: no activation needed) leaves each lane's 32 signed weights,
// its sub-scales and the super-block's scale in registers; the dots, the integer fold and the float chains follow when
// the activation is there.  The same arithmetic in the same order: the same bits.
template <int NR>
struct IqRows8Decoded {
    uint32_t w[NR][8];
    int ls[NR][2];
    uint32_t d[NR];  // f16 bits
};
template <int TYPE, int NR, typename Tables>
WD_DEV void iq_rows8_coal_decode(const Tables &t, int lane, const uint8_t *stage, IqRows8Decoded<NR> &dec) {
    constexpr int kBlk = IqRows8Raw<TYPE, NR>::kBlk;
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const IqFields f = iq_fields_lds<TYPE>(stage + i * kIqStageBytes + sb * kBlk, ib, sb);
        iq_decode<TYPE>(f, ib, t, dec.w[i], dec.ls[i]);
        dec.d[i] = f.d;
    }
}
template <int TYPE, int NR>
WD_DEV void iq_rows8_decoded_dots(const IqRows8Decoded<NR> &dec, const int8_t *act_qs, const float *act_d, int lane, float (&y)[NR]) {
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
    const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
    const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float dx = act_d[sb];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        int p[8];
        iq_dot_decoded(dec.w[i], dec.ls[i], a, p);
        const float ds = h2f(static_cast<uint16_t>(dec.d[i])) * dx;
        const int P = reduce_scatter_ib_pairs(p, lane);
        const float pf = static_cast<float>(P);
        float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
        for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
        const float r = close_chains_pairs(v);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}
// Two parked rows of which the first has been decoded ahead (iq_rows8_coal_decode with NR = 1) and the second is decoded
// here: what a caller does whose idle time before the activation arrives is worth one row's decode, not two.
template <int TYPE, typename Tables>
WD_DEV void iq_rows8_half_decoded_dots(const IqRows8Decoded<1> &dec, const Tables &t, const int8_t *act_qs, const float *act_d, int lane,
                                       float (&y)[2], const uint8_t *stage) {
    constexpr int kBlk = IqRows8Raw<TYPE, 2>::kBlk;
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
    const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
    const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float dx = act_d[sb];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        int p[8];
        float ds;
        if (i == 0) {
            iq_dot_decoded(dec.w[0], dec.ls[0], a, p);
            ds = h2f(static_cast<uint16_t>(dec.d[0])) * dx;
        } else {
            const IqFields f = iq_fields_lds<TYPE>(stage + kIqStageBytes + sb * kBlk, ib, sb);
            iq_chunks<TYPE>(f, ib, t, a, p);
            ds = h2f(f.d) * dx;
        }
        const int P = reduce_scatter_ib_pairs(p, lane);
        const float pf = static_cast<float>(P);
        float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
        for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
        const float r = close_chains_pairs(v);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}
// The second of a caller's two rows decoded long before the first: its sixteen-byte words are parked in `keep` (2048 bytes
// of LDS that belong to the wave until the dot products), decoded from there, and the 32 signed weights of every lane
// written back over them - nothing needs the parked words any more once every lane has read its fields (a wave's LDS
// operations complete in order), and a lane reads back only what it wrote itself.  What stays in registers are the
// sub-scales and the super-block's scale.
struct IqRowKept {
    int ls[2];
    uint32_t d;  // f16 bits
};
template <int TYPE, typename Tables>
WD_DEV void iq_row8_coal_decode_kept(const uint4 &words, const Tables &t, int lane, uint8_t *keep, IqRowKept &row) {
    constexpr int kBlk = IqRows8Raw<TYPE, 1>::kBlk;
    if (lane < IqRows8Raw<TYPE, 1>::kWords) reinterpret_cast<uint4 *>(keep)[lane] = words;
    wave_lds_fence();
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
    uint32_t w[8];
    const IqFields f = iq_fields_lds<TYPE>(keep + sb * kBlk, ib, sb);
    iq_decode<TYPE>(f, ib, t, w, row.ls);
    row.d = f.d;
    asm volatile("" ::: "memory");  // (the stores below stay behind every read above)
    uint4 *const out = reinterpret_cast<uint4 *>(keep);
    out[lane] = make_uint4(w[0], w[1], w[2], w[3]);
    out[64 + lane] = make_uint4(w[4], w[5], w[6], w[7]);
}
// The dot products of two rows decoded ahead: the first in registers (iq_rows8_coal_decode with NR = 1), the second kept
// in LDS (iq_row8_coal_decode_kept).  The arithmetic of iq_rows8_coal_dots in the same order.
template <int TYPE>
WD_DEV void iq_rows8_kept_decoded_dots(const IqRows8Decoded<1> &dec, const IqRowKept &row, const uint8_t *keep, const int8_t *act_qs,
                                       const float *act_d, int lane, float (&y)[2]) {
    const int ib = ((lane >> 4) << 1) | (lane & 1), sb = (lane >> 1) & 7;
    const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
    const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
    const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float dx = act_d[sb];
    const uint4 w0 = reinterpret_cast<const uint4 *>(keep)[lane], w1 = reinterpret_cast<const uint4 *>(keep)[64 + lane];
    const uint32_t w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        int p[8];
        if (i == 0) iq_dot_decoded(dec.w[0], dec.ls[0], a, p);
        else iq_dot_decoded(w, row.ls, a, p);
        const float ds = h2f(static_cast<uint16_t>(i == 0 ? dec.d[0] : row.d)) * dx;
        const int P = reduce_scatter_ib_pairs(p, lane);
        const float pf = static_cast<float>(P);
        float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
        for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
        const float r = close_chains_pairs(v);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}
template <int TYPE, int NR, bool PART = false>
WD_DEV void iq_rows8_coal_finish(const IqRows8Raw<TYPE, NR> &raw, const IqTables &t, const int8_t *act_qs, const float *act_d,
                                 int lane, float (&y)[NR], uint8_t *stage, int32_t *partials = nullptr, size_t pstride = 0) {
    iq_rows8_coal_park<TYPE, NR>(raw, lane, stage);
    iq_rows8_coal_dots<TYPE, NR, PART>(t, act_qs, act_d, lane, y, stage, partials, pstride);
}
template <int TYPE, int NR, bool PART = false>
WD_DEV void iq_rows8_coal(const uint8_t *const (&rows)[NR], const IqTables &t, const int8_t *act_qs, const float *act_d,
                          int lane, float (&y)[NR], uint8_t *stage, int32_t *partials = nullptr, size_t pstride = 0) {
    const IqRows8Raw<TYPE, NR> raw = iq_rows8_coal_request<TYPE, NR>(rows, lane);
    iq_rows8_coal_finish<TYPE, NR, PART>(raw, t, act_qs, act_d, lane, y, stage, partials, pstride);
}

constexpr int kIqStage10Bytes = 1120;  // per row of ten super-blocks: the 70 words that cover 12 + 1100 bytes
// The aligned fetch of one IQ row of NB = 8 or 10 super-blocks as a request and a store apart (for callers that keep a
// row in flight while they work on another): the 16-byte words that cover the row (it is 16-byte aligned for NB = 8 and
// 4-byte aligned for NB = 10), copied to a stage of kIqStageBytes / kIqStage10Bytes; the row then starts `lead` bytes
// into the stage.
template <int TYPE, int NB>
struct IqRowFetch {
    static constexpr int kBlk = (TYPE == 21) ? 110 : 82, kRow = NB * kBlk;
    static constexpr bool kTwoLoads = 12 + kRow > 1024;
    uint4 r0, r1;
    uint32_t lead;
    int words;
    WD_DEV void request(const uint8_t *row, int lane) {
        lead = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row)) & 15u;  // the same in every lane
        words = static_cast<int>((lead + kRow + 15) >> 4);
        const uint8_t *base = row - lead;
        r0 = gld_u128_aligned(base + 16 * min(lane, words - 1));
        if (kTwoLoads) r1 = gld_u128_aligned(base + 16 * min(64 + lane, words - 1));
    }
    WD_DEV void store(uint8_t *stage, int lane) const {  // lanes past the last word repeat it
        uint4 *st = reinterpret_cast<uint4 *>(stage);
        st[min(lane, words - 1)] = r0;
        if (kTwoLoads) st[min(64 + lane, words - 1)] = r1;
    }
};

// iq_rows_q8k<TYPE, NR, false> for nb == 10 (hidden 2560) with the aligned fetch.  A row of ten super-blocks is 1100
// or 820 bytes: 4-byte but not 16-byte aligned, so the wave fetches the 16-byte words that cover it (at most 70) and
// the fields are picked behind the row's offset in its first word.
// Lane layout as in iq_rows8_coal_dots (ib = 2 (lane >> 4) + (lane & 1), the other three lane bits a position 0..7
// inside the chain): one pass per row over super-blocks 0..7, then ONE pass for super-blocks 8 and 9 of all NR rows
// together - position 2 i takes super-block 8 of row i, position 2 i + 1 super-block 9 - instead of a mostly idle
// second pass per row.  The chain of row i continues there: its value moves from the main pass's last position to
// position 2 i (a row shift), two more steps follow, and the result moves back to the last position for the closing tree.
// rows[i]: 4-byte aligned, inside a tensor whose end is 16-byte aligned.  stage: NR * kIqStage10Bytes bytes of LDS
// owned by the wave, 16-byte aligned.  NR <= 4.
template <int TYPE, int NR, bool PART = false>
WD_DEV void iq_rows10_coal(const uint8_t *const (&rows)[NR], const IqTables &t, const int8_t *act_qs, const float *act_d,
                           int lane, float (&y)[NR], uint8_t *stage, int32_t *partials = nullptr, size_t pstride = 0) {
    static_assert(NR >= 1 && NR <= 4, "the tails of the rows share one pass of eight positions");
    constexpr int kBlk = (TYPE == 21) ? 110 : 82, kRow = 10 * kBlk;
    constexpr bool kTwoLoads = 12 + kRow > 1024;
    const int ib = ((lane >> 4) << 1) | (lane & 1), pos = (lane >> 1) & 7;
    uint32_t lead[NR];
    {
        uint4 raw0[NR], raw1[NR];
        int words[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            lead[i] = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(rows[i])) & 15u;  // the same in every lane
            words[i] = static_cast<int>((lead[i] + kRow + 15) >> 4);
            const uint8_t *base = rows[i] - lead[i];
            raw0[i] = gld_u128_aligned(base + 16 * min(lane, words[i] - 1));
            if (kTwoLoads) raw1[i] = gld_u128_aligned(base + 16 * min(64 + lane, words[i] - 1));
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) {  // lanes past the last word repeat it
            uint4 *st = reinterpret_cast<uint4 *>(stage + i * kIqStage10Bytes);
            st[min(lane, words[i] - 1)] = raw0[i];
            if (kTwoLoads) st[min(64 + lane, words[i] - 1)] = raw1[i];
        }
    }
    wave_lds_fence();
    float acc[NR];
    {   // super-blocks 0..7 of every row
        const int sb = pos;
        const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
        const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
        const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float dx = act_d[sb];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const IqFields f = iq_fields_lds<TYPE>(stage + i * kIqStage10Bytes + lead[i] + sb * kBlk, ib, sb);
            int p[8];
            iq_chunks<TYPE>(f, ib, t, a, p);
            const float ds = h2f(f.d) * dx;
            const int P = reduce_scatter_ib_pairs(p, lane);  // lane (c = ib, sb): chunk c of super-block sb
            if (PART) partials[i * pstride + sb * 8 + ib] = P;
            const float pf = static_cast<float>(P);
            float v = __builtin_fmaf(ds, pf, 0.0f);
#pragma unroll
            for (int s = 1; s < 8; ++s) v = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v));
            acc[i] = v;  // the chain over super-blocks 0..7: valid at position 7
        }
    }
    {   // super-blocks 8 and 9 of all rows in one pass
        const int ri = min(pos >> 1, NR - 1), sb = 8 + (pos & 1);
        const bool on = pos < 2 * NR;
        const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32);
        const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + sb * 256 + ib * 32 + 16);
        const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float dx = act_d[sb];
        uint32_t my_lead = lead[0];
#pragma unroll
        for (int i = 1; i < NR; ++i) my_lead = (ri == i) ? lead[i] : my_lead;
        const IqFields f = iq_fields_lds<TYPE>(stage + ri * kIqStage10Bytes + my_lead + sb * kBlk, ib, sb);
        int p[8];
        iq_chunks<TYPE>(f, ib, t, a, p);
        const float ds = on ? h2f(f.d) * dx : 0.0f;
        const int P = reduce_scatter_ib_pairs(p, lane);
        if (PART && on) partials[ri * pstride + sb * 8 + ib] = P;
        const float pf = on ? static_cast<float>(P) : 0.0f;
        // the chain value of row i, from position 7 of its own pass to position 2 i of this one (row_shl by 14 - 4 i lanes;
        // only the four lanes of positions 2 i and 2 i + 1 are written, and of these only position 2 i has a source)
        float carry = 0.0f;
        if (NR > 0) carry = dpp_f<0x10E, 0xf, 0x1>(carry, acc[0]);
        if (NR > 1) carry = dpp_f<0x10A, 0xf, 0x2>(carry, acc[NR > 1 ? 1 : 0]);
        if (NR > 2) carry = dpp_f<0x106, 0xf, 0x4>(carry, acc[NR > 2 ? 2 : 0]);
        if (NR > 3) carry = dpp_f<0x102, 0xf, 0x8>(carry, acc[NR > 3 ? 3 : 0]);
        const float v8 = __builtin_fmaf(ds, pf, carry);                       // valid at the even positions
        const float v9 = __builtin_fmaf(ds, pf, dpp_f<kDppShr2, 0xf, 0xf, true>(0.0f, v8));  // valid at the odd ones
        // back to position 7 for the closing tree: row_shr by 12 - 4 i lanes
        if (NR > 0) acc[0] = dpp_f<0x11C>(0.0f, v9);
        if (NR > 1) acc[NR > 1 ? 1 : 0] = dpp_f<0x118>(0.0f, v9);
        if (NR > 2) acc[NR > 2 ? 2 : 0] = dpp_f<0x114>(0.0f, v9);
        // (NR == 4: row 3's result is already at position 7)
        if (NR > 3) acc[NR > 3 ? 3 : 0] = v9;
    }
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const float r = close_chains_pairs(acc[i]);
        y[i] = (TYPE == 22) ? 0.125f * r : r;
    }
}

template <int TYPE, bool PART>
WD_DEV float iq_row_q8k(const uint8_t *row, int nb, const IqTables &t, const int8_t *act_qs, const float *act_d,
                        int lane, int32_t *partials) {
    const uint8_t *const rows[1] = {row};
    float y[1];
    iq_rows_q8k<TYPE, 1, PART, NoPre>(rows, nb, t, act_qs, act_d, lane, y, partials, 0);
    return y[0];
}

// ---- Q6_K x Q8_K (the output head) --------------------------------------------------------------------
// src/lowbit.cuh:2510-2612.  A super-block is 210 bytes: ql[128] (low four bits of the codes), qh[64] (high two bits),
// sixteen int8 scales, fp16 d.  Value 128 h + 32 s + l (h = half, s = 0..3, l = 0..31) has the code
// (ql[64 h + 32 (s & 1) + l] low nibble for s < 2, high nibble otherwise) | ((qh[32 h + l] >> 2 s) & 3) << 4 and the scale
// 2 (4 h + s) + (l >> 4).  The reference keeps eight float lanes per row (lane m = bytes 4m..4m+3 of every 32-value
// chunk): the integer lane sum of a super-block is sum over chunks of scale * dot4, minus the -32 correction
// (bsums[2m] scale[2m] + bsums[2m+1] scale[2m+1]) << 5, then one fma(d_w d_x, float(sum), acc_m) per super-block.
//
// Lane layout: lane = 16 (j >> 1) + 2 sb + (j & 1) with j = 4 h + q (q = 0..3) and sb = 0..7; the lane works on
// super-block 8 * pass + sb and takes bytes 8q..8q+7 of the three 32-byte runs of half h (two of ql, one of qh): these
// hold bytes 8q..8q+7 of all four chunks of the half, that is float lanes 2q and 2q+1, with compile-time shifts.
// v_permlane32_swap joins the two halves (lane and lane + 32 differ in h only) so that lanes 0..31 hold lane sum 2q
// and lanes 32..63 lane sum 2q+1: lane (j, sb) carries float lane m = 2q + h.  The eight super-blocks of a chain sit
// two lanes apart inside one 16-lane row, so the fma chain is DPP row_shr:2, the two chains of a row start in its
// lanes 0 and 1 (where row_shr:2 has no source and leaves the carry in place), and the carry between passes is
// row_shl:14.
// A pass (eight super-blocks, 1680 bytes) is fetched with two 16-byte loads per lane and copied to LDS as it lies in
// memory; blocks are only 2-byte aligned there, so the 8-byte fields are read as three aligned dwords and shifted by two
// bytes in the odd super-blocks.
constexpr int kQ6StageBytes = 1696;
// The activation's quants lie in LDS with 288 bytes per super-block: the eight super-blocks that the lanes of a wave
// read together then fall into different banks (at 256 bytes they would all share one).
constexpr int kQ6ActStride = 288;

struct Q6Fetch {
    uint4 u0, u1;
    uint32_t t16;
};
// Where a lane's pieces of a pass of `bytes` (a multiple of 210, at most 1680) lie, relative to the pass: two 16-byte
// words (at least 13 exist; lanes past the end repeat the last one) and a 2-byte piece of the tail.
struct Q6Pieces {
    uint32_t off0, off1, off_tail;
    bool has_tail;  // false: the pass is a whole number of 16-byte words (off_tail is 0 then, and its piece is not kept)
};
WD_DEV Q6Pieces q6k_pieces(int bytes, int lane) {
    const int words = bytes >> 4, tail = (bytes & 15) >> 1;
    Q6Pieces p;
    p.off0 = 16 * min(lane, words - 1), p.off1 = 16 * min(lane + 64, words - 1);
    p.has_tail = tail != 0;
    p.off_tail = tail ? 16 * words + 2 * min(lane, tail - 1) : 0;
    return p;
}
template <bool ALIGNED>
WD_DEV Q6Fetch q6k_fetch(const uint8_t *src, const Q6Pieces &p) {
    Q6Fetch f;
    f.u0 = ALIGNED ? gld_u128_aligned(src + p.off0) : gld_u128(src + p.off0);
    f.u1 = ALIGNED ? gld_u128_aligned(src + p.off1) : gld_u128(src + p.off1);
    f.t16 = gld_u16(src + p.off_tail);  // always three requests, so that the number in flight is known
    return f;
}
WD_DEV void q6k_stage(uint8_t *stage, const Q6Fetch &f, const Q6Pieces &p) {
    *reinterpret_cast<uint4 *>(stage + p.off0) = f.u0;
    *reinterpret_cast<uint4 *>(stage + p.off1) = f.u1;
    if (p.has_tail) *reinterpret_cast<uint16_t *>(stage + p.off_tail) = static_cast<uint16_t>(f.t16);
}
// Eight bytes of LDS at p = q + sh, q on a 4-byte boundary and sh = 0 or 2 (per lane).
WD_DEV uint2 lds_u64_shifted(const uint8_t *q, uint32_t sh) {
    const uint32_t *w = reinterpret_cast<const uint32_t *>(q);
    const uint32_t w0 = w[0], w1 = w[1], w2 = w[2];
    return make_uint2(__builtin_amdgcn_alignbyte(w1, w0, sh), __builtin_amdgcn_alignbyte(w2, w1, sh));
}
WD_DEV uint32_t lds_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// One pass of a row from the staged bytes (act_qs: LDS, kQ6ActStride bytes per super-block): returns the running float
// lane after super-blocks base .. base + 7.  acc: the lane's value after the previous pass (any value for base == 0).
// FULL: the row is a whole number of passes (every lane has a super-block).
template <bool PART, bool FULL>
WD_DEV float q6k_pass(const uint8_t *stage, int base, int nb, const int8_t *act_qs, const float *act_d, const int16_t *act_bsums,
                      int lane, float acc, int32_t *partials) {
    const int j = ((lane >> 4) << 1) | (lane & 1), sbl = (lane >> 1) & 7, half = j >> 2, q = j & 3;
    const int m = 2 * q + half;  // the float lane this lane carries once the halves are joined
    const int sb = base + sbl;
    const bool on = FULL || sb < nb;
    const int sbc = FULL ? sb : min(sb, nb - 1);  // lanes past the row's end read in-bounds data and contribute zero
    const uint8_t *blk = stage + 210 * sbl;
    const uint32_t sh = (sbl & 1) ? 2u : 0u;  // 210 * sbl is 2 (mod 4) in the odd super-blocks of a pass
    const uint8_t *fld = blk - sh + 64 * half + 8 * q;
    const uint2 l0 = lds_u64_shifted(fld, sh), l1 = lds_u64_shifted(fld + 32, sh);
    const uint2 hh = lds_u64_shifted(fld + 128 - 32 * half, sh);
    const int8_t *scq = reinterpret_cast<const int8_t *>(blk + 192) + 8 * half + (q >> 1);
    const int s0 = scq[0], s1 = scq[2], s2 = scq[4], s3 = scq[6];
    const uint2 *ap = reinterpret_cast<const uint2 *>(act_qs + sbc * kQ6ActStride + half * 128 + 8 * q);
    const uint2 a0 = ap[0], a1 = ap[4], a2 = ap[8], a3 = ap[12];
    constexpr uint32_t kLo = 0x0f0f0f0fu, kHi = 0x30303030u;
    int h0, h1;
    h0 = __mul24(s0, sdot4((l0.x & kLo) | ((hh.x << 4) & kHi), a0.x, 0));
    h1 = __mul24(s0, sdot4((l0.y & kLo) | ((hh.y << 4) & kHi), a0.y, 0));
    h0 += __mul24(s1, sdot4((l1.x & kLo) | ((hh.x << 2) & kHi), a1.x, 0));
    h1 += __mul24(s1, sdot4((l1.y & kLo) | ((hh.y << 2) & kHi), a1.y, 0));
    h0 += __mul24(s2, sdot4(((l0.x >> 4) & kLo) | (hh.x & kHi), a2.x, 0));
    h1 += __mul24(s2, sdot4(((l0.y >> 4) & kLo) | (hh.y & kHi), a2.y, 0));
    h0 += __mul24(s3, sdot4(((l1.x >> 4) & kLo) | ((hh.x >> 2) & kHi), a3.x, 0));
    h1 += __mul24(s3, sdot4(((l1.y >> 4) & kLo) | ((hh.y >> 2) & kHi), a3.y, 0));
    // lanes 0..31 (half 0) take both halves' sum of float lane 2q, lanes 32..63 that of 2q + 1
    const auto sw = __builtin_amdgcn_permlane32_swap(static_cast<uint32_t>(h0), static_cast<uint32_t>(h1), false, false);
    int lane_sum = static_cast<int>(sw[0] + sw[1]);
    const uint32_t pair = lds_u16(blk + 192 + 2 * m);
    const uint32_t bs = *reinterpret_cast<const uint32_t *>(act_bsums + sbc * 16 + 2 * m);
    const int c0 = static_cast<int8_t>(pair & 0xffu), c1 = static_cast<int8_t>(pair >> 8);
    const int b0 = static_cast<int16_t>(bs & 0xffffu), b1 = static_cast<int16_t>(bs >> 16);
    lane_sum -= static_cast<int>(static_cast<uint32_t>(b0 * c0 + b1 * c1) << 5);
    if (PART && on) partials[sb * 8 + m] = lane_sum;
    const float pf = on ? static_cast<float>(lane_sum) : 0.0f;
    const float ds = on ? h2f(static_cast<uint16_t>(lds_u16(blk + 208))) * act_d[sbc] : 0.0f;
    // `up` is the chain value of the super-block before the lane's own.  The chains start in lanes 0 and 1 of every row
    // with the carry of the previous pass (row_shl:14 reaches their last lanes); row_shr:2 has no source there, so it
    // leaves the carry in place while the other lanes converge one super-block per step.  Lanes past the row's end pass
    // the value through unchanged, fma(0, 0, up) == up.
    float up = dpp_f<kDppShl14>(0.0f, acc);
    up = base == 0 ? 0.0f : up;
    float v = __builtin_fmaf(ds, pf, up);
#pragma unroll
    for (int s = 1; s < 8; ++s) {
        up = dpp_f<kDppShr2>(up, v);
        v = __builtin_fmaf(ds, pf, up);
    }
    return v;
}

// ggml's closing tree over the eight float lanes, ((m0+m4)+(m2+m6)) + ((m1+m5)+(m3+m7)); float lane m = 2q + h ends in
// lane 16 (2 h + (q >> 1)) + 14 + (q & 1): m0 m2 in lanes 14 15, m4 m6 in 30 31, m1 m3 in 46 47, m5 m7 in 62 63.
// Swapping 16-lane rows adds m0+m4 | m2+m6 (lanes 14 15) and m1+m5 | m3+m7 (lanes 46 47), row_shr:1 adds the
// neighbours, swapping the wave's halves adds the two sides.  The result is valid in lane 15.
WD_DEV float q6k_close(float v) {
    const uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto rows = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    const float s = __builtin_bit_cast(float, static_cast<uint32_t>(rows[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(rows[1]));
    const float t = dpp_f<kDppShr1>(0.0f, s) + s;
    const uint32_t y = __builtin_bit_cast(uint32_t, t);
    const auto halves = __builtin_amdgcn_permlane32_swap(y, y, false, false);
    return __builtin_bit_cast(float, static_cast<uint32_t>(halves[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(halves[1]));
}

// ---- Q8_0 (and Q4_0 / IQ4_NL codes) x Q8_0 ------------------------------------------------
// Four rows per wave step: lane (r4 = lane >> 4, b = lane & 15) takes blocks b, b+16, ... of row r4.
// The per-block chunk sums are handed to the chain lanes through a per-wave LDS tile so that every
// chunk accumulator sees its blocks in ascending order.
template <int CH>
struct Q8TileN {
    float pf[CH][4 * 136];  // [pass][r4][b][c], row stride padded to 136 floats (bank spread)
    float ds[CH][64];       // [pass][r4][b]
};
using Q8Tile = Q8TileN<1>;

// kind: 0 = Q8_0 (34-byte blocks), 1 = IQ4_NL (18-byte blocks, codebook values)
struct Q8Block {
    uint4 q0, q1;  // Q8_0: 32 quants; IQ4_NL: q0 = 16 nibble bytes
    uint16_t d;
};

template <int KIND>
WD_DEV Q8Block q8_load(const uint8_t *blk) {
    Q8Block w;
    w.q0 = gld_u128(blk + 2);
    if (KIND == 0) w.q1 = gld_u128(blk + 18);
    w.d = gld_u16(blk);
    return w;
}

// The IQ4_NL codebook values of four 4-bit codes (one per byte of idx, each 0..15) as four int8: the 16 values are four
// dwords, v_perm_b32 picks among eight bytes, so the codes' low three bits select in both halves of the table and
// bit 3 chooses the half (src/lowbit.cuh:1648-1668 reads kvalues_iq4nl[code]).
WD_DEV uint32_t iq4nl_values(uint32_t idx) {
    // {-127, -104, -83, -65}, {-49, -35, -22, -10}, {1, 13, 25, 38}, {53, 69, 89, 113}
    constexpr uint32_t t0 = 0xbfad9881u, t1 = 0xf6eaddcfu, t2 = 0x26190d01u, t3 = 0x71594535u;
    const uint32_t sel = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t upper = ((idx >> 3) & 0x01010101u) * 0xffu;  // 0xff in the bytes whose code is 8..15
    return (hi & upper) | (lo & ~upper);
}

template <int KIND>
WD_DEV void q8_chunks(const Q8Block &w, const uint32_t (&a)[8], int (&p)[8]) {
    if (KIND == 0) {
        p[0] = sdot4(w.q0.x, a[0], 0), p[1] = sdot4(w.q0.y, a[1], 0), p[2] = sdot4(w.q0.z, a[2], 0);
        p[3] = sdot4(w.q0.w, a[3], 0), p[4] = sdot4(w.q1.x, a[4], 0), p[5] = sdot4(w.q1.y, a[5], 0);
        p[6] = sdot4(w.q1.z, a[6], 0), p[7] = sdot4(w.q1.w, a[7], 0);
    } else {
        // chunk l < 4: low nibbles of bytes 4l..4l+3; chunk l >= 4: high nibbles of bytes 4(l-4)..
        const uint32_t n[4] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w};
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            p[l] = sdot4(iq4nl_values(n[l] & 0x0f0f0f0fu), a[l], 0);
            p[l + 4] = sdot4(iq4nl_values((n[l] >> 4) & 0x0f0f0f0fu), a[l + 4], 0);
        }
    }
}

// NM matrices, the same four consecutive rows of each (row stride = nb * block bytes), against one
// Q8_0 activation.  rows[i]: first of the (up to) four rows of matrix i; nrows (0..4) rows are valid.
// y[i] for row r4 valid in lane r4*16.  CH passes (16 blocks per row each) of every matrix are
// loaded before the first one is decoded, and their chunk sums go through the tile together, so a
// row of up to 16*CH blocks needs one hand-off.
// partials (PART): int32 [4][nb][8] per matrix, matrices `pstride` ints apart.
template <int KIND, int NM, int CH, bool PART, typename Pre = NoPre>
WD_DEV void q8_rows4_multi(const uint8_t *const (&rows)[NM], int nrows, int nb, const int8_t *act_qs,
                           const uint16_t *act_d, Q8TileN<CH> &tile, int lane, float (&y)[NM], int32_t *partials,
                           size_t pstride, Pre pre = Pre()) {
    constexpr int kBlk = (KIND == 0) ? 34 : 18;
    const int r4 = lane >> 4, b = lane & 15, c = lane & 7;
    const bool row_on = r4 < nrows;
    const size_t row_off = static_cast<size_t>(r4) * nb * kBlk;
    // IQ4_NL pairs blocks into an even and an odd accumulator and treats a trailing unpaired block
    // apart (src/qwen38_cpu_moe.cuh:377-422).
    float acc[NM], acc_odd[NM], tail[NM];
#pragma unroll
    for (int i = 0; i < NM; ++i) acc[i] = acc_odd[i] = tail[i] = 0.0f;
    const int paired = (KIND == 1) ? (nb & ~1) : nb;
    for (int base0 = 0; base0 < nb; base0 += 16 * CH) {
        Q8Block wb[NM][CH];
        uint4 a0[CH], a1[CH];
        uint16_t dxh[CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const int bi = base0 + 16 * ch + b;
            if (row_on && bi < nb) {
#pragma unroll
                for (int i = 0; i < NM; ++i) wb[i][ch] = q8_load<KIND>(rows[i] + row_off + static_cast<size_t>(bi) * kBlk);
            }
        }
        if (base0 == 0) pre();
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const int bi = base0 + 16 * ch + b;
            if (row_on && bi < nb) {
                a0[ch] = *reinterpret_cast<const uint4 *>(act_qs + bi * 32);
                a1[ch] = *reinterpret_cast<const uint4 *>(act_qs + bi * 32 + 16);
                dxh[ch] = act_d[bi];
            }
        }
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            wave_lds_fence();  // earlier reads of the tile are done before it is overwritten
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                const int bi = base0 + 16 * ch + b;
                const bool on = row_on && bi < nb;
                int p[8];
                float ds = 0.0f;
                if (on) {
                    const uint32_t a[8] = {a0[ch].x, a0[ch].y, a0[ch].z, a0[ch].w, a1[ch].x, a1[ch].y, a1[ch].z, a1[ch].w};
                    q8_chunks<KIND>(wb[i][ch], a, p);
                    ds = h2f(wb[i][ch].d) * h2f(dxh[ch]);
                    if (PART) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) partials[i * pstride + (static_cast<size_t>(r4) * nb + bi) * 8 + j] = p[j];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) p[j] = 0;
                }
                float4 *dst = reinterpret_cast<float4 *>(&tile.pf[ch][r4 * 136 + b * 8]);
                dst[0] = make_float4(static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]),
                                     static_cast<float>(p[3]));
                dst[1] = make_float4(static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]),
                                     static_cast<float>(p[7]));
                tile.ds[ch][lane] = ds;
            }
            wave_lds_fence();
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                const int base = base0 + 16 * ch;
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    if (KIND == 1) {
                        const int blk_i = base + s;
                        if (blk_i < paired) {
                            const float pv = tile.pf[ch][r4 * 136 + s * 8 + c];
                            const float dv = tile.ds[ch][r4 * 16 + s];
                            if (blk_i & 1)
                                acc_odd[i] = __builtin_fmaf(dv, pv, acc_odd[i]);
                            else
                                acc[i] = __builtin_fmaf(dv, pv, acc[i]);
                        }
                    } else {
                        // every slot of the tile was written this pass, zeros for the blocks past the end of the row:
                        // those steps are fma(0, 0, acc) == acc (acc is never -0), so the chain needs no test
                        const float pv = tile.pf[ch][r4 * 136 + s * 8 + c];
                        const float dv = tile.ds[ch][r4 * 16 + s];
                        acc[i] = __builtin_fmaf(dv, pv, acc[i]);
                    }
                }
                if (KIND == 1 && (nb & 1) && base < nb && base + 16 >= nb) {
                    // trailing unpaired block: one rounded product with the whole-block integer sum
                    // (every chunk value is an exact integer < 2^24), added after the closing tree
                    const int s = (nb - 1) & 15;
                    float tot = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) tot += tile.pf[ch][r4 * 136 + s * 8 + j];
                    tail[i] = tile.ds[ch][r4 * 16 + s] * tot;
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NM; ++i) {
        const float r = close_lanes8((KIND == 1) ? acc[i] + acc_odd[i] : acc[i]);
        y[i] = (KIND == 1 && (nb & 1)) ? r + tail[i] : r;
    }
}

// ---- Q8_0 / IQ4_NL x Q8_0, four rows of 16 or 20 blocks, aligned fetch -----------------------------------------
// Four consecutive rows of NB blocks (NB = 16 or 20; Q8_0 or IQ4_NL) that start on a 16-byte boundary: 4 NB blocks are a
// whole number of 16-byte words (136 NB or 72 NB bytes), fetched as aligned words, copied to LDS and cut into blocks
// there - lane t takes block t (row t / NB), lanes 0..15 also block 64 + t when NB is 20.  Unaligned 16-byte requests at
// an 18- or 34-byte stride cost several times the address cycles of aligned ones, and with rows of 20 blocks the
// general routine needs a second, mostly idle pass.  The tile's chunk-sum area doubles as the staging area.
template <int NB>
struct __attribute__((aligned(16))) Q8TileNB {
    static constexpr int kRow = NB * 8 + 8;  // floats per row, padded (bank spread)
    float pf[4 * kRow];
    float ds[4 * NB];
};
template <int KIND>
WD_DEV Q8Block q8_block_from_lds(const uint8_t *stage, int t) {
    constexpr int kBlk = (KIND == 0) ? 34 : 18;
    const int byte0 = kBlk * t;
    Q8Block w;
    w.d = *reinterpret_cast<const uint16_t *>(stage + byte0);
    const uint32_t *sw = reinterpret_cast<const uint32_t *>(stage) + ((byte0 + 2) >> 2);
    const uint32_t sh = (t & 1) ? 0u : 2u;  // kBlk t + 2 is 2 (mod 4) for even t, 0 for odd t (kBlk = 2 mod 4 for both kinds)
    constexpr int kWords = (KIND == 0) ? 9 : 5;
    uint32_t r[kWords];
#pragma unroll
    for (int j = 0; j < kWords; ++j) r[j] = sw[j];
    w.q0.x = __builtin_amdgcn_alignbyte(r[1], r[0], sh), w.q0.y = __builtin_amdgcn_alignbyte(r[2], r[1], sh);
    w.q0.z = __builtin_amdgcn_alignbyte(r[3], r[2], sh), w.q0.w = __builtin_amdgcn_alignbyte(r[4], r[3], sh);
    if (KIND == 0) {
        w.q1.x = __builtin_amdgcn_alignbyte(r[5], r[4], sh), w.q1.y = __builtin_amdgcn_alignbyte(r[6], r[5], sh);
        w.q1.z = __builtin_amdgcn_alignbyte(r[7], r[6], sh), w.q1.w = __builtin_amdgcn_alignbyte(r[8], r[7], sh);
    }
    return w;
}
// The request and the rest apart, so that a caller can have several row groups in flight.
template <int KIND, int NB>
struct Q8CoalRaw {
    static constexpr int kBlk = (KIND == 0) ? 34 : 18;
    static constexpr int kWords = 4 * NB * kBlk / 16, kLoads = (kWords + 63) / 64;
    uint4 u[kLoads];
};
template <int KIND, int NB>
WD_DEV Q8CoalRaw<KIND, NB> q8_rows4_coal_request(const uint8_t *rows, int lane) {
    using Raw = Q8CoalRaw<KIND, NB>;
    static_assert(NB == 16 || NB == 20, "rows of 16 or 20 blocks");
    static_assert(4 * NB * Raw::kBlk % 16 == 0 && Raw::kWords * 16 + 8 <= static_cast<int>(sizeof(Q8TileNB<NB>)), "staging area");
    Raw raw;
#pragma unroll
    for (int i = 0; i < Raw::kLoads; ++i) raw.u[i] = gld_u128_aligned(rows + 16 * min(i * 64 + lane, Raw::kWords - 1));
    return raw;
}
// The fetched words into a staging area of Raw::kWords 16-byte words (the caller fences).
template <int KIND, int NB>
WD_DEV void q8_rows4_coal_stage(const Q8CoalRaw<KIND, NB> &raw, uint8_t *stage, int lane) {
    using Raw = Q8CoalRaw<KIND, NB>;
#pragma unroll
    for (int i = 0; i < Raw::kLoads; ++i) reinterpret_cast<uint4 *>(stage)[min(i * 64 + lane, Raw::kWords - 1)] = raw.u[i];
}
// Request and staging for a kind only known at run time (words: Q8CoalRaw<kind, NB>::kWords, the same in every lane):
// always as many loads as Q8_0 rows need, the surplus ones repeating the last word, so that the number of loads in
// flight does not depend on the kind.
template <int NB>
WD_DEV Q8CoalRaw<0, NB> q8_rows4_coal_request_any(const uint8_t *rows, int words, int lane) {
    Q8CoalRaw<0, NB> raw;
#pragma unroll
    for (int i = 0; i < Q8CoalRaw<0, NB>::kLoads; ++i) raw.u[i] = gld_u128_aligned(rows + 16 * min(i * 64 + lane, words - 1));
    return raw;
}
template <int NB>
WD_DEV void q8_rows4_coal_stage_any(const Q8CoalRaw<0, NB> &raw, uint8_t *stage, int words, int lane) {
#pragma unroll
    for (int i = 0; i < Q8CoalRaw<0, NB>::kLoads; ++i) reinterpret_cast<uint4 *>(stage)[min(i * 64 + lane, words - 1)] = raw.u[i];
}
// The dot products of the four staged rows; `stage` may be the tile itself (its chunk-sum area is overwritten only
// after the staged bytes have been read).  y of row r4 valid in lane 16 r4.  The float order is that of q8_rows4_multi.
// partials (PART): int32 [4 rows][NB blocks][8 chunk lanes].
template <int KIND, int NB, bool PART = false>
WD_DEV float q8_rows4_coal_dots(const uint8_t *stage, const int8_t *act_qs, const uint16_t *act_d, Q8TileNB<NB> &tile, int lane,
                                int32_t *partials = nullptr) {
    constexpr int kSecond = 4 * NB - 64, kRow = Q8TileNB<NB>::kRow;
    const int t1 = 64 + min(lane, max(kSecond, 1) - 1);
    const Q8Block w0 = q8_block_from_lds<KIND>(stage, lane);
    Q8Block w1 = w0;
    if (kSecond > 0) w1 = q8_block_from_lds<KIND>(stage, t1);
    wave_lds_fence();  // the staged bytes (and, by an earlier call, the tile) have been read; the tile now takes the chunk sums
    auto sums = [&](const Q8Block &w, int t) {
        const int row = t / NB, bi = t - row * NB;
        const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32);
        const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32 + 16);
        const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        int p[8];
        q8_chunks<KIND>(w, a, p);
        if (PART) {
#pragma unroll
            for (int j = 0; j < 8; ++j) partials[(row * NB + bi) * 8 + j] = p[j];
        }
        float4 *dst = reinterpret_cast<float4 *>(&tile.pf[row * kRow + bi * 8]);
        dst[0] = make_float4(static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]), static_cast<float>(p[3]));
        dst[1] = make_float4(static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]), static_cast<float>(p[7]));
        tile.ds[row * NB + bi] = h2f(w.d) * h2f(act_d[bi]);
    };
    sums(w0, lane);
    if (kSecond > 0 && lane < kSecond) sums(w1, t1);
    wave_lds_fence();
    const int r4 = lane >> 4, c = lane & 7;
    float acc = 0.0f, acc_odd = 0.0f;
#pragma unroll
    for (int s = 0; s < NB; ++s) {
        const float pv = tile.pf[r4 * kRow + s * 8 + c], dv = tile.ds[r4 * NB + s];
        if (KIND == 1 && (s & 1))
            acc_odd = __builtin_fmaf(dv, pv, acc_odd);  // IQ4_NL: even and odd blocks accumulate apart (NB is even: no tail)
        else
            acc = __builtin_fmaf(dv, pv, acc);
    }
    return close_lanes8(KIND == 1 ? acc + acc_odd : acc);
}
template <int KIND, int NB, bool PART = false>
WD_DEV float q8_rows4_coal_finish(const Q8CoalRaw<KIND, NB> &raw, const int8_t *act_qs, const uint16_t *act_d, Q8TileNB<NB> &tile,
                                  int lane, int32_t *partials = nullptr) {
    uint8_t *stage = reinterpret_cast<uint8_t *>(&tile);  // chunk sums and scales together are large enough
    wave_lds_fence();  // earlier reads of the tile are done before it is overwritten
    q8_rows4_coal_stage<KIND, NB>(raw, stage, lane);
    wave_lds_fence();
    return q8_rows4_coal_dots<KIND, NB, PART>(stage, act_qs, act_d, tile, lane, partials);
}
// rows: first of the four rows.  `pre` runs between the request and the first read of the activation.
template <int KIND, int NB, typename Pre = NoPre>
WD_DEV float q8_rows4_coal(const uint8_t *rows, const int8_t *act_qs, const uint16_t *act_d, Q8TileNB<NB> &tile, int lane,
                           Pre pre = Pre()) {
    const Q8CoalRaw<KIND, NB> raw = q8_rows4_coal_request<KIND, NB>(rows, lane);
    pre();
    return q8_rows4_coal_finish<KIND, NB>(raw, act_qs, act_d, tile, lane);
}

template <int KIND, bool PART>
WD_DEV float q8_rows4(const uint8_t *rows, int nrows, int nb, const int8_t *act_qs, const uint16_t *act_d,
                      Q8Tile &tile, int lane, int32_t *partials) {
    const uint8_t *const rr[1] = {rows};
    float y[1];
    q8_rows4_multi<KIND, 1, 1, PART, NoPre>(rr, nrows, nb, act_qs, act_d, tile, lane, y, partials, 0);
    return y[0];
}

// ---- Q8_0 x Q8_0, one row per wave ---------------------------------------------------------------------
// For long rows (gate/up projections): lane b takes blocks b, b + 64, ...  The chunk sums of a pass
// are handed over transposed ([chunk][block]) so that the chain lanes read them four at a time.
struct Q8RowTile {
    float pf[8][68];  // [c][block of the pass], rows padded to 68 floats (16-byte aligned, bank spread)
    float ds[64];
};

// rows[i]: the row of matrix i.  y[i] valid in lane 0 (every aligned group of 8 lanes runs the same chain).
// One pass of the row chains: block `bi` of every matrix (wb[i], loaded by the caller; lanes with on == false
// contribute nothing) against the activation; acc[i] is chunk lane (lane & 7)'s accumulator.
template <int NM>
WD_DEV void q8_row_wave_pass(const Q8Block (&wb)[NM], bool on, int bi, const int8_t *act_qs, const uint16_t *act_d,
                             Q8RowTile &tile, int lane, float (&acc)[NM]) {
    const int c = lane & 7;
    uint32_t a[8];
    float dx = 0.0f;
    if (on) {
        const uint4 a0 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32);
        const uint4 a1 = *reinterpret_cast<const uint4 *>(act_qs + bi * 32 + 16);
        a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
        dx = h2f(act_d[bi]);
    }
#pragma unroll
    for (int i = 0; i < NM; ++i) {
        int p[8];
        float ds = 0.0f;
        if (on) {
            q8_chunks<0>(wb[i], a, p);
            ds = h2f(wb[i].d) * dx;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) p[j] = 0;
        }
        wave_lds_fence();  // earlier reads of the tile are done before it is overwritten
#pragma unroll
        for (int j = 0; j < 8; ++j) tile.pf[j][lane] = static_cast<float>(p[j]);
        tile.ds[lane] = ds;
        wave_lds_fence();
        // blocks past the end of the row contribute fma(0, 0, acc) == acc
        // (partial unroll: a full one makes the compiler hold all 128 tile values in registers at once)
#pragma unroll 4
        for (int s4 = 0; s4 < 16; ++s4) {
            const float4 pv = *reinterpret_cast<const float4 *>(&tile.pf[c][4 * s4]);
            const float4 dv = *reinterpret_cast<const float4 *>(&tile.ds[4 * s4]);
            acc[i] = __builtin_fmaf(dv.x, pv.x, acc[i]);
            acc[i] = __builtin_fmaf(dv.y, pv.y, acc[i]);
            acc[i] = __builtin_fmaf(dv.z, pv.z, acc[i]);
            acc[i] = __builtin_fmaf(dv.w, pv.w, acc[i]);
        }
    }
}

// rows[i]: the row of matrix i.  y[i] valid in lane 0 (every aligned group of 8 lanes runs the same chain).
template <int NM, typename Pre = NoPre>
WD_DEV void q8_row_wave(const uint8_t *const (&rows)[NM], int nb, const int8_t *act_qs, const uint16_t *act_d,
                        Q8RowTile &tile, int lane, float (&y)[NM], Pre pre = Pre()) {
    float acc[NM];
#pragma unroll
    for (int i = 0; i < NM; ++i) acc[i] = 0.0f;
    for (int base = 0; base < nb; base += 64) {
        const int bi = base + lane;
        const bool on = bi < nb;
        Q8Block wb[NM];
        if (on) {
#pragma unroll
            for (int i = 0; i < NM; ++i) wb[i] = q8_load<0>(rows[i] + static_cast<size_t>(bi) * 34);
        }
        if (base == 0) pre();
        q8_row_wave_pass<NM>(wb, on, bi, act_qs, act_d, tile, lane, acc);
    }
#pragma unroll
    for (int i = 0; i < NM; ++i) y[i] = close_lanes8(acc[i]);
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
            const uint4 n = gld_u128(blk + 2);
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
            sumf += h2f(gld_u16(blk)) * h2f(act_d[bi]) * static_cast<float>(sumi);
        }
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) sumf += lane_xor(sumf, m);
    return sumf;
}

}  // namespace wd
