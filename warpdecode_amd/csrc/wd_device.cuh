// Device-side building blocks for the gfx950 MoE decode kernels: unaligned loads,
// half conversions, the ggml exponential, cross-lane helpers for 64-wide wavefronts.
//
// Everything that fixes a floating-point result is written as explicit single
// operations (the translation unit is compiled with -ffp-contract=off), so that the
// kernels round exactly where the CPU path of the reference rounds.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define WD_DEV __device__ __forceinline__

#include "wd_exp2f_table.inc"

namespace wd {

constexpr int kWave = 64;

// GGUF blocks are only 2-byte aligned (34-, 110-, 82-, 18-byte strides).  The byte-wise
// copy lets the compiler pick the widest load the target allows for unaligned addresses.
template <typename T>
WD_DEV T ldu(const void *p) {
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

WD_DEV float h2f(uint16_t h) {
    _Float16 f;
    __builtin_memcpy(&f, &h, 2);
    return static_cast<float>(f);  // exact, subnormal halves included
}

// f32 -> f16 bits as the reference CPU path rounds a block scale
// (src/qwen38_cpu_moe.cuh:109-137): round-to-nearest-even, except that magnitudes
// below 2^-24 become signed zero and NaN becomes infinity.
WD_DEV uint16_t f2h_ref(float v) {
    const _Float16 f = static_cast<_Float16>(v);
    uint16_t h;
    __builtin_memcpy(&h, &f, 2);
    if (__builtin_fabsf(v) < 0x1p-24f) h &= 0x8000u;
    if (v != v) h = static_cast<uint16_t>((h & 0x8000u) | 0x7c00u);
    return h;
}

WD_DEV uint32_t f_bits(float v) { return __builtin_bit_cast(uint32_t, v); }
WD_DEV float bits_f(uint32_t b) { return __builtin_bit_cast(float, b); }

// ggml_v_expf polynomial, one lane (src/qwen38_cpu_moe.cuh:816-834,
// src/qwen38_exact_math.cuh:94-115).
WD_DEV float exp_ggml(float x) {
    const float r = 0x1.8p23f;
    const float z = __builtin_fmaf(x, 0x1.715476p+0f, r);
    const float n = z - r;
    const float b = __builtin_fmaf(-n, 0x1.7f7d1cp-20f, __builtin_fmaf(-n, 0x1.62e4p-1f, x));
    const uint32_t e = f_bits(z) << 23;
    const float k = bits_f(e + 0x3f800000u);
    const float u = b * b;
    const float p2 = __builtin_fmaf(0x1.0e4020p-7f, b, 0x1.573e2ep-5f);
    const float p1 = __builtin_fmaf(0x1.555e66p-3f, b, 0x1.fffdb6p-2f);
    const float j = __builtin_fmaf(__builtin_fmaf(p2, u, p1), u, 0x1.ffffecp-1f * b);
    if (__builtin_fabsf(n) <= 126.0f) return __builtin_fmaf(j, k, k);
    const uint32_t g = (n <= 0.0f) ? 0x82000000u : 0u;
    const float s1 = bits_f(g + 0x7f000000u);
    if (__builtin_fabsf(n) > 192.0f) return s1 * s1;
    const float s2 = bits_f(e - g);
    return __builtin_fmaf(s2, j, s2) * s1;
}

// IEEE division (hipcc's default for '/': correctly rounded).
// expf as glibc computes it (sysdeps/ieee754/flt-32/e_expf.c: a table of 2^(i/32), a cubic in double, every step one
// rounded double operation), which the reference uses for its exact sigmoid: src/qwen38_exact_math.cuh:136-166.
WD_DEV float expf_glibc(float x) {
    constexpr uint64_t tab[32] = WD_EXP2F_TABLE;
    constexpr double shift = 0x1.8p+52, invln2n = 0x1.71547652b82fep+0 * 32.0;
    constexpr double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0, c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0,
                     c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const uint32_t ix = f_bits(x), abstop = (ix >> 20) & 0x7ffu;
    if (abstop >= (0x42b00000u >> 20)) {  // |x| >= 88, infinities, NaN
        if (ix == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8u) return x + x;
        if (x > 0x1.62e42ep6f) return bits_f(0x7f800000u);  // 2^97 * 2^97
        if (x < -0x1.9fe368p6f) return 0.0f;               // 2^-95 * 2^-95
    }
    const double z = invln2n * static_cast<double>(x);
    const double kd_shift = z + shift;
    const uint64_t ki = __builtin_bit_cast(uint64_t, kd_shift);
    const double kd = kd_shift - shift;
    const double r = z - kd;
    const double s = __builtin_bit_cast(double, tab[ki & 31u] + (ki << 47));
    const double p = c0 * r + c1;
    const double r2 = r * r;
    double y = c2 * r + 1.0;
    y = p * r2 + y;
    y = y * s;
    return static_cast<float>(y);
}
// src/qwen38_exact_math.cuh:195-198
WD_DEV float sigmoid_exact(float x) { return 1.0f / (1.0f + expf_glibc(-x)); }
// float -> half -> float, IEEE round to nearest even (src/qwen38_precision.hpp:40-55)
WD_DEV float round_half(float v) { return static_cast<float>(static_cast<_Float16>(v)); }
// The weight of one residual stream in the hyper-connection combine: 2 sigmoid(inject / hc), each step one rounded
// float operation (src/qwen38_hc.cuh:2542-2544).
WD_DEV float hc_weight(float inject, int hc) {
    const float z = inject * (1.0f / static_cast<float>(hc));
    return 2.0f * sigmoid_exact(z);
}

WD_DEV float silu_ggml(float v) { return v / (1.0f + exp_ggml(-v)); }
WD_DEV float sigmoid_ggml(float v) { return 1.0f / (1.0f + exp_ggml(-v)); }

WD_DEV int sdot4(uint32_t a, uint32_t b, int acc) {
    // (Not the three-operand form with a constant 0 through inline assembly, although it saves the move that zeroes the
    // two-operand form's accumulator: the result of a dot instruction needs wait states before another vector instruction
    // reads it, which the compiler inserts for instructions it knows and not behind assembly text - results were wrong.)
    // A dot product that starts from zero is asked for with the clamp bit: only the three-operand encoding has one, so the
    // compiler takes that encoding, with the constant 0 as its third operand, instead of the two-operand form and a
    // move that zeroes its accumulator first.  (Four products of bytes cannot overflow: the bit changes no result.)
    if (__builtin_constant_p(acc) && acc == 0) return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), 0, true);
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), acc, false);
}

// ---- cross-lane -----------------------------------------------------------------------
// Data-parallel-primitive (DPP) moves work inside rows of 16 lanes without touching LDS:
//   quad_perm 0xB1 / 0x4E   lane ^ 1 / lane ^ 2
//   row_ror:8               lane ^ 8;     row_ror:4   lane i reads lane (i - 4) mod 16 of its row
//   row_shr:n / row_shl:n   lane i reads lane i - n / i + n of its row (no source: keeps `old`,
//                           or 0 with bound_ctrl)
//   row_bcast15 / 31        rows 1,3 read lane 15 / 47; rows 2,3 read lane 31 (row_mask selects)
// Halves and row pairs are exchanged with v_permlane32_swap / v_permlane16_swap (gfx950).
WD_DEV int lane_id() { return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }

template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND = false>
WD_DEV int dpp_i(int old, int v) {
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, BANK_MASK, BOUND);
}
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND = false>
WD_DEV float dpp_f(float old, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                                                CTRL, ROW_MASK, BANK_MASK, BOUND));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppRor4 = 0x124, kDppRor8 = 0x128, kDppBcast15 = 0x142,
              kDppBcast31 = 0x143;
constexpr int kDppShr1 = 0x111, kDppShl1 = 0x101, kDppShl2 = 0x102, kDppShl4 = 0x104, kDppShl7 = 0x107;
constexpr int kDppShr2 = 0x112, kDppShl14 = 0x10E;

WD_DEV float readlane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Wave-wide reductions of order-free operations; the result is uniform.
WD_DEV float wave_max(float v) {
    v = __builtin_fmaxf(v, dpp_f<kDppXor1>(v, v));
    v = __builtin_fmaxf(v, dpp_f<kDppXor2>(v, v));
    v = __builtin_fmaxf(v, dpp_f<kDppRor4>(v, v));
    v = __builtin_fmaxf(v, dpp_f<kDppRor8>(v, v));
    v = __builtin_fmaxf(v, dpp_f<kDppBcast15, 0xa>(v, v));
    v = __builtin_fmaxf(v, dpp_f<kDppBcast31, 0xc>(v, v));
    return readlane_f(v, 63);
}
WD_DEV int wave_min_i(int v) {
    v = min(v, dpp_i<kDppXor1>(v, v));
    v = min(v, dpp_i<kDppXor2>(v, v));
    v = min(v, dpp_i<kDppRor4>(v, v));
    v = min(v, dpp_i<kDppRor8>(v, v));
    v = min(v, dpp_i<kDppBcast15, 0xa>(v, v));
    v = min(v, dpp_i<kDppBcast31, 0xc>(v, v));
    return __builtin_amdgcn_readlane(v, 63);
}
// Maximum over aligned groups of four / eight lanes (every lane gets its group's value).
WD_DEV float quad_max(float v) {
    v = __builtin_fmaxf(v, dpp_f<kDppXor1>(v, v));
    return __builtin_fmaxf(v, dpp_f<kDppXor2>(v, v));
}
// The same for values that are zero, positive or NaN - the magnitudes a quantiser takes a block's maximum of -, as
// unsigned integers on the bits: such floats order like their bit patterns, a NaN counts as zero (the reference takes
// the maximum with fmaxf from 0.0f, which drops it), and an integer maximum needs neither the copy nor the quieting of
// a possible signalling NaN that the compiler wraps round every float maximum fed from a lane shuffle: one instruction
// per step instead of four.
WD_DEV uint32_t nonneg_bits(float v) { return v == v ? f_bits(v) : 0u; }
template <int CTRL>
WD_DEV uint32_t umax_step(uint32_t u) {
    return max(u, static_cast<uint32_t>(dpp_i<CTRL, 0xf, 0xf, true>(0, static_cast<int>(u))));
}
WD_DEV float quad_max_nonneg(float v) {
    uint32_t u = nonneg_bits(v);
    u = umax_step<kDppXor1>(u);
    u = umax_step<kDppXor2>(u);
    return bits_f(u);
}
WD_DEV float oct_max_nonneg(float v) {  // aligned groups of eight lanes
    uint32_t u = nonneg_bits(v);
    u = umax_step<kDppXor1>(u);
    u = umax_step<kDppXor2>(u);
    u = umax_step<0x141>(u);  // row_half_mirror pairs the two quads of a group
    return bits_f(u);
}
WD_DEV float wave_max_nonneg(float v) {  // uniform
    uint32_t u = nonneg_bits(v);
    u = umax_step<kDppXor1>(u);
    u = umax_step<kDppXor2>(u);
    u = umax_step<kDppRor4>(u);
    u = umax_step<kDppRor8>(u);
    u = max(u, static_cast<uint32_t>(dpp_i<kDppBcast15, 0xa>(static_cast<int>(u), static_cast<int>(u))));
    u = max(u, static_cast<uint32_t>(dpp_i<kDppBcast31, 0xc>(static_cast<int>(u), static_cast<int>(u))));
    return bits_f(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(u), 63)));
}
WD_DEV int quad_sum_i(int v) {
    v += dpp_i<kDppXor1>(0, v);
    return v + dpp_i<kDppXor2>(0, v);
}

// General shuffles (LDS crossbar; slower than DPP, used off the hot paths).
template <typename T>
WD_DEV T lane_xor(T v, int mask) {
    return __shfl_xor(v, mask, kWave);
}
template <typename T>
WD_DEV T lane_down(T v, int delta) {
    return __shfl_down(v, delta, kWave);
}
template <typename T>
WD_DEV T lane_get(T v, int src) {
    return __shfl(v, src, kWave);
}

// Orders this wave's LDS traffic for cross-lane hand-offs through LDS.  The hardware
// executes a wave's LDS instructions in order; the fence keeps the compiler from moving
// a lane's read above another lane's (earlier) write.
WD_DEV void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Closing tree of eight chunk lanes held by lanes 0..7 of a 16-lane row (lane & 7 = chunk):
// ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)); valid in lane 0 of the row.
WD_DEV float close_lanes8(float v) {
    v = v + dpp_f<kDppShl4>(0.0f, v);
    v = v + dpp_f<kDppShl2>(0.0f, v);
    v = v + dpp_f<kDppShl1>(0.0f, v);
    return v;
}

// The same tree over eight uniform-addressable values: chunk c is taken from lane 8*c + 7.
// The result is uniform.
WD_DEV float close_lanes8_strided(float v) {
    const float l0 = readlane_f(v, 7), l1 = readlane_f(v, 15), l2 = readlane_f(v, 23), l3 = readlane_f(v, 31);
    const float l4 = readlane_f(v, 39), l5 = readlane_f(v, 47), l6 = readlane_f(v, 55), l7 = readlane_f(v, 63);
    const float a = l0 + l4, b = l1 + l5, c = l2 + l6, e = l3 + l7;
    return (a + c) + (b + e);
}

// Unaligned loads from global memory (address space 1), so that no flat (generic) load is issued.
typedef uint16_t __attribute__((aligned(2))) wd_u16a;
typedef uint32_t __attribute__((aligned(2))) wd_u32a;
typedef uint32_t wd_u64a __attribute__((ext_vector_type(2), aligned(2)));
typedef uint32_t wd_u128a __attribute__((ext_vector_type(4), aligned(2)));
#define WD_GLOBAL __attribute__((address_space(1)))
WD_DEV uint32_t gld_u8(const uint8_t *p) { return *((const WD_GLOBAL uint8_t *)(p)); }
WD_DEV uint16_t gld_u16(const uint8_t *p) { return *((const WD_GLOBAL wd_u16a *)(p)); }
WD_DEV uint32_t gld_u32(const uint8_t *p) { return *((const WD_GLOBAL wd_u32a *)(p)); }
WD_DEV uint2 gld_u64(const uint8_t *p) {
    const wd_u64a v = *((const WD_GLOBAL wd_u64a *)(p));
    return make_uint2(v.x, v.y);
}
WD_DEV uint4 gld_u128(const uint8_t *p) {
    const wd_u128a v = *((const WD_GLOBAL wd_u128a *)(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
// A pointer that is the same in every lane of the wave, moved to scalar registers (frees two vector registers and
// lets loads use the scalar base + vector offset form).
template <typename T>
WD_DEV T *uniform_ptr(T *p) {
    const uintptr_t v = reinterpret_cast<uintptr_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<T *>((static_cast<uintptr_t>(hi) << 32) | lo);
}
// A 32-bit value at a wave-uniform address through the scalar path (lower latency than a vector load).  Only for
// data written before the launch: the scalar cache is not coherent with stores of the running dispatch.
WD_DEV int sld_i32(const int32_t *p) {
    const uintptr_t v = reinterpret_cast<uintptr_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return *((const __attribute__((address_space(4))) int32_t *)((static_cast<uintptr_t>(hi) << 32) | lo));
}
// 16-byte aligned form (one full-width request per lane)
typedef uint32_t wd_u128 __attribute__((ext_vector_type(4), aligned(16)));
WD_DEV uint4 gld_u128_aligned(const uint8_t *p) {
    const wd_u128 v = *((const WD_GLOBAL wd_u128 *)(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

}  // namespace wd
