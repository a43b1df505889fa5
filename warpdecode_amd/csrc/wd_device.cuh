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
WD_DEV float silu_ggml(float v) { return v / (1.0f + exp_ggml(-v)); }
WD_DEV float sigmoid_ggml(float v) { return 1.0f / (1.0f + exp_ggml(-v)); }

WD_DEV int sdot4(uint32_t a, uint32_t b, int acc) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), acc, false);
}

// ---- cross-lane -----------------------------------------------------------------
WD_DEV int lane_id() { return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }

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

WD_DEV float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = __builtin_fmaxf(v, lane_xor(v, m));
    return v;
}
WD_DEV int wave_min_i(int v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = min(v, lane_xor(v, m));
    return v;
}

// Orders this wave's LDS traffic for cross-lane hand-offs through LDS.  The hardware
// executes a wave's LDS instructions in order; the fence keeps the compiler from moving
// a lane's read above another lane's (earlier) write.
WD_DEV void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Closing tree of eight chunk lanes held by eight consecutive lanes (lane & 7 = chunk):
// ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)); valid in the lane with (lane & 7) == 0.
WD_DEV float close_lanes8(float v) {
    v = v + lane_down(v, 4);
    v = v + lane_down(v, 2);
    v = v + lane_down(v, 1);
    return v;
}

}  // namespace wd
