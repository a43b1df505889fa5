/*
 * CPU oracle for the batch=1 MoE decode path.  TEST INFRASTRUCTURE ONLY: the
 * shipped library never links or calls this file.
 *
 * What each function follows and how it is pinned (tests/test_oracle_*.py):
 *
 *   f16 conversions        src/qwen38_cpu_moe.cuh:77-137     all 65536 halves vs numpy float16, RNE
 *                                                            vs numpy on random + boundary floats, and
 *                                                            vs the compiled reference header
 *   quantize_q8_0 / q8_K   :220-263                          compiled reference header (bit-exact) +
 *                                                            invariants (|q|<=127, bsums, sign rule)
 *   row_iq3_s/iq2_s/q8_0/  :298-440, :565-758                compiled reference header, AVX2 and scalar
 *   iq4_nl                                                   twins (bit-exact) + closed forms of
 *                                                            tests/lowbit_cuda_test.cu:50-98 + brute
 *                                                            force through an independent dequantiser
 *   exp/silu/sigmoid       :816-842                          compiled reference header (bit-exact) +
 *                                                            libm exp to 2 ulp
 *   dot_f32                :847-871                          compiled reference header (bit-exact)
 *   expert chain / layer   :1169-1291                        compiled reference run_layer (bit-exact)
 *   softmax_row / select   src/qwen38_moe.cuh:711-818        known answer of tests/qwen38_moe_cuda_test.cu
 *                                                            :237-254, numpy softmax/top-k away from
 *                                                            ties, tie / -inf / underflow rows by
 *                                                            hand.  The per-8 summation order is
 *                                                            PARITY UNPINNED at bit level: that block
 *                                                            of the reference only builds with CUDA
 *                                                            headers, which this image lacks.
 *   row_q4_0_q8_0          src/warodecode.cu:1534-1562       int32 block sums vs brute force; the
 *                                                            reference fixes no float order there
 *   row_q6_K_q8_K          src/lowbit.cuh:2510-2612          integer lane sums vs brute force through an
 *                                                            independent dequantiser (value formula of
 *                                                            src/ggml_dequant.hpp:102-140), the known
 *                                                            answer of tests/lowbit_cuda_test.cu:60-68,
 *                                                            float64 dot within 1e-5.  The float order
 *                                                            (eight lanes, fma per super-block, hsum
 *                                                            tree) is PARITY UNPINNED at bit level: the
 *                                                            reference has it only as a CUDA kernel and
 *                                                            ggml itself is not in the tree.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, no fast-math).
 */
#include "wd_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "../warpdecode_amd/csrc/wd_codebooks.inc"
#include "../warpdecode_amd/csrc/wd_exp2f_table.inc"

/* ------------------------------------------------------------------------- */
/* Codebooks                                                                 */
/* ------------------------------------------------------------------------- */
static uint32_t g_iq3s[512];
static uint64_t g_iq2s[1024];
static pthread_once_t g_grid_once = PTHREAD_ONCE_INIT;

static void expand_grids(void) {
    const char *s3 = WD_IQ3S_GRID_DIGITS;
    for (int e = 0; e < 512; ++e) {
        uint32_t v = 0;
        for (int j = 0; j < 4; ++j) {
            const uint32_t t = (uint32_t)(s3[e * 4 + j] - '0');
            v |= (2u * t + 1u) << (8 * j);
        }
        g_iq3s[e] = v;
    }
    const char *s2 = WD_IQ2S_GRID_DIGITS;
    for (int e = 0; e < 1024; ++e) {
        uint64_t v = 0;
        for (int j = 0; j < 8; ++j) {
            const uint64_t t = (uint64_t)(s2[e * 8 + j] - '0');
            v |= (8u + 17u * t + (t == 2)) << (8 * j);
        }
        g_iq2s[e] = v;
    }
}

const uint32_t *wdo_iq3s_grid(void) {
    pthread_once(&g_grid_once, expand_grids);
    return g_iq3s;
}

const uint64_t *wdo_iq2s_grid(void) {
    pthread_once(&g_grid_once, expand_grids);
    return g_iq2s;
}

/* ------------------------------------------------------------------------- */
/* Geometry                                                                  */
/* ------------------------------------------------------------------------- */
int wdo_block_elems(int type) {
    switch (type) {
        case WDO_IQ3_S:
        case WDO_IQ2_S:
        case WDO_Q6_K: return 256;
        case WDO_Q8_0:
        case WDO_Q4_0:
        case WDO_IQ4_NL: return 32;
        case WDO_F32: return 1;
        default: return 0;
    }
}

size_t wdo_block_bytes(int type) {
    switch (type) {
        case WDO_IQ3_S: return 110;
        case WDO_IQ2_S: return 82;
        case WDO_Q6_K: return 210;
        case WDO_Q8_0: return 34;
        case WDO_Q4_0:
        case WDO_IQ4_NL: return 18;
        case WDO_F32: return 4;
        default: return 0;
    }
}

size_t wdo_row_bytes(int type, int cols) {
    const int be = wdo_block_elems(type);
    if (be == 0 || cols <= 0 || cols % be != 0) return 0;
    return (size_t)(cols / be) * wdo_block_bytes(type);
}

/* ------------------------------------------------------------------------- */
/* Half precision                                                            */
/* ------------------------------------------------------------------------- */
static inline uint32_t f32_bits(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    return b;
}

static inline float bits_f32(uint32_t b) {
    float v;
    memcpy(&v, &b, 4);
    return v;
}

float wdo_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t ex = (h >> 10) & 31u;
    uint32_t man = h & 0x3ffu;
    if (ex == 31u) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (ex != 0u) return bits_f32(sign | ((ex + 112u) << 23) | (man << 13));
    if (man == 0u) return bits_f32(sign);
    /* subnormal half: value = man * 2^-24, renormalise */
    int e = 113; /* exponent field of 2^-14 */
    while ((man & 0x400u) == 0u) {
        man <<= 1;
        --e;
    }
    return bits_f32(sign | ((uint32_t)e << 23) | ((man & 0x3ffu) << 13));
}

uint16_t wdo_f32_to_f16(float value) {
    const uint32_t b = f32_bits(value);
    const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    const int e = (int)((b >> 23) & 0xffu) - 127;
    const uint32_t man = b & 0x7fffffu;
    /* The reference maps every exponent above 15 (NaN included) to infinity and
     * everything below 2^-25 to signed zero. */
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    if (e < -24) return sign;
    if (e < -14) {
        const uint32_t full = man | 0x800000u;
        const int shift = 13 + (-14 - e); /* 14..23 */
        uint32_t q = full >> shift;
        const uint32_t rest = full & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        if (rest > half || (rest == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q); /* q == 0x400 is the smallest normal: correct encoding */
    }
    uint32_t q = man >> 13;
    const uint32_t rest = man & 0x1fffu;
    uint32_t ef = (uint32_t)(e + 15);
    if (rest > 0x1000u || (rest == 0x1000u && (q & 1u))) {
        ++q;
        if (q == 0x400u) {
            q = 0;
            ++ef; /* may reach 31 = infinity, as IEEE rounding demands */
        }
    }
    return (uint16_t)(sign | (ef << 10) | q);
}

static inline float half_at(const uint8_t *p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return wdo_f16_to_f32(h);
}

/* ------------------------------------------------------------------------- */
/* Activation quantisers                                                     */
/* ------------------------------------------------------------------------- */
void wdo_quantize_q8_0(const float *x, int n, int8_t *qs, uint16_t *d) {
    for (int b = 0; b < n / 32; ++b) {
        const float *src = x + (size_t)b * 32;
        int8_t *dst = qs + (size_t)b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(src[i]));
        d[b] = wdo_f32_to_f16(amax / 127.0f);
        if (amax == 0.0f) {
            memset(dst, 0, 32);
            continue;
        }
        const float inv = 127.0f / amax;
        for (int i = 0; i < 32; ++i) {
            int q = (int)nearbyintf(src[i] * inv);
            if (q > 127) q = 127;
            if (q < -128) q = -128;
            dst[i] = (int8_t)q;
        }
    }
}

void wdo_quantize_q8_K(const float *x, int n, int8_t *qs, float *d, int16_t *bsums) {
    for (int b = 0; b < n / 256; ++b) {
        const float *src = x + (size_t)b * 256;
        int8_t *dst = qs + (size_t)b * 256;
        int16_t *bs = bsums + (size_t)b * 16;
        float amax = 0.0f;
        for (int i = 0; i < 256; ++i) amax = fmaxf(amax, fabsf(src[i]));
        if (amax == 0.0f) {
            d[b] = 0.0f;
            memset(dst, 0, 256);
            memset(bs, 0, 32);
            continue;
        }
        /* Always-negative inverse scale: the quants carry the opposite sign of x
         * and d is negative, so d*q has the sign of x. */
        const float iscale = -127.0f / amax;
        for (int i = 0; i < 256; ++i) {
            int q = (int)nearbyintf(src[i] * iscale);
            if (q > 127) q = 127;
            dst[i] = (int8_t)q;
        }
        for (int j = 0; j < 16; ++j) {
            int s = 0;
            for (int i = 0; i < 16; ++i) s += dst[16 * j + i];
            bs[j] = (int16_t)s;
        }
        d[b] = 1.0f / iscale;
    }
}

/* ------------------------------------------------------------------------- */
/* Row dots                                                                  */
/* ------------------------------------------------------------------------- */
/* Closing tree of the eight chunk lanes: ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)). */
static inline float close_lanes(const float l[8]) {
    const float a = l[0] + l[4];
    const float b = l[1] + l[5];
    const float c = l[2] + l[6];
    const float e = l[3] + l[7];
    return (a + c) + (b + e);
}

/* Signed dot of four codebook magnitudes (bytes of `mags`) against four activations. */
static inline int32_t dot4_signed(uint32_t mags, unsigned sign_bits, const int8_t *a) {
    int32_t s = 0;
    for (int j = 0; j < 4; ++j) {
        const int m = (int)((mags >> (8 * j)) & 0xffu);
        s += (int)a[j] * (((sign_bits >> j) & 1u) ? -m : m);
    }
    return s;
}

float wdo_row_iq3_s_q8_K(const uint8_t *w, const int8_t *qs_a, const float *d_a, int cols, int32_t *partials) {
    const uint32_t *grid = wdo_iq3s_grid();
    float lane[8] = {0};
    for (int sb = 0; sb < cols / 256; ++sb) {
        const uint8_t *blk = w + (size_t)sb * 110;
        const uint8_t *qs = blk + 2, *qh = blk + 66, *signs = blk + 74, *scales = blk + 106;
        const int8_t *a = qs_a + (size_t)sb * 256;
        const float d = half_at(blk) * d_a[sb];
        for (int c = 0; c < 8; ++c) {
            const int g = c >> 1, h = c & 1;
            int32_t p = 0;
            for (int ib = 0; ib < 8; ++ib) {
                const unsigned nib = (ib & 1) ? (scales[ib >> 1] >> 4) : (scales[ib >> 1] & 15u);
                const int ls = 1 + 2 * (int)nib;
                const unsigned idx = qs[ib * 8 + 2 * g + h] | (((unsigned)qh[ib] << (8 - 2 * g - h)) & 0x100u);
                const unsigned sbits = (unsigned)signs[ib * 4 + g] >> (4 * h);
                p += ls * dot4_signed(grid[idx], sbits, a + ib * 32 + c * 4);
            }
            if (partials) partials[sb * 8 + c] = p;
            lane[c] = fmaf(d, (float)p, lane[c]);
        }
    }
    return close_lanes(lane);
}

float wdo_row_iq2_s_q8_K(const uint8_t *w, const int8_t *qs_a, const float *d_a, int cols, int32_t *partials) {
    const uint64_t *grid = wdo_iq2s_grid();
    float lane[8] = {0};
    for (int sb = 0; sb < cols / 256; ++sb) {
        const uint8_t *blk = w + (size_t)sb * 82;
        const uint8_t *qs = blk + 2, *signs = blk + 34, *qh = blk + 66, *scales = blk + 74;
        const int8_t *a = qs_a + (size_t)sb * 256;
        const float d = half_at(blk) * d_a[sb];
        for (int c = 0; c < 8; ++c) {
            const int g = c >> 1, h = c & 1;
            int32_t p = 0;
            for (int ib = 0; ib < 8; ++ib) {
                const unsigned nib = (c < 4) ? (scales[ib] & 15u) : (scales[ib] >> 4);
                const int ls = 1 + 2 * (int)nib;
                const unsigned idx = qs[ib * 4 + g] | (((unsigned)qh[ib] << (8 - 2 * g)) & 0x300u);
                const uint32_t mags = (uint32_t)(grid[idx] >> (32 * h));
                const unsigned sbits = (unsigned)signs[ib * 4 + g] >> (4 * h);
                p += ls * dot4_signed(mags, sbits, a + ib * 32 + c * 4);
            }
            if (partials) partials[sb * 8 + c] = p;
            lane[c] = fmaf(d, (float)p, lane[c]);
        }
    }
    return 0.125f * close_lanes(lane);
}

float wdo_row_q8_0_q8_0(const uint8_t *w, const int8_t *qs_a, const uint16_t *d_a, int cols, int32_t *partials) {
    float lane[8] = {0};
    for (int b = 0; b < cols / 32; ++b) {
        const uint8_t *blk = w + (size_t)b * 34;
        const int8_t *q = (const int8_t *)(blk + 2);
        const int8_t *a = qs_a + (size_t)b * 32;
        const float d = half_at(blk) * wdo_f16_to_f32(d_a[b]);
        for (int c = 0; c < 8; ++c) {
            int32_t p = 0;
            for (int j = 0; j < 4; ++j) p += (int)q[4 * c + j] * (int)a[4 * c + j];
            if (partials) partials[b * 8 + c] = p;
            lane[c] = fmaf(d, (float)p, lane[c]);
        }
    }
    return close_lanes(lane);
}

static const int8_t k_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

float wdo_row_iq4_nl_q8_0(const uint8_t *w, const int8_t *qs_a, const uint16_t *d_a, int cols, int32_t *partials) {
    const int nb = cols / 32;
    float acc[2][8];
    memset(acc, 0, sizeof(acc));
    int32_t p[8];
    const int paired = nb & ~1;
    for (int b = 0; b < nb; ++b) {
        const uint8_t *blk = w + (size_t)b * 18;
        const int8_t *a = qs_a + (size_t)b * 32;
        for (int c = 0; c < 8; ++c) {
            const int hi = c >> 2;
            int32_t s = 0;
            for (int j = 0; j < 4; ++j) {
                const int i = 4 * (c & 3) + j;
                const unsigned nib = hi ? (blk[2 + i] >> 4) : (blk[2 + i] & 15u);
                s += (int)a[16 * hi + i] * (int)k_iq4nl[nib];
            }
            p[c] = s;
            if (partials) partials[b * 8 + c] = s;
        }
        if (b < paired) {
            const float d = half_at(blk) * wdo_f16_to_f32(d_a[b]);
            for (int c = 0; c < 8; ++c) acc[b & 1][c] = fmaf(d, (float)p[c], acc[b & 1][c]);
        }
    }
    float lane[8];
    for (int c = 0; c < 8; ++c) lane[c] = acc[0][c] + acc[1][c];
    float r = close_lanes(lane);
    if (nb & 1) {
        /* trailing unpaired block (p[] still holds its chunk sums): one rounded
         * product with the whole-block integer sum, added after the tree */
        const uint8_t *blk = w + (size_t)(nb - 1) * 18;
        int total = 0;
        for (int c = 0; c < 8; ++c) total += p[c];
        r += (half_at(blk) * wdo_f16_to_f32(d_a[nb - 1])) * (float)total;
    }
    return r;
}

float wdo_row_q4_0_q8_0(const uint8_t *w, const int8_t *qs_a, const uint16_t *d_a, int cols, int32_t *partials) {
    /* value i<16 = low nibble of byte i, value i>=16 = high nibble of byte i-16, minus 8. */
    double acc = 0.0;
    for (int b = 0; b < cols / 32; ++b) {
        const uint8_t *blk = w + (size_t)b * 18;
        const int8_t *a = qs_a + (size_t)b * 32;
        int32_t s = 0;
        for (int i = 0; i < 16; ++i) {
            s += ((int)(blk[2 + i] & 15u) - 8) * (int)a[i];
            s += ((int)(blk[2 + i] >> 4) - 8) * (int)a[16 + i];
        }
        if (partials) partials[b] = s;
        acc += (double)(half_at(blk) * wdo_f16_to_f32(d_a[b]) * (float)s);
    }
    return (float)acc;
}

float wdo_row_q6_K_q8_K(const uint8_t *w, const int8_t *qs, const float *d, const int16_t *bsums, int cols, int32_t *partials) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int sb = 0; sb < cols / 256; ++sb) {
        const uint8_t *blk = w + (size_t)sb * 210;
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t *sc = (const int8_t *)(blk + 192);
        const float dw = half_at(blk + 208);
        const int8_t *a = qs + (size_t)sb * 256;
        const int16_t *bs = bsums + (size_t)sb * 16;
        const float ds = dw * d[sb];
        for (int m = 0; m < 8; ++m) {
            /* float lane m: byte positions 4m..4m+3 of each of the eight 32-value chunks */
            int32_t sumi = 0;
            for (int is = 0; is < 8; ++is) {
                const int half = is >> 2, sub = is & 3;
                const int scale = sc[2 * is + (m >> 2)];  /* low 16 bytes of the chunk: scale 2 is, high 16: 2 is + 1 */
                for (int j = 0; j < 4; ++j) {
                    const int l = 4 * m + j;
                    const unsigned qlb = ql[64 * half + ((sub & 1) ? 32 : 0) + l];
                    const unsigned qhb = qh[32 * half + l];
                    const int v = (int)((sub < 2 ? (qlb & 15u) : (qlb >> 4)) | (((qhb >> (2 * sub)) & 3u) << 4));
                    sumi += v * (int)a[32 * is + l] * scale;
                }
            }
            /* the -32 offset of the codes, folded in through the 16-value sums of the activation */
            const int32_t corr = (int32_t)((uint32_t)((int32_t)bs[2 * m] * sc[2 * m] + (int32_t)bs[2 * m + 1] * sc[2 * m + 1]) << 5);
            const int32_t lane_sum = sumi - corr;
            if (partials) partials[sb * 8 + m] = lane_sum;
            acc[m] = fmaf(ds, (float)lane_sum, acc[m]);
        }
    }
    const float r0 = acc[4] + acc[0], r1 = acc[5] + acc[1], r2 = acc[6] + acc[2], r3 = acc[7] + acc[3];
    return (r0 + r2) + (r1 + r3);
}

void wdo_gemv_q6_K(const uint8_t *w, int rows, int cols, const int8_t *qs, const float *d, const int16_t *bsums, float *out,
                   int32_t *partials) {
    const size_t rb = (size_t)(cols / 256) * 210;
    for (int r = 0; r < rows; ++r)
        out[r] = wdo_row_q6_K_q8_K(w + (size_t)r * rb, qs, d, bsums, cols, partials ? partials + (size_t)r * (cols / 256) * 8 : NULL);
}

static int partials_per_row(int type, int cols) {
    switch (type) {
        case WDO_IQ3_S:
        case WDO_IQ2_S: return cols / 256 * 8;
        case WDO_Q8_0:
        case WDO_IQ4_NL: return cols / 32 * 8;
        case WDO_Q4_0: return cols / 32;
        default: return 0;
    }
}

static float row_dot(int type, const uint8_t *w, const int8_t *qs, const void *d, int cols, int32_t *partials) {
    switch (type) {
        case WDO_IQ3_S: return wdo_row_iq3_s_q8_K(w, qs, (const float *)d, cols, partials);
        case WDO_IQ2_S: return wdo_row_iq2_s_q8_K(w, qs, (const float *)d, cols, partials);
        case WDO_Q8_0: return wdo_row_q8_0_q8_0(w, qs, (const uint16_t *)d, cols, partials);
        case WDO_IQ4_NL: return wdo_row_iq4_nl_q8_0(w, qs, (const uint16_t *)d, cols, partials);
        case WDO_Q4_0: return wdo_row_q4_0_q8_0(w, qs, (const uint16_t *)d, cols, partials);
        default: return NAN;
    }
}

void wdo_gemv(int type, const uint8_t *w, int rows, int cols, const int8_t *act_qs, const void *act_d,
              float *out, int32_t *partials) {
    const size_t rb = wdo_row_bytes(type, cols);
    const int pp = partials_per_row(type, cols);
    for (int r = 0; r < rows; ++r) {
        out[r] = row_dot(type, w + (size_t)r * rb, act_qs, act_d, cols, partials ? partials + (size_t)r * pp : NULL);
    }
}

/* ------------------------------------------------------------------------- */
/* Independent dequantiser (brute-force checks only)                          */
/* ------------------------------------------------------------------------- */
void wdo_dequant_row(int type, const uint8_t *w, int cols, float *out) {
    if (type == WDO_Q8_0) {
        for (int b = 0; b < cols / 32; ++b) {
            const uint8_t *blk = w + (size_t)b * 34;
            const float d = half_at(blk);
            for (int i = 0; i < 32; ++i) out[b * 32 + i] = d * (float)(int8_t)blk[2 + i];
        }
    } else if (type == WDO_Q4_0 || type == WDO_IQ4_NL) {
        for (int b = 0; b < cols / 32; ++b) {
            const uint8_t *blk = w + (size_t)b * 18;
            const float d = half_at(blk);
            for (int i = 0; i < 32; ++i) {
                const unsigned nib = (i < 16) ? (blk[2 + i] & 15u) : (blk[2 + i - 16] >> 4);
                const int code = (type == WDO_Q4_0) ? (int)nib - 8 : (int)k_iq4nl[nib];
                out[b * 32 + i] = d * (float)code;
            }
        }
    } else if (type == WDO_Q6_K) {
        /* value i of a super-block: half = i / 128, quarter q = (i % 128) / 32, l = i % 32; low four bits from
         * ql[64 half + 32 (q & 1) + l] (low nibble for q < 2, high for q >= 2), two high bits from
         * qh[32 half + l] >> 2q, scale sc[8 half + 2 q + l / 16]; value = d * sc * (code - 32). */
        for (int sb = 0; sb < cols / 256; ++sb) {
            const uint8_t *blk = w + (size_t)sb * 210;
            const int8_t *sc = (const int8_t *)(blk + 192);
            const float d = half_at(blk + 208);
            for (int i = 0; i < 256; ++i) {
                const int half = i >> 7, q = (i & 127) >> 5, l = i & 31;
                const unsigned lo = blk[64 * half + 32 * (q & 1) + l];
                const unsigned code = ((q < 2) ? (lo & 15u) : (lo >> 4)) | (((blk[128 + 32 * half + l] >> (2 * q)) & 3u) << 4);
                out[sb * 256 + i] = d * (float)sc[8 * half + 2 * q + (l >> 4)] * (float)((int)code - 32);
            }
        }
    } else if (type == WDO_IQ3_S) {
        const uint32_t *grid = wdo_iq3s_grid();
        for (int sb = 0; sb < cols / 256; ++sb) {
            const uint8_t *blk = w + (size_t)sb * 110;
            const float d = half_at(blk);
            for (int i = 0; i < 256; ++i) {
                /* value i: 32-block ib, quad q (0..7) inside it, element j */
                const int ib = i >> 5, q = (i >> 2) & 7, j = i & 3;
                const unsigned hb = ((unsigned)blk[66 + ib] >> q) & 1u;
                const unsigned idx = blk[2 + ib * 8 + q] | (hb << 8);
                const int mag = (int)((grid[idx] >> (8 * j)) & 0xffu);
                const unsigned sb_bit = ((unsigned)blk[74 + ib * 4 + (q >> 1)] >> (4 * (q & 1) + j)) & 1u;
                const unsigned sc = blk[106 + (ib >> 1)];
                const int ls = 1 + 2 * (int)((ib & 1) ? (sc >> 4) : (sc & 15u));
                out[sb * 256 + i] = d * (float)(ls * (sb_bit ? -mag : mag));
            }
        }
    } else if (type == WDO_IQ2_S) {
        const uint64_t *grid = wdo_iq2s_grid();
        for (int sb = 0; sb < cols / 256; ++sb) {
            const uint8_t *blk = w + (size_t)sb * 82;
            const float d = half_at(blk);
            for (int i = 0; i < 256; ++i) {
                /* value i: 32-block ib, octet o (0..3) inside it, element j (0..7) */
                const int ib = i >> 5, o = (i >> 3) & 3, j = i & 7;
                const unsigned hb = ((unsigned)blk[66 + ib] >> (2 * o)) & 3u;
                const unsigned idx = blk[2 + ib * 4 + o] | (hb << 8);
                const int mag = (int)((grid[idx] >> (8 * j)) & 0xffu);
                const unsigned sb_bit = ((unsigned)blk[34 + ib * 4 + o] >> j) & 1u;
                const unsigned sc = blk[74 + ib];
                const int ls = 1 + 2 * (int)((o < 2) ? (sc & 15u) : (sc >> 4));
                out[sb * 256 + i] = (d * 0.125f) * (float)(ls * (sb_bit ? -mag : mag));
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Transcendentals                                                           */
/* ------------------------------------------------------------------------- */
float wdo_exp_ggml(float x) {
    const float r = 0x1.8p23f;
    const float z = fmaf(x, 0x1.715476p+0f, r);
    const float n = z - r;
    const float b = fmaf(-n, 0x1.7f7d1cp-20f, fmaf(-n, 0x1.62e4p-1f, x));
    const uint32_t e = f32_bits(z) << 23;
    const float k = bits_f32(e + 0x3f800000u);
    const float u = b * b;
    const float p2 = fmaf(0x1.0e4020p-7f, b, 0x1.573e2ep-5f);
    const float p1 = fmaf(0x1.555e66p-3f, b, 0x1.fffdb6p-2f);
    const float j = fmaf(fmaf(p2, u, p1), u, 0x1.ffffecp-1f * b);
    if (fabsf(n) <= 126.0f) return fmaf(j, k, k);
    const uint32_t g = (n <= 0.0f) ? 0x82000000u : 0u;
    const float s1 = bits_f32(g + 0x7f000000u);
    if (fabsf(n) > 192.0f) return s1 * s1;
    const float s2 = bits_f32(e - g);
    return fmaf(s2, j, s2) * s1;
}

float wdo_silu_ggml(float x) { return x / (1.0f + wdo_exp_ggml(-x)); }

float wdo_sigmoid_ggml(float x) { return 1.0f / (1.0f + wdo_exp_ggml(-x)); }

/* ------------------------------------------------------------------------- */
/* Hyper-connection combine of the FFN branch (the consumer of the layer)     */
/* ------------------------------------------------------------------------- */
static const uint64_t k_exp2f_tab[32] = WD_EXP2F_TABLE;

static inline uint64_t f64_bits(double v) {
    uint64_t b;
    memcpy(&b, &v, 8);
    return b;
}
static inline double bits_f64(uint64_t b) {
    double v;
    memcpy(&v, &b, 8);
    return v;
}

/* src/qwen38_exact_math.cuh:136-166.  Every step is one rounded double operation (this file is built with
 * -ffp-contract=off). */
float wdo_expf_glibc(float x) {
    const double shift = 0x1.8p+52, invln2n = 0x1.71547652b82fep+0 * 32.0;
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0, c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0, c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const uint32_t ix = f32_bits(x), abstop = (ix >> 20) & 0x7ffu;
    if (abstop >= (0x42b00000u >> 20)) { /* |x| >= 88, infinities, NaN */
        if (ix == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8u) return x + x;
        if (x > 0x1.62e42ep6f) return 0x1p97f * 0x1p97f;
        if (x < -0x1.9fe368p6f) return 0x1p-95f * 0x1p-95f;
    }
    const double z = invln2n * (double)x;
    const double kd_shift = z + shift;
    const uint64_t ki = f64_bits(kd_shift);
    const double kd = kd_shift - shift;
    const double r = z - kd;
    const uint64_t t = k_exp2f_tab[ki % 32u] + (ki << 47);
    const double s = bits_f64(t);
    const double p = c0 * r + c1;
    const double r2 = r * r;
    double y = c2 * r + 1.0;
    y = p * r2 + y;
    y = y * s;
    return (float)y;
}

void wdo_expf_glibc_n(const float *x, int n, float *out) {
    for (int i = 0; i < n; ++i) out[i] = wdo_expf_glibc(x[i]);
}
void wdo_libm_expf_n(const float *x, int n, float *out) {
    for (int i = 0; i < n; ++i) out[i] = expf(x[i]);
}

float wdo_sigmoid_exact(float x) { return 1.0f / (1.0f + wdo_expf_glibc(-x)); }

/* src/qwen38_precision.hpp:40-55 (the host branch; the device branch is the hardware conversion) */
float wdo_round_half(float value) {
    if (!isfinite(value) || value == 0.0f) return value;
    const float magnitude = fabsf(value);
    if (magnitude >= 65520.0f) return copysignf(INFINITY, value);
    if (magnitude < ldexpf(1.0f, -14)) return copysignf(ldexpf(nearbyintf(ldexpf(magnitude, 24)), -24), value);
    const float quantum = ldexpf(1.0f, ilogbf(magnitude) - 10);
    return copysignf(nearbyintf(magnitude / quantum) * quantum, value);
}

void wdo_round_half_n(const float *x, int n, float *out) {
    for (int i = 0; i < n; ++i) out[i] = wdo_round_half(x[i]);
}

/* IEEE round-to-nearest-even float -> half bits (the device's __float2half): the rounded value is representable, so
 * the block-scale conversion above is exact on it (its flush of magnitudes below 2^-24 cannot apply). */
uint16_t wdo_f32_to_f16_rn(float value) {
    if (value != value) return 0x7e00u;
    return wdo_f32_to_f16(wdo_round_half(value));
}

/* Q8_1 activation of the reference's plain Q8_0 GEMV (q8_1_quantize_f32_kernel, src/lowbit.cuh:287-308): per block of
 * 32, d = amax / 127, q = roundf(x / d) (halves away from zero, a division - not a multiplication by the inverse),
 * scale stored as half(d). */
void wdo_quantize_q8_1(const float *x, int n, int8_t *qs, uint16_t *d) {
    for (int b = 0; b < n / 32; ++b) {
        const float *src = x + (size_t)b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(src[i]));
        const float scale = amax / 127.0f;
        for (int i = 0; i < 32; ++i) qs[(size_t)b * 32 + i] = amax == 0.0f ? 0 : (int8_t)roundf(src[i] / scale);
        d[b] = wdo_f32_to_f16_rn(scale);
    }
}

/* y[row] = sum over the row's blocks, in ascending order, of (d_w * d_x) * (float)dot32 - one rounded multiply of the
 * two scales, one of the product with the integer sum, one rounded add (q8_0_q8_1_gemv_f32_kernel,
 * src/lowbit.cuh:310-341; the reference builds with --use_fast_math, which may fuse the last two: results there are
 * defined up to that).  block_sums (optional): int32 [rows][cols / 32]. */
void wdo_gemv_q8_0_q8_1(const uint8_t *w, int rows, int cols, const int8_t *qs, const uint16_t *d, float *y, int32_t *block_sums) {
    const int nb = cols / 32;
    for (int r = 0; r < rows; ++r) {
        const uint8_t *row = w + (size_t)r * nb * 34;
        float sum = 0.0f;
        for (int b = 0; b < nb; ++b) {
            const uint8_t *blk = row + (size_t)b * 34;
            int dot = 0;
            for (int i = 0; i < 32; ++i) dot += (int)(int8_t)blk[2 + i] * (int)qs[b * 32 + i];
            if (block_sums) block_sums[(size_t)r * nb + b] = dot;
            const float scale = half_at(blk) * wdo_f16_to_f32(d[b]);
            const float prod = scale * (float)dot;
            sum = sum + prod;
        }
        y[r] = sum;
    }
}

/* Q8_0 activation from half input (q8_0_quantize_half_kernel, src/warodecode.cu:1504-1520): the values widened to
 * float, inv = 127 / amax, q = lrintf(v * inv) clamped to +-127, scale = half(amax / 127) by IEEE rounding. */
void wdo_quantize_q8_0_f16(const uint16_t *x, int n, int8_t *qs, uint16_t *d) {
    for (int b = 0; b < n / 32; ++b) {
        float v[32], amax = 0.0f;
        for (int i = 0; i < 32; ++i) {
            v[i] = wdo_f16_to_f32(x[(size_t)b * 32 + i]);
            amax = fmaxf(amax, fabsf(v[i]));
        }
        const float inv = amax == 0.0f ? 0.0f : 127.0f / amax;
        for (int i = 0; i < 32; ++i) {
            long q = lrintf(v[i] * inv);
            if (q > 127) q = 127;
            if (q < -127) q = -127;
            qs[(size_t)b * 32 + i] = (int8_t)q;
        }
        d[b] = wdo_f32_to_f16_rn(amax / 127.0f);
    }
}

float wdo_moe_branch_f32(float routed, float shared, float gate) {
    const float weighted = shared * gate;
    return routed + weighted;
}
float wdo_residual_add_f32(float residual, float branch, float weight) {
    const float weighted = branch * weight;
    return residual + weighted;
}

static float hc_weight(float inject, int hc) { return 2.0f * wdo_sigmoid_exact(inject * (1.0f / (float)hc)); }

void wdo_hc_combine_f32(float *residual, const float *block_out, const float *inject, int hidden, int hc, int round_half) {
    for (int c = 0; c < hc; ++c) {
        const float w = hc_weight(inject[c], hc);
        for (int h = 0; h < hidden; ++h) {
            const float v = wdo_residual_add_f32(residual[(size_t)c * hidden + h], block_out[h], w);
            residual[(size_t)c * hidden + h] = round_half ? wdo_round_half(v) : v;
        }
    }
}

void wdo_hc_combine_moe_f32(float *residual, const float *routed, const void *shared, int shared_is_half, const float *shared_gate,
                            const float *inject, int hidden, int hc, int round_half) {
    for (int c = 0; c < hc; ++c) {
        const float w = hc_weight(inject[c], hc);
        for (int h = 0; h < hidden; ++h) {
            const float sh = shared_is_half ? wdo_f16_to_f32(((const uint16_t *)shared)[h]) : ((const float *)shared)[h];
            const float branch = wdo_moe_branch_f32(routed[h], sh, shared_gate[0]);
            const float v = wdo_residual_add_f32(residual[(size_t)c * hidden + h], branch, w);
            residual[(size_t)c * hidden + h] = round_half ? wdo_round_half(v) : v;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* F32 dot in the 4 x 8 accumulator order                                     */
/* ------------------------------------------------------------------------- */
float wdo_dot_f32(const float *a, const float *b, int n) {
    float s[32];
    for (int t = 0; t < 32; ++t) s[t] = 0.0f;
    const int np = n & ~31;
    for (int i = 0; i < np; i += 32) {
        for (int t = 0; t < 32; ++t) s[t] = fmaf(a[i + t], b[i + t], s[t]);
    }
    /* fold accumulators 2->0, 3->1, then 1->0 (accumulator j holds s[8j..8j+7]) */
    for (int l = 0; l < 8; ++l) {
        s[l] = s[l] + s[16 + l];
        s[8 + l] = s[8 + l] + s[24 + l];
    }
    for (int l = 0; l < 8; ++l) s[l] = s[l] + s[8 + l];
    const float t0 = s[0] + s[4], t1 = s[1] + s[5], t2 = s[2] + s[6], t3 = s[3] + s[7];
    float acc = (t0 + t1) + (t2 + t3);
    for (int c = np; c < n; ++c) acc = acc + a[c] * b[c];
    return acc;
}

void wdo_router_logits(const float *w, const float *x, int rows, int cols, float *logits) {
    for (int r = 0; r < rows; ++r) logits[r] = wdo_dot_f32(w + (size_t)r * cols, x, cols);
}

/* ------------------------------------------------------------------------- */
/* Router chain                                                              */
/* ------------------------------------------------------------------------- */
void wdo_softmax_row(const float *logits, int n, float *probs) {
    float mx = -INFINITY;
    for (int e = 0; e < n; ++e) mx = fmaxf(mx, logits[e]);
    double sum = 0.0;
    int i = 0;
    for (; i + 8 <= n; i += 8) {
        float v[8];
        for (int j = 0; j < 8; ++j) {
            v[j] = wdo_exp_ggml(logits[i + j] - mx);
            probs[i + j] = v[j];
        }
        const float lo = v[0] + v[4], lh = v[2] + v[6], hi = v[1] + v[5], hh = v[3] + v[7];
        sum += (double)((lo + lh) + (hi + hh));
    }
    for (; i < n; ++i) {
        probs[i] = wdo_exp_ggml(logits[i] - mx);
        sum += (double)probs[i];
    }
    if (sum == 0.0) {
        for (int e = 0; e < n; ++e) probs[e] = -INFINITY;
        return;
    }
    const float inv = (float)(1.0 / sum);
    for (int e = 0; e < n; ++e) probs[e] = probs[e] * inv;
}

void wdo_router_select(const float *probs, int n, int k, float w_scale, int *ids, float *weights) {
    float top[64];
    if (k > 64) k = 64;
    for (int j = 0; j < k; ++j) {
        float best = -INFINITY;
        int best_id = 0;
        for (int e = 0; e < n; ++e) {
            if (!(probs[e] > best)) continue;
            int taken = 0;
            for (int m = 0; m < j; ++m) taken |= (ids[m] == e);
            if (!taken) {
                best = probs[e];
                best_id = e;
            }
        }
        ids[j] = best_id;
        top[j] = probs[best_id];
    }
    double wsum = 0.0;
    for (int j = 0; j < k; ++j) wsum += (double)top[j];
    const float denom = fmaxf((float)wsum, 6.103515625e-5f);
    for (int j = 0; j < k; ++j) weights[j] = top[j] / denom;
    if (w_scale != 0.0f && w_scale != 1.0f) {
        for (int j = 0; j < k; ++j) weights[j] = weights[j] * w_scale;
    }
}

/* ------------------------------------------------------------------------- */
/* Expert chain and layer                                                    */
/* ------------------------------------------------------------------------- */
static int act_is_q8k(int type) { return type == WDO_IQ3_S || type == WDO_IQ2_S; }

typedef struct {
    /* quantised layer input, both flavours (filled on demand) */
    int8_t *xk_qs;
    float *xk_d;
    int16_t *xk_bs;
    int8_t *x0_qs;
    uint16_t *x0_d;
} xq_t;

static void expert_ffn_q(int gate_type, int up_type, int down_type, const uint8_t *gate, const uint8_t *up,
                         const uint8_t *down, int H, int F, const xq_t *xq, float *out, float *gate_up,
                         float *act, int8_t *act_qs, uint16_t *act_d, int32_t *gup, int32_t *dp) {
    float *gu = gate_up ? gate_up : (float *)malloc(sizeof(float) * 2 * (size_t)F);
    float *ac = act ? act : (float *)malloc(sizeof(float) * (size_t)F);
    int8_t *aq = act_qs ? act_qs : (int8_t *)malloc((size_t)F);
    uint16_t *ad = act_d ? act_d : (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(F / 32));
    const int ppg = partials_per_row(gate_type, H);
    wdo_gemv(gate_type, gate, F, H, act_is_q8k(gate_type) ? xq->xk_qs : xq->x0_qs,
             act_is_q8k(gate_type) ? (const void *)xq->xk_d : (const void *)xq->x0_d, gu, gup);
    wdo_gemv(up_type, up, F, H, act_is_q8k(up_type) ? xq->xk_qs : xq->x0_qs,
             act_is_q8k(up_type) ? (const void *)xq->xk_d : (const void *)xq->x0_d, gu + F,
             gup ? gup + (size_t)F * ppg : NULL);
    for (int r = 0; r < F; ++r) ac[r] = wdo_silu_ggml(gu[r]) * gu[F + r];
    wdo_quantize_q8_0(ac, F, aq, ad);
    wdo_gemv(down_type, down, H, F, aq, ad, out, dp);
    if (!gate_up) free(gu);
    if (!act) free(ac);
    if (!act_qs) free(aq);
    if (!act_d) free(ad);
}

static void xq_make(xq_t *q, const float *x, int H, int need_k, int need_0) {
    memset(q, 0, sizeof(*q));
    if (need_k) {
        q->xk_qs = (int8_t *)malloc((size_t)H);
        q->xk_d = (float *)malloc(sizeof(float) * (size_t)(H / 256));
        q->xk_bs = (int16_t *)malloc(sizeof(int16_t) * (size_t)(H / 16));
        wdo_quantize_q8_K(x, H, q->xk_qs, q->xk_d, q->xk_bs);
    }
    if (need_0) {
        q->x0_qs = (int8_t *)malloc((size_t)H);
        q->x0_d = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(H / 32));
        wdo_quantize_q8_0(x, H, q->x0_qs, q->x0_d);
    }
}

static void xq_free(xq_t *q) {
    free(q->xk_qs);
    free(q->xk_d);
    free(q->xk_bs);
    free(q->x0_qs);
    free(q->x0_d);
}

void wdo_expert_ffn(int gate_type, int up_type, int down_type, const uint8_t *gate, const uint8_t *up,
                    const uint8_t *down, int hidden, int ffn, const float *x, float *out, float *gate_up,
                    float *act, int8_t *act_qs, uint16_t *act_d, int32_t *gate_up_partials,
                    int32_t *down_partials) {
    xq_t xq;
    const int need_k = act_is_q8k(gate_type) || act_is_q8k(up_type);
    const int need_0 = !act_is_q8k(gate_type) || !act_is_q8k(up_type);
    xq_make(&xq, x, hidden, need_k, need_0);
    expert_ffn_q(gate_type, up_type, down_type, gate, up, down, hidden, ffn, &xq, out, gate_up, act, act_qs, act_d,
                 gate_up_partials, down_partials);
    xq_free(&xq);
}

typedef struct {
    const wdo_layer *L;
    const xq_t *xq;
    wdo_dump *dump;
    const int *ids;
    float *expert_out; /* [k][H] */
    float *shared_out; /* [H] */
    int n_tasks;       /* k (+1 when a shared expert exists) */
    int next;
    pthread_mutex_t mu;
} layer_job;

static void run_task(layer_job *job, int t) {
    const wdo_layer *L = job->L;
    const int H = L->hidden, F = L->expert_ffn, k = L->top_k;
    wdo_dump *dp = job->dump;
    if (t < k) {
        const int e = job->ids[t];
        const size_t gs = (size_t)F * wdo_row_bytes(L->gate_type, H);
        const size_t us = (size_t)F * wdo_row_bytes(L->up_type, H);
        const size_t ds = (size_t)H * wdo_row_bytes(L->down_type, F);
        const int ppg = partials_per_row(L->gate_type, H);
        const int ppd = partials_per_row(L->down_type, F);
        expert_ffn_q(L->gate_type, L->up_type, L->down_type, L->gate + gs * (size_t)e, L->up + us * (size_t)e,
                     L->down + ds * (size_t)e, H, F, job->xq, job->expert_out + (size_t)t * H,
                     dp && dp->gate_up ? dp->gate_up + (size_t)t * 2 * F : NULL,
                     dp && dp->act ? dp->act + (size_t)t * F : NULL,
                     dp && dp->act_qs ? dp->act_qs + (size_t)t * F : NULL,
                     dp && dp->act_d ? dp->act_d + (size_t)t * (F / 32) : NULL,
                     dp && dp->gate_up_partials ? dp->gate_up_partials + (size_t)t * 2 * F * ppg : NULL,
                     dp && dp->down_partials ? dp->down_partials + (size_t)t * H * ppd : NULL);
    } else {
        expert_ffn_q(L->shared_type, L->shared_type, L->shared_type, L->shared_gate, L->shared_up, L->shared_down, H,
                     F, job->xq, job->shared_out, NULL, NULL, NULL, NULL, NULL, NULL);
    }
}

static void *worker(void *arg) {
    layer_job *job = (layer_job *)arg;
    for (;;) {
        pthread_mutex_lock(&job->mu);
        const int t = job->next++;
        pthread_mutex_unlock(&job->mu);
        if (t >= job->n_tasks) break;
        run_task(job, t);
    }
    return NULL;
}

void wdo_moe_layer_mt(const wdo_layer *L, const float *x, float *out, wdo_dump *dump, int preselected,
                      int threads) {
    const int H = L->hidden, E = L->n_experts, k = L->top_k;
    const int has_shared = L->shared_gate_inp != NULL;
    int *ids = (int *)malloc(sizeof(int) * (size_t)k);
    float *wts = (float *)malloc(sizeof(float) * (size_t)k);
    if (preselected) {
        memcpy(ids, dump->ids, sizeof(int) * (size_t)k);
        memcpy(wts, dump->weights, sizeof(float) * (size_t)k);
    } else {
        float *logits = (float *)malloc(sizeof(float) * (size_t)E);
        float *probs = (float *)malloc(sizeof(float) * (size_t)E);
        wdo_router_logits(L->router, x, E, H, logits);
        wdo_softmax_row(logits, E, probs);
        wdo_router_select(probs, E, k, L->w_scale, ids, wts);
        if (dump && dump->logits) memcpy(dump->logits, logits, sizeof(float) * (size_t)E);
        if (dump && dump->ids) memcpy(dump->ids, ids, sizeof(int) * (size_t)k);
        if (dump && dump->weights) memcpy(dump->weights, wts, sizeof(float) * (size_t)k);
        free(logits);
        free(probs);
    }

    xq_t xq;
    const int any_k = act_is_q8k(L->gate_type) || act_is_q8k(L->up_type);
    const int any_0 = !act_is_q8k(L->gate_type) || !act_is_q8k(L->up_type) || has_shared;
    xq_make(&xq, x, H, any_k, any_0);

    layer_job job;
    job.L = L;
    job.xq = &xq;
    job.dump = dump;
    job.ids = ids;
    job.expert_out = (dump && dump->expert_out) ? dump->expert_out : (float *)malloc(sizeof(float) * (size_t)k * H);
    job.shared_out = (dump && dump->shared_out) ? dump->shared_out : (float *)malloc(sizeof(float) * (size_t)H);
    job.n_tasks = k + (has_shared ? 1 : 0);
    job.next = 0;
    pthread_mutex_init(&job.mu, NULL);
    if (threads <= 1) {
        for (int t = 0; t < job.n_tasks; ++t) run_task(&job, t);
    } else {
        if (threads > 64) threads = 64;
        pthread_t th[64];
        for (int i = 1; i < threads; ++i) pthread_create(&th[i], NULL, worker, &job);
        worker(&job);
        for (int i = 1; i < threads; ++i) pthread_join(th[i], NULL);
    }
    pthread_mutex_destroy(&job.mu);

    /* ordered combine: product rounded, then sum rounded, top-k order */
    for (int i = 0; i < H; ++i) out[i] = 0.0f;
    for (int j = 0; j < k; ++j) {
        const float *src = job.expert_out + (size_t)j * H;
        const float wj = wts[j];
        for (int i = 0; i < H; ++i) {
            const float prod = src[i] * wj;
            out[i] = out[i] + prod;
        }
    }
    if (dump && dump->routed) memcpy(dump->routed, out, sizeof(float) * (size_t)H);
    if (has_shared) {
        const float g = wdo_sigmoid_ggml(wdo_dot_f32(L->shared_gate_inp, x, H));
        if (dump && dump->shared_gate) *dump->shared_gate = g;
        for (int i = 0; i < H; ++i) {
            const float prod = job.shared_out[i] * g;
            out[i] = out[i] + prod;
        }
    }
    if (!(dump && dump->expert_out)) free(job.expert_out);
    if (!(dump && dump->shared_out)) free(job.shared_out);
    xq_free(&xq);
    free(ids);
    free(wts);
}

void wdo_moe_layer(const wdo_layer *L, const float *x, float *out, wdo_dump *dump, int preselected) {
    wdo_moe_layer_mt(L, x, out, dump, preselected, 1);
}
