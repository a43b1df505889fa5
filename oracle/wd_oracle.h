/*
 * CPU oracle for the batch=1 MoE decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the arithmetic of the reference CPU MoE path
 * (src/qwen38_cpu_moe.cuh) and of the router chain (src/qwen38_moe.cuh:711-818).
 * Nothing in the shipped library links, loads or calls this file: it exists so
 * that the tests, the smoke check and the benchmark's cpu_baseline leg have an
 * independent answer to compare the HIP kernels against.
 *
 * Pinning status of every function is listed at the top of wd_oracle.c.
 *
 * Activation buffers are structure-of-arrays (quants, scales, block sums in
 * separate arrays); the reference CPU code uses array-of-structures blocks with
 * the same values.
 */
#ifndef WD_ORACLE_H
#define WD_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGML tensor type ids used on this path (src/gguf.hpp:26-44). */
enum {
    WDO_F32 = 0,
    WDO_Q4_0 = 2,
    WDO_Q8_0 = 8,
    WDO_Q6_K = 14,
    WDO_IQ4_NL = 20,
    WDO_IQ3_S = 21,
    WDO_IQ2_S = 22,
};

/* Expanded codebooks (ggml iq3s_grid / iq2s_grid). */
const uint32_t *wdo_iq3s_grid(void);
const uint64_t *wdo_iq2s_grid(void);

/* Block geometry (src/gguf.hpp:289-307, src/qwen38_cpu_moe.cuh:62-69). */
int wdo_block_elems(int type);
size_t wdo_block_bytes(int type);
size_t wdo_row_bytes(int type, int cols);

/* src/qwen38_cpu_moe.cuh:77-137 */
float wdo_f16_to_f32(uint16_t bits);
uint16_t wdo_f32_to_f16(float value);

/* src/qwen38_cpu_moe.cuh:220-263.  n is a multiple of 32 / 256. */
void wdo_quantize_q8_0(const float *x, int n, int8_t *qs, uint16_t *d);
void wdo_quantize_q8_K(const float *x, int n, int8_t *qs, float *d, int16_t *bsums);
/* The reference's plain Q8_0 x Q8_1 path (src/lowbit.cuh:287-362) and its half-input Q8_0 quantiser
 * (src/warodecode.cu:1504-1520); wdo_f32_to_f16_rn is IEEE round-to-nearest-even (the device's __float2half). */
uint16_t wdo_f32_to_f16_rn(float value);
void wdo_quantize_q8_1(const float *x, int n, int8_t *qs, uint16_t *d);
void wdo_gemv_q8_0_q8_1(const uint8_t *w, int rows, int cols, const int8_t *qs, const uint16_t *d, float *y, int32_t *block_sums);
void wdo_quantize_q8_0_f16(const uint16_t *x, int n, int8_t *qs, uint16_t *d);

/*
 * Row dots.  `partials` (may be NULL) receives the exact int32 chunk sums:
 *   IQ3_S / IQ2_S x Q8_K : [cols/256][8]   one per (super-block, chunk lane)
 *   Q8_0 / IQ4_NL x Q8_0 : [cols/32][8]    one per (block, chunk lane)
 *   Q4_0 x Q8_0          : [cols/32]       one per block
 * src/qwen38_cpu_moe.cuh:298-440 (scalar twins), :565-758 (AVX2).
 */
float wdo_row_iq3_s_q8_K(const uint8_t *w, const int8_t *qs, const float *d, int cols, int32_t *partials);
float wdo_row_iq2_s_q8_K(const uint8_t *w, const int8_t *qs, const float *d, int cols, int32_t *partials);
float wdo_row_q8_0_q8_0(const uint8_t *w, const int8_t *qs, const uint16_t *d, int cols, int32_t *partials);
float wdo_row_iq4_nl_q8_0(const uint8_t *w, const int8_t *qs, const uint16_t *d, int cols, int32_t *partials);
/* src/warodecode.cu:1534-1562 (dense Q4_0 x Q8 activation; float order is not canonical there). */
float wdo_row_q4_0_q8_0(const uint8_t *w, const int8_t *qs, const uint16_t *d, int cols, int32_t *partials);
/* Q6_K x Q8_K row of the output head, src/lowbit.cuh:2510-2612 (the warp form of ggml's AVX2
 * ggml_vec_dot_q6_K_q8_K): eight float lanes, lane m = bytes 4m..4m+3 of every 32-value chunk; partials [cols/256][8] =
 * integer lane sums after the -32 correction.  PARITY UNPINNED for the float order (see wd_oracle.c). */
float wdo_row_q6_K_q8_K(const uint8_t *w, const int8_t *qs, const float *d, const int16_t *bsums, int cols, int32_t *partials);
void wdo_gemv_q6_K(const uint8_t *w, int rows, int cols, const int8_t *qs, const float *d, const int16_t *bsums, float *out,
                   int32_t *partials);

/*
 * Matrix x quantised activation.  `act_d` is float* for Q8_K consumers
 * (IQ3_S, IQ2_S) and uint16_t* (fp16 bits) for Q8_0 consumers.
 * `partials` may be NULL; otherwise rows * (per-row partial count) int32.
 */
void wdo_gemv(int type, const uint8_t *w, int rows, int cols, const int8_t *act_qs, const void *act_d,
              float *out, int32_t *partials);

/* Dequantise one row to f32 (value = scale * code).  Independent decoder used by the
 * brute-force checks; src/ggml_dequant.hpp:184-194 for Q4_0/Q8_0. */
void wdo_dequant_row(int type, const uint8_t *w, int cols, float *out);

/* src/qwen38_cpu_moe.cuh:816-842 */
float wdo_exp_ggml(float x);
float wdo_silu_ggml(float x);
float wdo_sigmoid_ggml(float x);

/* The consumer of the layer's output: the hyper-connection combine of the FFN branch.
 * wdo_expf_glibc: glibc's expf (table of 2^(i/32), cubic in double, no fused operations), the routine the reference
 * ports to the device in src/qwen38_exact_math.cuh:136-166; wdo_sigmoid_exact: 1 / (1 + expf(-x)), :195-198.
 * wdo_round_half: IEEE float -> half -> float, src/qwen38_precision.hpp:40-55.
 * wdo_moe_branch_f32 / wdo_residual_add_f32: one rounded multiply and one rounded add each, src/qwen38_precision.hpp:32-38.
 * wdo_hc_combine_f32: residual[c][h] += block_out[h] * (2 * sigmoid(inject[c] * (1 / hc))) for the hc residual streams,
 * src/qwen38_hc.cuh:2530-2547; wdo_hc_combine_moe_f32 takes the branch apart as routed + shared * gate, :2241-2263
 * (shared_is_half: the shared expert's output is given as half bits, as the reference holds it, else as float). */
float wdo_expf_glibc(float x);
void wdo_expf_glibc_n(const float *x, int n, float *out);  /* the same over an array */
void wdo_libm_expf_n(const float *x, int n, float *out);   /* the host C library's expf, for the pin tests */
float wdo_sigmoid_exact(float x);
void wdo_round_half_n(const float *x, int n, float *out);
float wdo_round_half(float value);
float wdo_moe_branch_f32(float routed, float shared, float gate);
float wdo_residual_add_f32(float residual, float branch, float weight);
void wdo_hc_combine_f32(float *residual, const float *block_out, const float *inject, int hidden, int hc, int round_half);
void wdo_hc_combine_moe_f32(float *residual, const float *routed, const void *shared, int shared_is_half, const float *shared_gate,
                            const float *inject, int hidden, int hc, int round_half);

/* src/qwen38_cpu_moe.cuh:847-871 */
float wdo_dot_f32(const float *a, const float *b, int n);

/* logits[r] = dot_f32(w + r*cols, x).  src/qwen38_moe.cuh:198-245 computes the same value. */
void wdo_router_logits(const float *w, const float *x, int rows, int cols, float *logits);

/* src/qwen38_moe.cuh:711-749 and :765-818 */
void wdo_softmax_row(const float *logits, int n, float *probs);
void wdo_router_select(const float *probs, int n, int k, float w_scale, int *ids, float *weights);

/* One MoE layer description (host pointers). */
typedef struct {
    int hidden;        /* H */
    int expert_ffn;    /* F */
    int n_experts;     /* E */
    int top_k;         /* k */
    float w_scale;     /* expert weight scale, 1.0 = none */
    const float *router;          /* f32 [E][H] */
    int gate_type, up_type, down_type;
    const uint8_t *gate;          /* [E][F][row_bytes(H)] */
    const uint8_t *up;            /* [E][F][row_bytes(H)] */
    const uint8_t *down;          /* [E][H][row_bytes(F)] */
    /* optional shared expert (NULL shared_gate_inp = none); Q8_0 weights */
    const float *shared_gate_inp; /* f32 [H] */
    int shared_type;              /* WDO_Q8_0 */
    const uint8_t *shared_gate;   /* [F][row_bytes(H)] */
    const uint8_t *shared_up;
    const uint8_t *shared_down;   /* [H][row_bytes(F)] */
} wdo_layer;

/* Optional dumps of intermediates for parity checks (any pointer may be NULL). */
typedef struct {
    float *logits;        /* [E] */
    int *ids;             /* [k] */
    float *weights;       /* [k] */
    float *gate_up;       /* [k][2][F]  gate then up per selected expert */
    float *act;           /* [k][F]     silu(gate)*up */
    int8_t *act_qs;       /* [k][F]     Q8_0 of act */
    uint16_t *act_d;      /* [k][F/32] */
    float *expert_out;    /* [k][H] */
    float *routed;        /* [H] weighted sum of routed experts */
    float *shared_out;    /* [H] */
    float *shared_gate;   /* [1] sigmoid gate */
    int32_t *gate_up_partials; /* [k][2][F][per-row partial count for gate type] */
    int32_t *down_partials;    /* [k][H][F/32][8] */
} wdo_dump;

/*
 * One expert FFN on a f32 input: quantise x for the gate/up type, gate/up row
 * dots, silu(g)*u, Q8_0 requantise, down row dots.
 * src/qwen38_cpu_moe.cuh:1169-1217 (routed experts) and
 * src/qwen38_moe.cuh:3852-3891 (shared expert chain, Q8_0 weights).
 * gate_up / act / act_qs / act_d / partial pointers may be NULL.
 */
void wdo_expert_ffn(int gate_type, int up_type, int down_type, const uint8_t *gate, const uint8_t *up,
                    const uint8_t *down, int hidden, int ffn, const float *x, float *out, float *gate_up,
                    float *act, int8_t *act_qs, uint16_t *act_d, int32_t *gate_up_partials,
                    int32_t *down_partials);

/*
 * Whole layer: router -> top-k -> experts -> ordered weighted sum -> + shared * gate.
 * If preselected != 0, ids/weights are taken from dump->ids / dump->weights
 * instead of the router (the reference's `preselected` flag,
 * src/qwen38_moe.cuh:3650-3663).  out is f32 [H].
 * src/qwen38_cpu_moe.cuh:1245-1291, src/qwen38_precision.hpp:32-34.
 */
void wdo_moe_layer(const wdo_layer *layer, const float *x, float *out, wdo_dump *dump, int preselected);

/* Same, with the k expert FFNs (and the shared expert) spread over `threads` pthreads.
 * Results are bit-identical to wdo_moe_layer.  Used by the CPU baseline timer. */
void wdo_moe_layer_mt(const wdo_layer *layer, const float *x, float *out, wdo_dump *dump, int preselected,
                      int threads);

#ifdef __cplusplus
}
#endif
#endif
