/*
 * warpdecode_amd — C ABI of the MI355X (gfx950) batch=1 MoE decode path.
 *
 * Plain C: pointers and sizes only.  Every pointer named `d_*` or documented as
 * "device" is HBM memory of the current HIP device; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  Every function returns 0 on
 * success and a negative wd_status otherwise; wd_last_error() gives the text.
 * Nothing here allocates device memory except the functions that say so.
 *
 * The reference engine has no C ABI of its own: its operator surface is a set of
 * inline C++ launchers and RAII classes (namespace wd).  Each entry point below
 * cites the reference launcher it replaces; host/wd_ops.hpp in this repository
 * re-creates those C++ names on top of this ABI.
 */
#ifndef WARPDECODE_AMD_H
#define WARPDECODE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    WD_OK = 0,
    WD_ERR_ARG = -1,      /* geometry / type / null-pointer error (reference: std::runtime_error) */
    WD_ERR_HIP = -2,      /* a HIP runtime call failed */
    WD_ERR_STATE = -3,    /* object used before initialisation / after destruction */
    WD_ERR_UNSUPPORTED = -4
} wd_status;

/* GGML tensor type ids (reference: src/gguf.hpp:26-44). */
typedef enum {
    WD_TYPE_F32 = 0,
    WD_TYPE_F16 = 1,
    WD_TYPE_Q4_0 = 2,
    WD_TYPE_Q8_0 = 8,
    WD_TYPE_Q6_K = 14,
    WD_TYPE_IQ4_NL = 20,
    WD_TYPE_IQ3_S = 21,
    WD_TYPE_IQ2_S = 22
} wd_type;

/* ---- library ------------------------------------------------------------- */
const char *wd_last_error(void);
/* Selects the device, checks it is gfx950-class and uploads the codebooks. */
int wd_init(int device);
/* Bytes of one row / of a whole [rows][cols] tensor of `type` (reference: TensorInfo::byte_size,
 * src/gguf.hpp:276-310).  0 for an unsupported type or a column count that is not whole blocks. */
size_t wd_row_bytes(int type, int cols);
size_t wd_tensor_bytes(int type, int rows, int cols);

/* ---- thin runtime helpers (reference: cudaMalloc / cudaMallocHost / cudaMemcpyAsync /
 *      stream and event calls made inline by src/lowbit.cuh, src/expert_cache.cuh) ---------- */
int wd_malloc(void **d_ptr, size_t bytes);
int wd_free(void *d_ptr);
int wd_malloc_host(void **h_ptr, size_t bytes);   /* pinned */
int wd_free_host(void *h_ptr);
int wd_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes, void *stream); /* async when stream != NULL */
int wd_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes, void *stream);
int wd_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes, void *stream);
int wd_memset(void *d_dst, int value, size_t bytes, void *stream);
int wd_stream_create(void **stream);
int wd_stream_destroy(void *stream);
int wd_stream_sync(void *stream);
int wd_device_sync(void);

/* ---- activation quantisers -------------------------------------------------
 * Q8_K: 256-value blocks, int8 quants, f32 scale (always negative), int16 sums of 16.
 *   reference: launch_q8_k_quantize_f32, src/lowbit.cuh:873-891; CPU quantize_q8_K,
 *   src/qwen38_cpu_moe.cuh:239-263.  elements % 256 == 0.
 * Q8_0: 32-value blocks, int8 quants, fp16 scale.
 *   reference: q38_moe_quantize_activation_q8_0, src/qwen38_moe.cuh:1470-1481 and
 *   q38_hc_q8_0_quantize_f32_exact_kernel, src/qwen38_hc.cuh:368-392; CPU quantize_q8_0,
 *   src/qwen38_cpu_moe.cuh:220-237.  elements % 32 == 0.  Also the activation format of the dense
 *   Q4_0 path (reference: q8_0_quantize_half_kernel, src/warodecode.cu:1504-1520). */
int wd_q8_k_quantize_f32(const float *d_x, int elements, int8_t *d_qs, float *d_scales, int16_t *d_bsums,
                         void *stream);
int wd_q8_0_quantize_f32(const float *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream);
/* The same from half input, as the dense Q4_0 path quantises its activations (values widened to float, inv = 127 / amax,
 * q = lrintf(v * inv) clamped to +-127, scale = half(amax / 127) by IEEE rounding).
 *   reference: q8_0_quantize_half_kernel, src/warodecode.cu:1504-1520.  d_x: half bits, 8-byte aligned. */
int wd_q8_0_quantize_f16(const uint16_t *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream);
/* Q8_1 activation of the reference's plain Q8_0 GEMV: d = amax / 127, q = roundf(x / d), scale = half(d).
 *   reference: q8_1_quantize_f32_kernel, src/lowbit.cuh:287-308 (buffer: Q8_1Buffer, :251-285). */
int wd_q8_1_quantize_f32(const float *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream);
/* y[r] = sum over the row's Q8_0 blocks in ascending order of (d_w * d_x) * (float)dot32 (three roundings per block).
 *   reference: q8_0_q8_1_gemv_f32_kernel / launch_q8_0_gemv_q8_1_f32, src/lowbit.cuh:310-362.
 * d_block_sums: NULL or int32 [rows][cols / 32], the exact integer sums. */
int wd_gemv_q8_0_q8_1_f32(const uint8_t *d_w, int rows, int cols, const int8_t *d_qs, const uint16_t *d_scales, float *d_y,
                          int32_t *d_block_sums, void *stream);
/* Element-wise half <-> float (IEEE round-to-nearest-even on the way down, the reference's __float2half / __half2float):
 * what a caller with half activations or half outputs puts around the F32 layer calls
 * (reference: q38_moe_select_experts_input<__half>, q38_finish_moe, src/qwen38_moe.cuh:2384-2453). */
int wd_convert_f16_to_f32(const uint16_t *d_src, float *d_dst, size_t n, void *stream);
int wd_convert_f32_to_f16(const float *d_src, uint16_t *d_dst, size_t n, void *stream);

/* ---- router ----------------------------------------------------------------
 * logits[r] = dot(w[r,:], x) in the 4x8-accumulator order of ggml_vec_dot_f32.
 *   reference: launch_q38_router_gemv_f32, src/qwen38_moe.cuh:247-263.  w is f32 [rows][cols]. */
int wd_router_gemv_f32(const float *d_w, const float *d_x, float *d_logits, int rows, int cols, void *stream);
/* softmax over all experts, top-k by probability (ties to the lower id), renormalise, optional scale.
 *   reference: q38_launch_topk_softmax, src/qwen38_moe.cuh:1065-1090.
 *   n_experts % 8 == 0, n_experts <= 1024, 0 < k <= 16.  ids int32[k], weights f32[k] (device). */
int wd_topk_softmax(const float *d_logits, int n_experts, int k, float expert_scale, int32_t *d_ids,
                    float *d_weights, void *stream);

/* ---- low-bit GEMV, one matrix ------------------------------------------------
 * out[r] = row_dot(w[r], activation).  w: raw GGUF block bytes, rows packed back to back.
 * `d_partials` (may be NULL) receives the exact int32 chunk sums used for parity checks:
 *   IQ3_S / IQ2_S : [rows][cols/256][8];  Q8_0 / IQ4_NL : [rows][cols/32][8];  Q4_0 : [rows][cols/32].
 * reference: launch_iq3_s_gemv_q8_k_f32 (src/lowbit.cuh:1483), launch_iq2_s_gemv_q8_k_f32 (:1181),
 *   q38_hc_launch_exact_q8_0_gemv_f32 (src/qwen38_hc.cuh:1020-1049),
 *   q4_0_q8_0_gemv_kernel via launch_q4_float (src/warodecode.cu:1534-1562, :1746-1768; the planar
 *   prepack of the reference is not needed: raw 18-byte blocks are read directly). */
/* Q6_K x Q8_K GEMV (the output head): 210-byte super-blocks of 256 six-bit codes with sixteen int8 sub-block scales;
 * the -32 offset of the codes is taken out through the activation's 16-value sums.  Eight float lanes per row (lane m =
 * bytes 4m..4m+3 of every 32-value chunk), one fma per super-block, ggml's closing tree.  d_partials (may be NULL):
 * int32 [rows][cols/256][8], the integer lane sums after the correction.
 * reference: launch_q6_k_gemv_q8_k_f32 / q6_k_q8_k_gemv_kernel, src/lowbit.cuh:2510-2636. */
int wd_gemv_q6_k_q8_k_f32(const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs, const float *d_act_scales,
                          const int16_t *d_act_bsums, float *d_out, int32_t *d_partials, void *stream);
int wd_gemv_q8_k_f32(int type, const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs,
                     const float *d_act_scales, float *d_out, int32_t *d_partials, void *stream);
int wd_gemv_q8_0_f32(int type, const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs,
                     const uint16_t *d_act_scales, float *d_out, int32_t *d_partials, void *stream);

/* Several dense GEMVs of the same row length against Q8_0 activations in one launch - `type` WD_TYPE_Q8_0 (the exact-order
 * kernel) or WD_TYPE_Q4_0: the projections a block applies to one or a few activations are each bound by their launch,
 * not by their bytes (a 2048 x 2048 Q8_0 matrix alone reaches a seventh of the device's bandwidth).  Item i computes
 * d_out[rows] = W_i (rows x cols) . activation_i exactly as wd_gemv_q8_0_f32 does for it alone - the same workgroups do
 * the same arithmetic, the results are the same bits.  `items` is host memory; items whose shape the shared kernel does
 * not take (Q8_0: rows < 8, fewer than 64 or more than 512 blocks per row, 8192 or more rows; Q4_0: rows that are not a
 * power-of-two number of 8-block groups up to 64; either: pointers not 16-byte aligned) are launched by themselves, in
 * order.  At most 16 items go into one launch; longer lists are cut.
 * reference: the call sites of q38_hc_launch_exact_q8_0_gemv_f32, one launch per projection (src/qwen38_hc.cuh:1020-1049),
 * and of launch_q4_float (src/warodecode.cu:1746-1768). */
typedef struct wd_gemv_item {
    const uint8_t *d_w;            /* rows of 34-byte (Q8_0) or 18-byte (Q4_0) blocks */
    int rows;
    const int8_t *d_act_qs;        /* the activation's Q8_0 quants [cols] and scales [cols / 32] (wd_q8_0_quantize_f32) */
    const uint16_t *d_act_scales;
    float *d_out;                  /* [rows] */
} wd_gemv_item;
int wd_gemv_q8_0_batch_f32(int type, const wd_gemv_item *items, int n_items, int cols, void *stream);

/* ---- low-bit GEMV, one dispatch over several expert matrices ------------------
 * out[e][r] for e < experts; d_w_experts is a DEVICE array of `experts` device pointers
 * (the reference's expert pointer table).  One shared activation.
 * reference: launch_iq3_s_gemv_q8_k_experts_f32 (src/lowbit.cuh:2390-2418),
 *            launch_iq2_s_gemv_q8_k_experts_f32 (:2352-2388).  experts <= 64. */
int wd_gemv_q8_k_experts_f32(int type, const uint8_t *const *d_w_experts, int experts, int rows, int cols,
                             const int8_t *d_act_qs, const float *d_act_scales, float *d_out,
                             int32_t *d_partials, void *stream);
/* Per-expert activations act[e][cols] (the down projection): reference down stage of
 * q38_moe_run_batched_experts, src/qwen38_moe.cuh:3313-3388. */
int wd_gemv_q8_0_experts_f32(int type, const uint8_t *const *d_w_experts, int experts, int rows, int cols,
                             const int8_t *d_act_qs, const uint16_t *d_act_scales, float *d_out,
                             int32_t *d_partials, void *stream);

/* ---- elementwise stages ------------------------------------------------------
 * act[e][i] = silu_ggml(gate_up[e][0][i]) * gate_up[e][1][i]
 *   reference: q38_moe_silu_scale_mul_experts_kernel, src/qwen38_moe.cuh:1240-1254. */
int wd_silu_mul_experts_f32(const float *d_gate_up, float *d_act, int ffn, int experts, void *stream);
/* accum[i] = add_rn(accum[i], mul_rn(experts[j][i], weights[j])) for j ascending.
 *   reference: q38_moe_weighted_accum_experts_f32_kernel, src/qwen38_moe.cuh:1291-1304. */
int wd_weighted_accum_experts_f32(const float *d_experts, const float *d_weights, float *d_accum, int n, int k,
                                  void *stream);
/* routed[i] = add_rn(routed[i], mul_rn(shared[i], gate[0])).
 *   reference: q38_add_shared_f32_kernel / q38_finish_moe_f32, src/qwen38_moe.cuh:1691-1699, :2442-2453. */
int wd_add_shared_f32(float *d_routed, const float *d_shared, const float *d_gate, int n, void *stream);

/* ---- whole layer ---------------------------------------------------------------
 * Device-side description of one MoE layer.  Expert e of a routed tensor lives at
 * base + e * stride (raw GGUF bytes, the layout of a 3-D GGUF expert tensor) unless
 * `slot_of_expert` is set, in which case it lives in slot slot_of_expert[e] of an
 * expert-slot pool: gate at pool + slot*slot_bytes, up at + gate_bytes, down at
 * + gate_bytes + up_bytes (reference: GpuExpertCache::views, src/expert_cache.cuh:2495-2511).
 */
typedef struct {
    int hidden, expert_ffn, n_experts, top_k;
    float expert_scale;            /* 0 or 1 = none (reference: q38_moe_router_select w_scale) */
    int gate_type, up_type, down_type;
    const float *router;           /* device f32 [n_experts][hidden] */
    const uint8_t *gate, *up, *down;          /* device bases (resident mode) */
    size_t gate_stride, up_stride, down_stride; /* bytes per expert */
    const int32_t *slot_of_expert; /* device int32 [n_experts] or NULL */
    const uint8_t *slot_pool;      /* device */
    size_t slot_bytes, slot_gate_bytes, slot_up_bytes;
    /* shared expert (Q8_0); shared_gate_inp == NULL disables it */
    const float *shared_gate_inp;  /* device f32 [hidden] */
    const uint8_t *shared_gate, *shared_up, *shared_down; /* device Q8_0 */
} wd_moe_layer;

/* Scratch for a layer pass (device memory owned by the library object). */
typedef struct wd_moe_scratch wd_moe_scratch;
int wd_moe_scratch_create(wd_moe_scratch **out, int hidden, int expert_ffn, int n_experts, int max_k);
int wd_moe_scratch_destroy(wd_moe_scratch *s);
/* 0 when every bounded wait inside the fused dispatches was satisfied so far, 1 when one ran out, 2 when a kernel
 * was asked for an expert whose entry in slot_of_expert is negative (not in the slot pool: the kernel read slot 0
 * instead); the layer's results are then invalid and the fused combine has written NaN.  -1 on error.
 * Synchronous read of one device word. */
int wd_moe_scratch_status(wd_moe_scratch *s);
/* The device word behind it (u32), for callers that copy it beside other results instead of a read of its own. */
const unsigned *wd_moe_scratch_status_word(wd_moe_scratch *s);
/* Sets the number of polls after which such a wait gives up (0 = the default, seconds of waiting) and clears the
 * status word.  For tests of the failure path: with a limit of 1 the waiting workgroups give up at once, set the
 * status and leave without touching memory; every kernel still ends normally.  Synchronous. */
int wd_moe_scratch_set_wait_limit(wd_moe_scratch *s, unsigned polls);
/* Device views, named after Qwen38MoeScratch accessors (src/qwen38_moe.cuh:1701-2150). */
float *wd_moe_scratch_logits(wd_moe_scratch *s);      /* f32 [n_experts] */
int32_t *wd_moe_scratch_ids(wd_moe_scratch *s);       /* i32 [k] */
float *wd_moe_scratch_weights(wd_moe_scratch *s);     /* f32 [k] */
float *wd_moe_scratch_gate_up(wd_moe_scratch *s);     /* f32 [k+1][2][ffn] (slot k = shared expert) */
float *wd_moe_scratch_act(wd_moe_scratch *s);         /* f32 [k+1][ffn] */
int8_t *wd_moe_scratch_act_qs(wd_moe_scratch *s);     /* i8  [k+1][ffn] */
uint16_t *wd_moe_scratch_act_scales(wd_moe_scratch *s); /* f16 [k+1][ffn/32] */
float *wd_moe_scratch_expert_out(wd_moe_scratch *s);  /* f32 [k+1][hidden] (only with keep_expert_out) */
float *wd_moe_scratch_accum(wd_moe_scratch *s);       /* f32 [hidden] routed weighted sum (d_accum) */
float *wd_moe_scratch_down_f32(wd_moe_scratch *s);    /* f32 [hidden] shared expert output (down_f32) */
float *wd_moe_scratch_shared_gate(wd_moe_scratch *s); /* f32 [1] sigmoid gate (d_shared_gate) */
int32_t *wd_moe_scratch_gate_up_partials(wd_moe_scratch *s); /* NULL until enabled */
int32_t *wd_moe_scratch_down_partials(wd_moe_scratch *s);
/* Allocates the int32 chunk-sum dumps ([k][2][ffn][P_gate] and [k][hidden][P_down]) and makes the
 * layer pass fill them: variants of the fused dispatches store them beside their results when the
 * gate/up rows are IQ3_S or IQ2_S; other layers, and WD_MOE_STAGED, take one dispatch per operator.
 * The shared expert's sums are not part of the dump.  Parity harness only. */
int wd_moe_scratch_enable_partials(wd_moe_scratch *s, int gate_type, int down_type);

/* Profiling aid: makes the fused layer dispatches record 100 MHz time stamps of workgroup `wg` and returns the
 * device buffer (NULL on failure): uint64 [3][16][8] = [dispatch][wave][point]; dispatch 0 = router and shared
 * workgroups of the merged launch (wave rows 8 and 9: begin/end and the phases of the selection), 1 = routed gate/up
 * workgroups, 2 = dispatch C.  Only the traced workgroup pays for it.
 * Counterpart of the reference's kernel profiler sites, src/qwen38_moe.cuh:296-535. */
unsigned long long *wd_moe_scratch_trace(wd_moe_scratch *s, int wg);
/* The same for the one-launch form of wd_moe_stack_f32: uint64 [12][16] = [wave][point] of workgroup `wg` in layer
 * `layer` (which wave has which role depends on the SIMDs the waves landed on; as a rule waves 0..9 are routed rungs,
 * 10 the shared expert, 11 the router row; points: 0 layer begin, 1 input seen, 2 input in LDS, 3 logit stored,
 * 4 the rung's expert known (and, without a routing trace, its gate/up rows requested), 5 activation stored,
 * 6 activations seen, 7 down rows done, 8/9 begin and end of the combine, 10 activation record pushed out, 11 gate/up
 * rows parked and down rows requested, 12 all logits gathered, 13 ids published, 14 weights published - the last three
 * in workgroup 0's router wave).  wg == -1: uint64 [512][4][16], waves 0, 9, 10 and 11 of every workgroup. */
unsigned long long *wd_moe_scratch_trace_resident(wd_moe_scratch *s, int wg, int layer);

/* flags for wd_moe_layer_f32 */
#define WD_MOE_PRESELECTED 1u      /* ids/weights already in scratch: skip the router (reference `preselected`) */
#define WD_MOE_KEEP_EXPERT_OUT 2u  /* also store the per-expert down outputs in scratch */
#define WD_MOE_STAGED 4u           /* one dispatch per stage (the operators above) instead of the fused kernels */
/* Measurement aids for the fused path: run only the named dispatch(es) of a layer.  The scratch must hold
 * the results of the dispatches left out (run the whole layer once first). */
#define WD_MOE_ONLY_A 0x10u /* router + selection + shared gate/up */
#define WD_MOE_ONLY_B 0x20u /* routed gate/up + SwiGLU */
#define WD_MOE_ONLY_C 0x40u /* down projections + combine */
#define WD_MOE_SPLIT_AB 0x100u /* router and routed gate/up as two launches instead of one with an in-dispatch hand-off */
#define WD_MOE_DRY 0x80u    /* every workgroup of the fused dispatches returns at once: the launch floor */
#define WD_MOE_PER_LAYER 0x200u /* wd_moe_stack_f32: launch every layer's dispatches instead of one resident launch for the stack */

/* One decode step of one layer: router -> top-k -> grouped gate/up -> SwiGLU -> Q8_0 ->
 * grouped down -> ordered weighted sum -> + shared * sigmoid gate.  d_out is f32 [hidden]
 * = q38_moe_branch_f32(routed, shared, gate).  The routed sum, the shared expert output and the
 * gate are left in the scratch views above, as the reference leaves them for its caller.
 * reference: run_qwen38_routed_moe_separate_f32_x (src/qwen38_moe.cuh:3650-3779) +
 *   run_qwen38_shared_expert_f32_x (:3963-3969) + q38_finish_moe_f32 (:2442-2453). */
int wd_moe_layer_f32(const wd_moe_layer *layer, const float *d_x, float *d_out, wd_moe_scratch *scratch,
                     unsigned flags, void *stream);

/* The hyper-connection combine that consumes the layer's output: residual is [hc][hidden] and stream c receives
 * branch * (2 * sigmoid(inject[c] * (1 / hc))), the sigmoid through glibc's expf, every step one rounded float operation;
 * round_half stores the sums rounded through half (the reference's legacy residual lifetime).
 * wd_hc_combine_f32: branch = block_out (the finished layer output).
 * reference: run_qwen38_hc_combine_f32_block_f32_inject, src/qwen38_hc.cuh:2530-2570.
 * wd_hc_combine_moe_f32: branch = routed + shared * shared_gate[0]; shared_is_half: d_shared holds half bits (as the
 * reference's scratch does), else floats.  reference: run_qwen38_hc_combine_moe_f32_inject, src/qwen38_hc.cuh:2241-2263, :2587-2600.
 * wd_moe_layer_hc_f32: wd_moe_layer_f32 followed by wd_hc_combine_f32 on its output, the combine folded into the layer's
 * last dispatch (no further launch).  d_residual must not be written by other work while the call runs; the layer's
 * input d_x may be computed from it beforehand.  reference sequence: src/qwen38_forward.cuh:3330-3371. */
int wd_hc_combine_f32(float *d_residual, const float *d_block_out, const float *d_inject, int hidden, int hc, int round_half,
                      void *stream);
int wd_hc_combine_moe_f32(float *d_residual, const float *d_routed, const void *d_shared, int shared_is_half,
                          const float *d_shared_gate, const float *d_inject, int hidden, int hc, int round_half, void *stream);
int wd_moe_layer_hc_f32(const wd_moe_layer *layer, const float *d_x, float *d_out, float *d_residual, const float *d_inject,
                        int hc, int round_half, wd_moe_scratch *scratch, unsigned flags, void *stream);

/* The shared expert alone: sigmoid(shared_gate_inp . x) into the scratch's shared_gate view and the Q8_0
 * gate/up -> SwiGLU -> Q8_0 -> down chain into its down_f32 view; only the shared_* fields, hidden and
 * expert_ffn of `layer` are read.  For callers that keep the reference's three calls (routed, shared,
 * finish); wd_moe_layer_f32 does all three in its fused dispatches.
 * reference: run_qwen38_shared_expert_f32_x (src/qwen38_moe.cuh:3963-3969),
 *   q38_moe_run_shared_expert_f32_input (:3915-3948). */
int wd_shared_expert_f32(const wd_moe_layer *layer, const float *d_x, wd_moe_scratch *scratch, void *stream);

/* wd_moe_layer_f32 for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the same fused dispatches, with the intermediate values in a static device array of 128 KiB instead
 * of a wd_moe_scratch object; the call allocates and frees nothing.  No counterpart in the reference.
 * Limits: hidden <= 4096, expert_ffn <= 1024, n_experts <= 1024, top_k <= 16 (larger layers are refused with
 * WD_ERR_ARG); flags 0 or WD_MOE_SPLIT_AB.  Only d_out is handed back (no views of ids, weights or partial sums).
 * Every call on a GPU uses that GPU's one array: calls that overlap on a GPU race.  If a bounded wait inside the
 * dispatches runs out, d_out is filled with NaN. */
int wd_moe_layer_noalloc_f32(const wd_moe_layer *layer, const float *d_x, float *d_out, unsigned flags, void *stream);

/* One decode step through a stack of layers: for each layer, x += residual_scale * layer(x) (the scaled
 * residual add stands in for the caller's own glue between two MoE blocks).  d_layer_out f32 [hidden] receives the last
 * layer's output.  d_ids_trace (device int32 [n_layers][top_k], may be NULL) replays a routing trace:
 * the router still runs and its weights are used, but the expert ids come from the trace.
 * `layers` is a host array.  No counterpart in the reference, whose caller loops over layers
 * (Qwen38Decoder::step, src/qwen38_forward.cuh:2923-3371).
 * Stacks of up to 64 layers of the 512-expert layer shape (hidden 2048, ffn 512, at most 512 experts, top-k <= 10,
 * IQ3_S or IQ2_S gate/up, Q8_0 down, 16-byte aligned tensors, experts addressed directly) run as ONE launch of 512
 * workgroups that stay on the device for the whole step and hand values to each other through global memory; this
 * needs a device that holds the whole grid at once (checked) and flags == 0.  Everything else, and
 * WD_MOE_PER_LAYER, takes the per-layer dispatches.  The results are the same bits either way.  The first call with
 * a given set of layers allocates and uploads their descriptors (synchronous; not under stream capture, where an
 * unseen set takes the per-layer dispatches). */
int wd_moe_stack_f32(const wd_moe_layer *layers, int n_layers, float *d_x, float *d_layer_out,
                     wd_moe_scratch *scratch, const int32_t *d_ids_trace, float residual_scale, unsigned flags,
                     void *stream);

/* M tokens through one layer; the weights of an expert selected by several tokens are read once.
 * d_x f32 [tokens][hidden], d_out f32 [tokens][hidden].  Bit-identical to `tokens` calls of
 * wd_moe_layer_f32.  tokens <= 8.  reference: Qwen38MoeTokenBatch, src/qwen38_moe.cuh:2743-3237
 * (which re-reads the weights per (token, expert) pair). */
int wd_moe_layer_tokens_f32(const wd_moe_layer *layer, const float *d_x, float *d_out, int tokens,
                            wd_moe_scratch *const *scratch_per_token, unsigned flags, void *stream);
/* The same pass over the experts a caller holds as separate views instead of tensors that contain every expert (the
 * form in which the reference's token batch receives them, one (gate, up, down) triple per acquired expert:
 * Qwen38MoeTokenBatch::set_pair_weights / run, src/qwen38_moe.cuh:2907-3109).  h_gate / h_up / h_down: host arrays of
 * n_entries (<= 128) device pointers; the ids in the scratches are entry numbers, the weights the router weights, and
 * flags must contain WD_MOE_PRESELECTED.  `layer` supplies geometry, tensor types and (optionally) the shared expert;
 * its routed tensor pointers are ignored.  IQ3_S / IQ2_S gate and up; Q8_0 down with ffn <= 512, or 16-byte aligned
 * down views with ffn 512 / 640.  The table travels through a small pinned ring owned by the first scratch (allocated
 * at first use); every expert's bytes are read once for all tokens that selected it, results are those of one pass
 * per token. */
int wd_moe_layer_tokens_pairs_f32(const wd_moe_layer *layer, const uint8_t *const *h_gate, const uint8_t *const *h_up,
                                  const uint8_t *const *h_down, int n_entries, const float *d_x, float *d_out, int tokens,
                                  wd_moe_scratch *const *scratch_per_token, unsigned flags, void *stream);

/* ---- expert-slot cache -----------------------------------------------------------
 * LRU pool of fixed-size slots in HBM, key (layer << 32 | expert); a miss copies the expert's
 * gate|up|down slices from pinned host memory with hipMemcpyAsync on a private copy stream and
 * makes `stream` wait for it.  reference: GpuExpertCache (src/expert_cache.cuh:2156-2536),
 * ExpertStagePath (:858-1583), ExpertCacheMonitor (:1592-2105). */
typedef struct wd_expert_cache wd_expert_cache;
typedef struct {
    uint64_t accesses, hits, misses, evictions, bytes_copied;
    uint64_t slots, slot_bytes, resident;
} wd_expert_cache_stats;
int wd_expert_cache_create(wd_expert_cache **out, size_t capacity_bytes, size_t gate_bytes, size_t up_bytes,
                           size_t down_bytes, int n_layers, int n_experts, int layer_partition);
int wd_expert_cache_destroy(wd_expert_cache *c);
/* Host (pinned) sources of one layer's 3-D expert tensors; strides are bytes per expert. */
int wd_expert_cache_register_layer(wd_expert_cache *c, int layer, const uint8_t *h_gate, const uint8_t *h_up,
                                   const uint8_t *h_down);
/* The same for host tensors whose experts are further apart than their size, e.g. the fused gate_up tensor of the
 * reference's target model (2 * ffn rows per expert, gate rows first: h_gate = base, h_up = base + ffn rows,
 * gate_stride = up_stride = 2 * ffn rows; src/qwen38_moe.cuh:3462-3514, GpuFusedExpertCache,
 * src/expert_cache.cuh:2546-2882).  In a wd_moe_layer the same tensor is gate = base, up = base + ffn rows with both
 * strides 2 * ffn rows. */
int wd_expert_cache_register_layer_strided(wd_expert_cache *c, int layer, const uint8_t *h_gate, const uint8_t *h_up,
                                           const uint8_t *h_down, size_t gate_stride, size_t up_stride,
                                           size_t down_stride);
/* Makes `k` experts of `layer` resident (LRU order of the ids given), updates the device slot table
 * of that layer and returns, per id, whether it was a hit.  All k slots stay valid until the next
 * acquire call on this cache.  hit_out may be NULL. */
int wd_expert_cache_acquire(wd_expert_cache *c, int layer, const int32_t *h_ids, int k, uint8_t *hit_out,
                            void *stream);
const int32_t *wd_expert_cache_slot_table(wd_expert_cache *c, int layer); /* device int32 [n_experts] */
const uint8_t *wd_expert_cache_pool(wd_expert_cache *c);
/* Host-side index: slot that holds (layer, expert) now, or -1 (reference: the `slot` of
 * ExpertDeviceWeights, src/expert_cache.cuh:2148-2154). */
long long wd_expert_cache_slot_of(wd_expert_cache *c, int layer, int expert);
int wd_expert_cache_get_stats(wd_expert_cache *c, wd_expert_cache_stats *out);
/* Counterfactual caches that see the same (layer, expert) accesses as the pool and hold keys only: what would a pool
 * of `slots` have hit under LRU (policy 0) or exact LFU (policy 1)?  Add them before the first acquire.
 * reference: ShadowLru / ShadowFreq, src/expert_cache.cuh:1592-1668. */
/* Misses are filled by one copy kernel per acquire call that reads the host tensors directly when these are pinned
 * and 16-byte aligned (default), else - or with enabled = 0 - by hipMemcpyAsync per piece.  No counterpart in the
 * reference (its fills are cudaMemcpyAsync per contiguous run, src/expert_cache.cuh:1166-1254). */
int wd_expert_cache_set_copy_kernel(wd_expert_cache *c, int enabled);
/* Read-ahead for file-backed layers when the router decides layer by layer what is needed (no trace known to the host):
 * at a layer's first acquire of a token, the experts the previous token took in this layer and the next depth - 1 ones,
 * as far as they are not resident, are read from the file by a reader thread into a ring of `slots` pinned buffers laid
 * out like a slot (0: depth * 16); an acquire that then wants one of them queues its DMA from that buffer instead of
 * reading the file itself.  A prediction that comes true puts the same bytes into the slot as the on-demand read; one
 * that does not only wastes a read.  depth 0 switches it off.  Counters: "read_ahead" in wd_expert_cache_dump_json.
 * reference: ExpertReadAhead, ExpertStagePath::note_access / post_prefetch, ExpertCacheOptions::prefetch_depth
 * (src/expert_cache.cuh:105-114, :547-824, :1094-1153). */
int wd_expert_cache_set_read_ahead(wd_expert_cache *c, int depth, int slots);
/* File-backed fills: a read-only mapping [map_base, map_base + map_bytes) of the file behind `fd` (the cache keeps its
 * own duplicate of the descriptor).  Layers whose registered host tensors lie inside the mapping and are not pinned are
 * then filled by pread() of the expert's slices into a pinned ring (`threads` readers share every expert) and one DMA per
 * miss, instead of a pageable copy from the mapping.  reference: ExpertFileMap, ExpertPreadPool and the pinned ring of
 * ExpertStagePath (src/expert_cache.cuh:204-508, :1166-1254); there the file is found through /proc/self/maps. */
int wd_expert_cache_attach_file(wd_expert_cache *c, const uint8_t *map_base, size_t map_bytes, int fd, int threads);
/* The readable file mapping of this process that holds ptr, from /proc/self/maps: [start, end) in the address space,
 * the file's path and the file offset of `start` (consecutive lines of one file that continue each other count as one).
 * wd_expert_cache_attach_mappings looks every registered host tensor up that way, opens the files it finds and attaches
 * them like wd_expert_cache_attach_file (tensors in anonymous or pinned memory are left to the other fill paths);
 * n_attached (may be NULL) receives the number of mappings attached by the call.
 * reference: ExpertFileMap::resolve, src/expert_cache.cuh:204-330. */
typedef struct wd_file_mapping {
    uint64_t start, end, file_offset;
    char path[4096];
} wd_file_mapping;
int wd_file_mapping_of(const void *ptr, wd_file_mapping *out);
int wd_expert_cache_attach_mappings(wd_expert_cache *cache, int threads, int *n_attached);
int wd_expert_cache_add_shadow(wd_expert_cache *c, int policy, size_t slots);
/* The monitor's counters as one JSON object (hit rate, bytes copied, per-layer accesses and misses, distinct pairs,
 * reuse of the previous call's experts per layer, host time spent in acquire, shadow hit rates).  Returns the length
 * needed; writes at most `cap` bytes including the terminator.  reference: ExpertCacheMonitor::dump,
 * src/expert_cache.cuh:1879-1960. */
size_t wd_expert_cache_dump_json(wd_expert_cache *c, char *buf, size_t cap);
/* Device-side timings for the dump (off by default; on, every acquire with misses records up to four events on the cache's
 * copy stream): "io_dma_stall_ms/_max_ms/_calls" - how long the copy stream waited for the last readers of the slots it
 * was about to overwrite - and "io_dma_ms/_max_ms/_calls" - how long the fills of that acquire (of that group of layers,
 * when a token is acquired ahead) then took.  Always in the dump, from host clocks: "intra_gap_ms" / "layer_gap_ms", the
 * time between an acquire's return and the next acquire of the same / of another layer, their per-token means,
 * "acquire_per_token" and "tokens" (an acquire of a lower layer than the one before begins a token).
 * reference: StagePool::harvest_timing, src/expert_cache.cuh:1395-1416; ExpertCacheMonitor::note_gap_ms, :1833-1847;
 * the dump's keys, :1908-1930. */
int wd_expert_cache_set_timing(wd_expert_cache *c, int enabled);


/* One decode step through a stack of layers whose routed experts come from `cache` (layer l of the stack is
 * layer l of the cache; the slot fields of `layers` are ignored and taken from the cache).  x is updated as in
 * wd_moe_stack_f32.  With a routing trace (host and device copies of int32 [n_layers][top_k]) the fills of the
 * next layer overlap the current layer's dispatches - or, with a pool of at least two tokens' experts and a stack of
 * the geometry wd_moe_stack_f32 runs as one launch, the whole token is acquired ahead and runs as ONE resident launch
 * that waits, layer by layer, for the fills still on their way (they run beside it on the cache's stream;
 * WD_MOE_PER_LAYER in `flags` keeps the dispatches per layer; the results are the same bits).  Without a trace each
 * layer's ids go to the host first, as in
 * the reference's loop (q38_moe_select_experts_f32_x + GpuExpertCache::acquire per selected expert,
 * src/qwen38_moe.cuh:2323-2380, :3650-3779).  Counters: wd_expert_cache_get_stats. */
int wd_moe_stack_cached_f32(const wd_moe_layer *layers, int n_layers, wd_expert_cache *cache, float *d_x,
                            float *d_layer_out, wd_moe_scratch *scratch, const int32_t *h_ids_trace,
                            const int32_t *d_ids_trace, float residual_scale, unsigned flags, void *stream);


/* ---- site profiler ---------------------------------------------------------------------------
 * Event brackets around regions of the MoE path, accumulated per decode token into device time (HIP events on the
 * bracket's stream), host time (steady clock) and their gap; one report line per site.  reference:
 * Q38MoeKernelProfiler / Q38MoeKernelScope and its sites, src/qwen38_moe.cuh:296-535.  Sites 0..23 carry the
 * reference's numbers and names; a caller brackets them exactly where the reference does, and the library brackets
 * the ones its own code covers: moe.routed_total (a layer call), moe.acquire, moe.shared, moe.finish, and - on the
 * WD_MOE_STAGED path, whose dispatches are the reference's stages - moe.router.gemv, moe.router.topk, moe.rx_quant,
 * moe.batch.gate_up, moe.batch.silu, moe.batch.q8_quant, moe.batch.down, moe.batch.accum.  Sites from
 * WD_PROFILE_FIRST_OWN_SITE on are dispatches that only exist here.  Off by default: every hook is then one load
 * and a branch.  A bracket on a stream that is being captured is not recorded and counts as dropped.  Process-wide;
 * brackets of one site must not overlap across threads. */
enum {
    WD_SITE_STAGE_TOTAL = 0, WD_SITE_ROUTED_TOTAL, WD_SITE_ROUTER, WD_SITE_ROUTER_QUANT, WD_SITE_ROUTER_GEMV,
    WD_SITE_ROUTER_TOPK, WD_SITE_ROUTER_D2H, WD_SITE_ROUTER_SYNC, WD_SITE_ACCUM_ZERO, WD_SITE_RX_QUANT,
    WD_SITE_ACQUIRE, WD_SITE_PTR_H2D, WD_SITE_BATCH_TOTAL, WD_SITE_GATE_UP_GEMV, WD_SITE_SILU,
    WD_SITE_Q8_QUANT, WD_SITE_DOWN_GEMV, WD_SITE_ACCUM, WD_SITE_CAPTURE, WD_SITE_LOOP_TOTAL,
    WD_SITE_FINISH, WD_SITE_SHARED, WD_SITE_SHARED_GATE, WD_SITE_MIRROR,
    WD_PROFILE_FIRST_OWN_SITE,
    WD_SITE_FUSED_AB = WD_PROFILE_FIRST_OWN_SITE, /* router + selection + shared and routed gate/up in one launch */
    WD_SITE_FUSED_A,        /* router + selection + shared gate/up as a launch of its own */
    WD_SITE_FUSED_B,        /* routed gate/up + SwiGLU as a launch of its own */
    WD_SITE_FUSED_C,        /* down projections + ordered combine */
    WD_SITE_STACK_TOTAL,    /* one wd_moe_stack_f32 / wd_moe_stack_cached_f32 call */
    WD_SITE_STACK_RESIDENT, /* the one-launch form of the stack */
    WD_SITE_CACHE_FILL,     /* the fills of one acquire, on the cache's copy stream */
    WD_SITE_TOKENS_TOTAL,   /* one multi-token pass */
    WD_SITE_TOKENS_A, WD_SITE_TOKENS_B, WD_SITE_TOKENS_C,
    WD_SITE_HC_COMBINE,     /* the hyper-connection combine as a launch of its own */
    WD_PROFILE_SITE_COUNT
};
typedef struct {
    unsigned long long calls;      /* brackets whose two events were read */
    unsigned long long recorded;   /* brackets that recorded both events */
    unsigned long long dropped;    /* brackets without room, on a capturing stream, or whose event record failed */
    unsigned long long unreadable; /* brackets whose elapsed time could not be read at the flush */
    double device_ms, host_ms;     /* totals over all flushed tokens */
} wd_profile_site_stat;
int wd_profile_enable(int on);                       /* the first enable creates the events */
int wd_profile_enabled(void);
int wd_profile_begin(int site, void *stream);        /* reference mark_begin; nested brackets of a site count once */
int wd_profile_end(int site, void *stream);          /* reference mark_end */
int wd_profile_flush_token(void);                    /* once per token, after the bracketed streams were synchronised */
int wd_profile_site(int site, wd_profile_site_stat *out, unsigned long long *tokens);
const char *wd_profile_site_name(int site);          /* "unknown" outside 0..WD_PROFILE_SITE_COUNT-1 */
/* The reference's summary (print_summary): "[moe-profile] <site> dev= host= gap= calls/token= recorded= dropped=
 * evfail=", per token, one line per site that saw anything.  Returns the bytes needed without the terminator. */
size_t wd_profile_report(char *buf, size_t cap);
int wd_profile_reset(void);                          /* forgets every total; keeps the events and the switch */


/* ---- GGUF container ---------------------------------------------------------------------------
 * Read-only memory map of a GGUF file (versions 2 and 3) with its metadata and tensor directory parsed; tensor
 * views point into the mapping (raw block bytes, as the expert cache, wd_memcpy_h2d and the layer descriptors
 * take them).  reference: GgufFile / MappedFile / TensorInfo, src/gguf.hpp:71-491. */
typedef struct wd_gguf wd_gguf;
typedef struct {
    const char *name;          /* owned by the wd_gguf object */
    uint32_t n_dims;
    uint64_t dims[4];          /* GGUF order: dims[0] = columns; unused ones are 1 */
    uint32_t type;             /* ggml type id (WD_TYPE_* for the ones this library computes with) */
    uint64_t relative_offset;  /* from the start of the data section */
    uint64_t bytes;            /* size of the tensor data; 0 when the type's block size is unknown here */
    const uint8_t *data;       /* inside the mapping, valid until wd_gguf_close */
} wd_gguf_tensor_info;
int wd_gguf_open(wd_gguf **out, const char *path);
int wd_gguf_close(wd_gguf *g);
uint32_t wd_gguf_version(const wd_gguf *g);
size_t wd_gguf_data_offset(const wd_gguf *g);              /* file offset of the data section (for pread users) */
const uint8_t *wd_gguf_map_base(const wd_gguf *g);         /* the mapping of the whole file, its size, its descriptor */
size_t wd_gguf_map_bytes(const wd_gguf *g);
int wd_gguf_fd(const wd_gguf *g);
long long wd_gguf_tensor_count(const wd_gguf *g);
long long wd_gguf_find(const wd_gguf *g, const char *name); /* index or -1 */
int wd_gguf_tensor(const wd_gguf *g, long long index, wd_gguf_tensor_info *out);
/* Metadata: numbers of any scalar type as a double (WD_OK, or WD_ERR_ARG when absent or not a number), strings
 * (NULL when absent), arrays of fixed-size elements (length, or -1; *data points into the mapping). */
int wd_gguf_meta_number(const wd_gguf *g, const char *key, double *out);
const char *wd_gguf_meta_string(const wd_gguf *g, const char *key);
long long wd_gguf_meta_array(const wd_gguf *g, const char *key, uint32_t *elem_type, const void **data);

#ifdef __cplusplus
}
#endif
#endif
