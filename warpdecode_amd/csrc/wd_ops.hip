// Stand-alone operators of the MoE decode path: activation quantisers, router GEMV,
// softmax/top-k, low-bit GEMVs (one matrix or one dispatch over several expert matrices)
// and the elementwise stages.  Each extern "C" entry point mirrors one launcher of the
// reference operator surface (see include/warpdecode_amd.h for the citations).
#include <cstring>

#include "wd_common.h"
#include "wd_fused.cuh"
#include "wd_profile.hpp"

namespace wd {

thread_local std::string g_last_error;
std::string &last_error_slot() { return g_last_error; }

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

}  // namespace wd

using namespace wd;

extern "C" {

const char *wd_last_error(void) { return last_error_slot().c_str(); }

int wd_init(int device) {
    int count = 0;
    WD_HIP(hipGetDeviceCount(&count));
    WD_REQUIRE(device >= 0 && device < count, "wd_init: device %d out of range (%d devices)", device, count);
    WD_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    WD_HIP(hipGetDeviceProperties(&prop, device));
    WD_REQUIRE(prop.warpSize == 64, "wd_init: device %s has %d-wide waves; this library is built for gfx950",
               prop.name, prop.warpSize);
    return noalloc_setup_current_device();
}

size_t wd_row_bytes(int type, int cols) { return row_bytes(type, cols); }
size_t wd_tensor_bytes(int type, int rows, int cols) {
    return rows > 0 ? static_cast<size_t>(rows) * row_bytes(type, cols) : 0;
}

// ---- runtime helpers ------------------------------------------------------------------
int wd_malloc(void **d_ptr, size_t bytes) {
    WD_REQUIRE(d_ptr != nullptr, "wd_malloc: null output pointer");
    WD_HIP(hipMalloc(d_ptr, bytes));
    return WD_OK;
}
int wd_free(void *d_ptr) {
    WD_HIP(hipFree(d_ptr));
    return WD_OK;
}
int wd_malloc_host(void **h_ptr, size_t bytes) {
    WD_REQUIRE(h_ptr != nullptr, "wd_malloc_host: null output pointer");
    WD_HIP(hipHostMalloc(h_ptr, bytes, hipHostMallocDefault));
    return WD_OK;
}
int wd_free_host(void *h_ptr) {
    WD_HIP(hipHostFree(h_ptr));
    return WD_OK;
}
int wd_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes, void *stream) {
    if (stream)
        WD_HIP(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    else
        WD_HIP(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice));
    return WD_OK;
}
int wd_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes, void *stream) {
    if (stream)
        WD_HIP(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    else
        WD_HIP(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost));
    return WD_OK;
}
int wd_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes, void *stream) {
    WD_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return WD_OK;
}
int wd_memset(void *d_dst, int value, size_t bytes, void *stream) {
    WD_REQUIRE(bytes % 4 == 0, "wd_memset: size must be a multiple of 4 bytes");
    const uint32_t b = static_cast<uint32_t>(value) & 0xffu;
    const size_t n = bytes / 4;
    if (n == 0) return WD_OK;
    // a fill kernel rather than hipMemsetAsync, so the call may sit inside a captured graph
    k_fill_u32<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream)>>>(
        static_cast<uint32_t *>(d_dst), b * 0x01010101u, n);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
int wd_stream_create(void **stream) {
    WD_REQUIRE(stream != nullptr, "wd_stream_create: null output pointer");
    hipStream_t s;
    WD_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return WD_OK;
}
int wd_stream_destroy(void *stream) {
    WD_HIP(hipStreamDestroy(as_stream(stream)));
    return WD_OK;
}
int wd_stream_sync(void *stream) {
    WD_HIP(hipStreamSynchronize(as_stream(stream)));
    return WD_OK;
}
int wd_device_sync(void) {
    WD_HIP(hipDeviceSynchronize());
    return WD_OK;
}

// ---- quantisers -------------------------------------------------------------------------
int wd_q8_k_quantize_f32(const float *d_x, int elements, int8_t *d_qs, float *d_scales, int16_t *d_bsums,
                         void *stream) {
    WD_REQUIRE(elements > 0 && elements % 256 == 0,
               "Q8_K quantisation requires a positive multiple of 256 elements (got %d)", elements);
    WD_REQUIRE(d_x && d_qs && d_scales && d_bsums, "wd_q8_k_quantize_f32: null pointer");
    const int blocks = elements / 256;
    k_q8_k_quantize<<<dim3((blocks + 3) / 4), dim3(256), 0, as_stream(stream)>>>(d_x, blocks, d_qs, d_scales, d_bsums);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_q8_0_quantize_f32(const float *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream) {
    WD_REQUIRE(elements > 0 && elements % 32 == 0,
               "Q8_0 quantisation requires a positive multiple of 32 elements (got %d)", elements);
    WD_REQUIRE(d_x && d_qs && d_scales, "wd_q8_0_quantize_f32: null pointer");
    const int blocks = elements / 32;
    k_q8_0_quantize<<<dim3((blocks + 31) / 32), dim3(256), 0, as_stream(stream)>>>(d_x, blocks, d_qs, d_scales);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_q8_1_quantize_f32(const float *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream) {
    WD_REQUIRE(elements > 0 && elements % 32 == 0, "Q8_1 input must be a positive multiple of 32 (got %d)", elements);
    WD_REQUIRE(d_x && d_qs && d_scales, "wd_q8_1_quantize_f32: null pointer");
    const int blocks = elements / 32;
    k_q8_1_quantize<<<dim3((blocks + 31) / 32), dim3(256), 0, as_stream(stream)>>>(d_x, blocks, d_qs, d_scales);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
int wd_q8_0_quantize_f16(const uint16_t *d_x, int elements, int8_t *d_qs, uint16_t *d_scales, void *stream) {
    WD_REQUIRE(elements > 0 && elements % 32 == 0, "Q8_0 quantisation requires a positive multiple of 32 elements (got %d)", elements);
    WD_REQUIRE(d_x && d_qs && d_scales, "wd_q8_0_quantize_f16: null pointer");
    WD_REQUIRE(reinterpret_cast<uintptr_t>(d_x) % 8 == 0, "wd_q8_0_quantize_f16: the input must be 8-byte aligned");
    const int blocks = elements / 32;
    k_q8_0_quantize_f16<<<dim3((blocks + 31) / 32), dim3(256), 0, as_stream(stream)>>>(d_x, blocks, d_qs, d_scales);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
int wd_gemv_q8_0_q8_1_f32(const uint8_t *d_w, int rows, int cols, const int8_t *d_qs, const uint16_t *d_scales, float *d_y,
                          int32_t *d_block_sums, void *stream) {
    WD_REQUIRE(rows > 0 && cols > 0 && cols % 32 == 0, "Q8_0 x Q8_1 GEMV geometry mismatch (%d x %d)", rows, cols);
    WD_REQUIRE(d_w && d_qs && d_scales && d_y, "wd_gemv_q8_0_q8_1_f32: null pointer");
    WD_REQUIRE(reinterpret_cast<uintptr_t>(d_qs) % 4 == 0, "wd_gemv_q8_0_q8_1_f32: the quantised input must be 4-byte aligned");
    k_gemv_q8_0_q8_1<<<dim3((rows + 3) / 4), dim3(256), 0, as_stream(stream)>>>(d_w, rows, cols, d_qs, d_scales, d_y, d_block_sums);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
int wd_convert_f16_to_f32(const uint16_t *d_src, float *d_dst, size_t n, void *stream) {
    WD_REQUIRE(d_src && d_dst && n > 0, "wd_convert_f16_to_f32: invalid arguments");
    k_f16_to_f32<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream)>>>(d_src, d_dst, n);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
int wd_convert_f32_to_f16(const float *d_src, uint16_t *d_dst, size_t n, void *stream) {
    WD_REQUIRE(d_src && d_dst && n > 0, "wd_convert_f32_to_f16: invalid arguments");
    k_f32_to_f16<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream)>>>(d_src, d_dst, n);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

// ---- router -------------------------------------------------------------------------------
int wd_router_gemv_f32(const float *d_w, const float *d_x, float *d_logits, int rows, int cols, void *stream) {
    WD_REQUIRE(rows > 0 && cols > 0, "router GEMV: invalid shape %d x %d", rows, cols);
    WD_REQUIRE(d_w && d_x && d_logits, "wd_router_gemv_f32: null pointer");
    k_router_gemv<<<dim3((rows + 7) / 8), dim3(256), 0, as_stream(stream)>>>(d_w, d_x, d_logits, rows, cols, nullptr,
                                                                             nullptr);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_topk_softmax(const float *d_logits, int n_experts, int k, float expert_scale, int32_t *d_ids,
                    float *d_weights, void *stream) {
    WD_REQUIRE(n_experts > 0 && n_experts <= 1024 && n_experts % 8 == 0,
               "top-k softmax: n_experts must be a multiple of 8 in (0, 1024] (got %d)", n_experts);
    WD_REQUIRE(k > 0 && k <= 16 && k <= n_experts, "top-k softmax: k must be in (0, 16] (got %d)", k);
    WD_REQUIRE(d_logits && d_ids && d_weights, "wd_topk_softmax: null pointer");
    k_topk_softmax<<<dim3(1), dim3(64), 0, as_stream(stream)>>>(d_logits, n_experts, k, expert_scale, d_ids, d_weights,
                                                                nullptr, nullptr);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

// ---- GEMVs --------------------------------------------------------------------------------
static int launch_gemv_q8k(int type, MatSrc src, int mats, int rows, int cols, const int8_t *qs, const float *d,
                           float *out, int32_t *partials, hipStream_t stream) {
    WD_REQUIRE(type == WD_TYPE_IQ3_S || type == WD_TYPE_IQ2_S, "Q8_K-activation GEMV supports IQ3_S and IQ2_S (type %d)",
               type);
    WD_REQUIRE(rows > 0 && cols > 0 && cols % 256 == 0, "invalid low-bit matrix shape %d x %d", rows, cols);
    WD_REQUIRE(mats > 0 && mats <= 64, "expert batch must be in (0, 64] (got %d)", mats);
    WD_REQUIRE(qs && d && out, "low-bit GEMV: null pointer");
    const dim3 grid((rows + 15) / 16, mats), block(256);
    const int ppr = partials_per_row(type, cols);
    if (type == WD_TYPE_IQ3_S) {
        if (partials)
            k_gemv_iq<21, true><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, out, partials, ppr);
        else
            k_gemv_iq<21, false><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, out, nullptr, 0);
    } else {
        if (partials)
            k_gemv_iq<22, true><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, out, partials, ppr);
        else
            k_gemv_iq<22, false><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, out, nullptr, 0);
    }
    WD_LAUNCH_CHECK();
    return WD_OK;
}

// The split configuration of the streaming kernel for rows of nb blocks in `groups` groups of eight rows; null when the
// kernel for that shape is another one.
struct Q8Split { int nb, kb, nch, waves; };
static const Q8Split *q8_split_for(int nb, int groups) {
    static const Q8Split kSplits[] = {{64, 32, 1, 2}, {80, 16, 1, 5}, {128, 32, 1, 4}, {160, 32, 1, 5}, {256, 32, 1, 8},
                                      {256, 32, 2, 4}, {320, 32, 2, 5}, {512, 32, 2, 8}};
    for (const Q8Split &sp : kSplits) {
        if (groups >= 1024 || sp.nb != nb) continue;
        // 8192 columns: eight waves when a compute unit gets one workgroup, four (two chunks each) when it gets more
        if (nb == 256 && (sp.waves == 8) != (groups <= 256)) continue;
        return &sp;
    }
    return nullptr;
}

static int launch_gemv_q8_0(int type, MatSrc src, int mats, int rows, int cols, const int8_t *qs, const uint16_t *d,
                            int act_per_mat, float *out, int32_t *partials, hipStream_t stream) {
    WD_REQUIRE(type == WD_TYPE_Q8_0 || type == WD_TYPE_IQ4_NL || type == WD_TYPE_Q4_0,
               "Q8_0-activation GEMV supports Q8_0, IQ4_NL and Q4_0 (type %d)", type);
    WD_REQUIRE(rows > 0 && cols > 0 && cols % 32 == 0, "invalid low-bit matrix shape %d x %d", rows, cols);
    WD_REQUIRE(mats > 0 && mats <= 64, "expert batch must be in (0, 64] (got %d)", mats);
    WD_REQUIRE(qs && d && out, "low-bit GEMV: null pointer");
    const dim3 grid((rows + 15) / 16, mats), block(256);
    const int ppr = partials_per_row(type, cols);
    const int act_stride = act_per_mat ? cols : 0;
    const int nb = cols / 32;
    if (type == WD_TYPE_Q4_0 && mats == 1 && src.single && nb % 8 == 0 && nb / 8 <= 64 && 64 % (nb / 8) == 0 &&
        reinterpret_cast<uintptr_t>(src.single) % 16 == 0 && reinterpret_cast<uintptr_t>(qs) % 16 == 0) {
        // whole 8-block groups per row and a 16-byte aligned base: the streaming kernel
        const int rpp = 64 / (nb / 8);
        const long long passes = (static_cast<long long>(rows) + rpp - 1) / rpp;
        // four waves per workgroup stream best; two when the whole matrix is only a few hundred passes
        const int wpb = passes <= 256 ? 2 : 4;
        const unsigned wgs = static_cast<unsigned>((passes + wpb - 1) / wpb);
        const size_t lds = static_cast<size_t>(nb / 8) * 272 + static_cast<size_t>(nb) * 8;
#define WD_Q4S_LAUNCH(WPB)                                                                                              \
    do {                                                                                                                \
        if (partials)                                                                                                   \
            k_gemv_q4_stream<true, 1, WPB><<<wgs, WPB * 64, lds, stream>>>(src.single, rows, nb, qs, d, out, partials); \
        else                                                                                                            \
            k_gemv_q4_stream<false, 1, WPB><<<wgs, WPB * 64, lds, stream>>>(src.single, rows, nb, qs, d, out, nullptr); \
    } while (0)
        if (wpb == 2)
            WD_Q4S_LAUNCH(2);
        else
            WD_Q4S_LAUNCH(4);
#undef WD_Q4S_LAUNCH
        WD_LAUNCH_CHECK();
        return WD_OK;
    }
    if (type == WD_TYPE_Q8_0 && mats == 1 && src.single && nb % 16 == 0 && cols <= 16384 && rows >= 8 &&
        reinterpret_cast<uintptr_t>(src.single) % 16 == 0 && reinterpret_cast<uintptr_t>(qs) % 16 == 0) {
        // whole 16-byte words per row chunk and a 16-byte aligned base: the streaming kernel, eight rows per wave
        const int groups = (rows + 7) / 8;
        // few row groups: the waves of a workgroup share a group, the chain runs over prepared pairs
        if (const Q8Split *found = q8_split_for(nb, groups)) {
            const Q8Split &sp = *found;
            const size_t lds = static_cast<size_t>(cols) + static_cast<size_t>(nb) * 4 + 256 +
                               static_cast<size_t>(sp.waves) * 8 * (sp.kb == 32 ? kQ8sRowStride<32> : kQ8sRowStride<16>);
            auto launch = [&](auto kernel) { kernel<<<groups, 64 * sp.waves, lds, stream>>>(src.single, rows, nb, qs, d, out, partials); };
#define WD_Q8_SPLIT(KB_, NCH_, WAVES_)                                                                      \
    if (sp.kb == KB_ && sp.nch == NCH_ && sp.waves == WAVES_) {                                               \
        partials ? launch(k_gemv_q8_rows8_split<KB_, NCH_, WAVES_, true>) : launch(k_gemv_q8_rows8_split<KB_, NCH_, WAVES_, false>); \
    }
            WD_Q8_SPLIT(32, 1, 2)
            WD_Q8_SPLIT(16, 1, 5)
            WD_Q8_SPLIT(32, 1, 4)
            WD_Q8_SPLIT(32, 1, 5)
            WD_Q8_SPLIT(32, 1, 8)
            WD_Q8_SPLIT(32, 2, 4)
            WD_Q8_SPLIT(32, 2, 5)
            WD_Q8_SPLIT(32, 2, 8)
#undef WD_Q8_SPLIT
            WD_LAUNCH_CHECK();
            return WD_OK;
        }
        // Workgroups of four waves (taking several row groups each beyond 1024 workgroups) when there is a row group
        // or more per SIMD; otherwise single waves, which keep two chunks in flight to cover the memory latency.
        const int waves = groups >= 1024 ? 4 : 1;
        int wgs_wanted = (groups + waves - 1) / waves;
        wgs_wanted = std::min(wgs_wanted, waves == 4 ? 1024 : 2048);
        const unsigned wgs = static_cast<unsigned>(wgs_wanted);
        // single waves: 32-block chunks, two of them in flight; full workgroups: 16-block chunks, one ahead
        const int kb = (waves == 1 && nb % 32 == 0) ? 32 : 16;
        const size_t lds = static_cast<size_t>(cols) + static_cast<size_t>(nb) * 4 +
                           static_cast<size_t>(waves) * 8 * (kb == 32 ? kQ8sRowStride<32> : kQ8sRowStride<16>);
        auto launch = [&](auto kernel) { kernel<<<wgs, 64 * waves, lds, stream>>>(src.single, rows, nb, qs, d, out, partials); };
        if (waves == 4) partials ? launch(k_gemv_q8_rows8<16, true, 4, 1>) : launch(k_gemv_q8_rows8<16, false, 4, 1>);
        else if (kb == 32) partials ? launch(k_gemv_q8_rows8<32, true, 1, 2>) : launch(k_gemv_q8_rows8<32, false, 1, 2>);
        else partials ? launch(k_gemv_q8_rows8<16, true, 1, 2>) : launch(k_gemv_q8_rows8<16, false, 1, 2>);
        WD_LAUNCH_CHECK();
        return WD_OK;
    }
#define WD_Q8_LAUNCH(KIND)                                                                                          \
    do {                                                                                                            \
        if (partials)                                                                                               \
            k_gemv_q8<KIND, true><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, act_stride, out, partials, ppr); \
        else                                                                                                        \
            k_gemv_q8<KIND, false><<<grid, block, 0, stream>>>(src, rows, cols, qs, d, act_stride, out, nullptr, 0); \
    } while (0)
    if (type == WD_TYPE_Q8_0)
        WD_Q8_LAUNCH(0);
    else if (type == WD_TYPE_IQ4_NL)
        WD_Q8_LAUNCH(1);
    else
        WD_Q8_LAUNCH(2);
#undef WD_Q8_LAUNCH
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_gemv_q6_k_q8_k_f32(const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs, const float *d_act_scales,
                          const int16_t *d_act_bsums, float *d_out, int32_t *d_partials, void *stream) {
    WD_REQUIRE(d_w && d_act_qs && d_act_scales && d_act_bsums && d_out, "Q6_K GEMV: null pointer");
    WD_REQUIRE(rows > 0 && cols > 0 && cols % 256 == 0, "Q6_K x Q8_K GEMV geometry mismatch (%d x %d)", rows, cols);
    WD_REQUIRE(cols <= 32768, "Q6_K GEMV: at most 32768 columns (got %d)", cols);
    WD_REQUIRE(reinterpret_cast<uintptr_t>(d_act_qs) % 16 == 0 && reinterpret_cast<uintptr_t>(d_act_bsums) % 4 == 0,
               "Q6_K GEMV: the activation quants must be 16-byte aligned, the sums 4-byte aligned");
    const int nb = cols / 256;
    // rows are 210 * nb bytes: they all start on 16-byte boundaries when the matrix does and nb is a multiple of 8
    const bool aligned = reinterpret_cast<uintptr_t>(d_w) % 16 == 0 && nb % 8 == 0;
    // enough rows per wave to pay for staging the activation, few enough to keep every compute unit busy
    int rpw = rows / (4 * 2048);
    rpw = rpw < 1 ? 1 : (rpw > 10 ? 10 : rpw);
    const unsigned wgs = static_cast<unsigned>((static_cast<long long>(rows) + 4LL * rpw - 1) / (4LL * rpw));
    const size_t lds = static_cast<size_t>(nb) * kQ6ActStride + ((nb * 4 + 15) & ~15) + static_cast<size_t>(nb) * 32 + 4 * kQ6StageBytes;
    hipStream_t st = as_stream(stream);
    const bool full = nb % 8 == 0;
    auto launch = [&](auto kernel) { kernel<<<wgs, 256, lds, st>>>(d_w, rows, cols, d_act_qs, d_act_scales, d_act_bsums, d_out, d_partials); };
    if (d_partials) {
        if (aligned) launch(k_gemv_q6k<true, true, true>);  // aligned implies whole passes
        else if (full) launch(k_gemv_q6k<true, false, true>);
        else launch(k_gemv_q6k<true, false, false>);
    } else {
        if (aligned) launch(k_gemv_q6k<false, true, true>);
        else if (full) launch(k_gemv_q6k<false, false, true>);
        else launch(k_gemv_q6k<false, false, false>);
    }
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_gemv_q8_k_f32(int type, const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs,
                     const float *d_act_scales, float *d_out, int32_t *d_partials, void *stream) {
    WD_REQUIRE(d_w != nullptr, "low-bit GEMV: null weight pointer");
    MatSrc src{};
    src.single = d_w;
    return launch_gemv_q8k(type, src, 1, rows, cols, d_act_qs, d_act_scales, d_out, d_partials, as_stream(stream));
}

int wd_gemv_q8_0_f32(int type, const uint8_t *d_w, int rows, int cols, const int8_t *d_act_qs,
                     const uint16_t *d_act_scales, float *d_out, int32_t *d_partials, void *stream) {
    WD_REQUIRE(d_w != nullptr, "low-bit GEMV: null weight pointer");
    MatSrc src{};
    src.single = d_w;
    return launch_gemv_q8_0(type, src, 1, rows, cols, d_act_qs, d_act_scales, 0, d_out, d_partials, as_stream(stream));
}

// Q4_0 matrices: the workgroups per item of the streaming kernel (waves per workgroup in *wpb), 0 when the item takes
// another kernel alone.
static int q4_stream_wgs(const wd_gemv_item &it, int nb, int *wpb) {
    if (!(nb % 8 == 0 && nb / 8 <= 64 && 64 % (nb / 8) == 0 && reinterpret_cast<uintptr_t>(it.d_w) % 16 == 0 &&
          reinterpret_cast<uintptr_t>(it.d_act_qs) % 16 == 0))
        return 0;
    const int rpp = 64 / (nb / 8);
    const long long passes = (static_cast<long long>(it.rows) + rpp - 1) / rpp;
    *wpb = passes <= 256 ? 2 : 4;
    const long long wgs = (passes + *wpb - 1) / *wpb;
    return wgs <= 4096 ? static_cast<int>(wgs) : 0;  // (large matrices are not bound by their launch)
}
static int gemv_q4_0_batch(const wd_gemv_item *items, int n_items, int cols, void *stream) {
    const int nb = cols / 32;
    int i = 0;
    while (i < n_items) {
        int wpb = 0, other = 0;
        const int wgs0 = q4_stream_wgs(items[i], nb, &wpb);
        int j = i + 1;
        if (wgs0)
            while (j < n_items && j - i < kGemvBatchMax && q4_stream_wgs(items[j], nb, &other) && other == wpb) ++j;
        if (!wgs0 || j - i == 1) {
            if (const int rc = wd_gemv_q8_0_f32(WD_TYPE_Q4_0, items[i].d_w, items[i].rows, cols, items[i].d_act_qs, items[i].d_act_scales,
                                                items[i].d_out, nullptr, stream))
                return rc;
            ++i;
            continue;
        }
        GemvBatch b{};
        b.n = j - i;
        int wgs = 0;
        for (int q = 0; q < b.n; ++q) {
            const wd_gemv_item &it = items[i + q];
            b.w[q] = it.d_w, b.act_qs[q] = it.d_act_qs, b.act_d[q] = it.d_act_scales, b.out[q] = it.d_out, b.rows[q] = it.rows;
            b.first_group[q] = wgs;
            wgs += q4_stream_wgs(it, nb, &other);
        }
        for (int q = b.n; q <= kGemvBatchMax; ++q) b.first_group[q] = wgs;
        const size_t lds = static_cast<size_t>(nb / 8) * 272 + static_cast<size_t>(nb) * 8;
        if (wpb == 2)
            k_gemv_q4_stream_batch<2><<<wgs, 128, lds, as_stream(stream)>>>(b, nb);
        else
            k_gemv_q4_stream_batch<4><<<wgs, 256, lds, as_stream(stream)>>>(b, nb);
        WD_LAUNCH_CHECK();
        i = j;
    }
    return WD_OK;
}

int wd_gemv_q8_0_batch_f32(int type, const wd_gemv_item *items, int n_items, int cols, void *stream) {
    WD_REQUIRE(type == WD_TYPE_Q8_0 || type == WD_TYPE_Q4_0, "batched GEMV: Q8_0 (exact order) or Q4_0 matrices (type %d)", type);
    WD_REQUIRE(items != nullptr && n_items > 0, "batched GEMV: no items");
    WD_REQUIRE(cols > 0 && cols % 32 == 0, "batched GEMV: invalid row length %d", cols);
    for (int i = 0; i < n_items; ++i)
        WD_REQUIRE(items[i].d_w && items[i].d_act_qs && items[i].d_act_scales && items[i].d_out && items[i].rows > 0,
                   "batched GEMV: item %d has a null pointer or no rows", i);
    if (type == WD_TYPE_Q4_0) return gemv_q4_0_batch(items, n_items, cols, stream);
    const int nb = cols / 32;
    // One launch for as many items in a row as take the same kernel: every item must be a shape the split kernel takes
    // alone (then its workgroups do here exactly what they do there); anything else is launched by itself.
    auto splits_alike = [&](const wd_gemv_item &it, const Q8Split *want) {
        const Q8Split *sp = nb % 16 == 0 && cols <= 16384 && it.rows >= 8 && reinterpret_cast<uintptr_t>(it.d_w) % 16 == 0 &&
                                    reinterpret_cast<uintptr_t>(it.d_act_qs) % 16 == 0
                                ? q8_split_for(nb, (it.rows + 7) / 8)
                                : nullptr;
        return sp != nullptr && (want == nullptr || sp == want) ? sp : nullptr;
    };
    int i = 0;
    while (i < n_items) {
        const Q8Split *sp = splits_alike(items[i], nullptr);
        int j = i + 1;
        if (sp)
            while (j < n_items && j - i < kGemvBatchMax && splits_alike(items[j], sp)) ++j;
        if (!sp || j - i == 1) {
            if (const int rc = wd_gemv_q8_0_f32(type, items[i].d_w, items[i].rows, cols, items[i].d_act_qs, items[i].d_act_scales,
                                                items[i].d_out, nullptr, stream))
                return rc;
            ++i;
            continue;
        }
        GemvBatch b{};
        b.n = j - i;
        int groups = 0;
        for (int q = 0; q < b.n; ++q) {
            const wd_gemv_item &it = items[i + q];
            b.w[q] = it.d_w, b.act_qs[q] = it.d_act_qs, b.act_d[q] = it.d_act_scales, b.out[q] = it.d_out, b.rows[q] = it.rows;
            b.first_group[q] = groups;
            groups += (it.rows + 7) / 8;
        }
        for (int q = b.n; q <= kGemvBatchMax; ++q) b.first_group[q] = groups;
        const size_t lds = static_cast<size_t>(cols) + static_cast<size_t>(nb) * 4 + 256 +
                           static_cast<size_t>(sp->waves) * 8 * (sp->kb == 32 ? kQ8sRowStride<32> : kQ8sRowStride<16>);
        const hipStream_t st = as_stream(stream);
#define WD_Q8_BATCH(KB_, NCH_, WAVES_)                                    \
    if (sp->kb == KB_ && sp->nch == NCH_ && sp->waves == WAVES_)          \
        k_gemv_q8_rows8_split_batch<KB_, NCH_, WAVES_><<<groups, 64 * WAVES_, lds, st>>>(b, nb);
        WD_Q8_BATCH(32, 1, 2)
        WD_Q8_BATCH(16, 1, 5)
        WD_Q8_BATCH(32, 1, 4)
        WD_Q8_BATCH(32, 1, 5)
        WD_Q8_BATCH(32, 1, 8)
        WD_Q8_BATCH(32, 2, 4)
        WD_Q8_BATCH(32, 2, 5)
        WD_Q8_BATCH(32, 2, 8)
#undef WD_Q8_BATCH
        WD_LAUNCH_CHECK();
        i = j;
    }
    return WD_OK;
}

int wd_gemv_q8_k_experts_f32(int type, const uint8_t *const *d_w_experts, int experts, int rows, int cols,
                             const int8_t *d_act_qs, const float *d_act_scales, float *d_out,
                             int32_t *d_partials, void *stream) {
    WD_REQUIRE(d_w_experts != nullptr, "expert GEMV: null pointer table");
    MatSrc src{};
    src.table = d_w_experts;
    return launch_gemv_q8k(type, src, experts, rows, cols, d_act_qs, d_act_scales, d_out, d_partials,
                           as_stream(stream));
}

int wd_gemv_q8_0_experts_f32(int type, const uint8_t *const *d_w_experts, int experts, int rows, int cols,
                             const int8_t *d_act_qs, const uint16_t *d_act_scales, float *d_out,
                             int32_t *d_partials, void *stream) {
    WD_REQUIRE(d_w_experts != nullptr, "expert GEMV: null pointer table");
    MatSrc src{};
    src.table = d_w_experts;
    return launch_gemv_q8_0(type, src, experts, rows, cols, d_act_qs, d_act_scales, 1, d_out, d_partials,
                            as_stream(stream));
}

// ---- elementwise ------------------------------------------------------------------------------
int wd_silu_mul_experts_f32(const float *d_gate_up, float *d_act, int ffn, int experts, void *stream) {
    WD_REQUIRE(ffn > 0 && experts > 0 && d_gate_up && d_act, "silu*up: invalid arguments");
    k_silu_mul_experts<<<dim3((ffn + 255) / 256, experts), dim3(256), 0, as_stream(stream)>>>(d_gate_up, d_act, ffn);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_weighted_accum_experts_f32(const float *d_experts, const float *d_weights, float *d_accum, int n, int k,
                                  void *stream) {
    WD_REQUIRE(n > 0 && k > 0 && d_experts && d_weights && d_accum, "weighted accumulate: invalid arguments");
    k_weighted_accum<<<dim3((n + 255) / 256), dim3(256), 0, as_stream(stream)>>>(d_experts, d_weights, d_accum, n, k);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int wd_add_shared_f32(float *d_routed, const float *d_shared, const float *d_gate, int n, void *stream) {
    WD_REQUIRE(n > 0 && d_routed && d_shared && d_gate, "add shared: invalid arguments");
    SiteScope site(WD_SITE_FINISH, as_stream(stream));
    k_add_shared<<<dim3((n + 255) / 256), dim3(256), 0, as_stream(stream)>>>(d_routed, d_shared, d_gate, d_routed, n);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

// ---- site profiler -----------------------------------------------------------------------
int wd_profile_enable(int on) { return SiteProfiler::instance().enable(on != 0); }
int wd_profile_enabled(void) { return SiteProfiler::instance().enabled() ? 1 : 0; }
int wd_profile_begin(int site, void *stream) {
    WD_REQUIRE(site >= 0 && site < WD_PROFILE_SITE_COUNT, "profiler: site %d out of range", site);
    SiteProfiler::instance().begin(site, as_stream(stream));
    return WD_OK;
}
int wd_profile_end(int site, void *stream) {
    WD_REQUIRE(site >= 0 && site < WD_PROFILE_SITE_COUNT, "profiler: site %d out of range", site);
    SiteProfiler::instance().end(site, as_stream(stream));
    return WD_OK;
}
int wd_profile_flush_token(void) { return SiteProfiler::instance().flush_token(); }
int wd_profile_site(int site, wd_profile_site_stat *out, unsigned long long *tokens) {
    WD_REQUIRE(site >= 0 && site < WD_PROFILE_SITE_COUNT && out, "profiler: site %d out of range, or a null output", site);
    *out = SiteProfiler::instance().stat(site);
    if (tokens) *tokens = SiteProfiler::instance().tokens();
    return WD_OK;
}
const char *wd_profile_site_name(int site) { return profile_site_name(site); }
size_t wd_profile_report(char *buf, size_t cap) {
    const std::string r = SiteProfiler::instance().report();
    if (buf && cap) {
        const size_t n = r.size() < cap - 1 ? r.size() : cap - 1;
        std::memcpy(buf, r.data(), n);
        buf[n] = 0;
    }
    return r.size();
}
int wd_profile_reset(void) {
    SiteProfiler::instance().reset();
    return WD_OK;
}

}  // extern "C"
