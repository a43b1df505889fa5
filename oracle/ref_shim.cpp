// Thin extern "C" window onto the reference's own CPU MoE header, compiled from
// where it lies (-I/root/reference/src).  TEST INFRASTRUCTURE ONLY.  It exists to
// (a) pin oracle/wd_oracle.c bit-for-bit against the real reference arithmetic and
// (b) serve as the "reference" CPU baseline timed by bench.py.  The output of this
// build (oracle/_ref/libwdref.so) is never committed and the shipped library never
// loads it.  Structure-of-arrays activations are repacked into the reference's
// array-of-structures blocks here; no arithmetic is done in this file except the
// shared-expert composition, which calls the reference primitives in the order of
// src/qwen38_moe.cuh:3852-3891.
#include <cstdint>
#include <cstring>
#include <memory>
#include <vector>

#include "qwen38_cpu_moe.cuh"
#include "qwen38_precision.hpp"

using namespace wd::cpu_moe;

namespace {

std::vector<q8_K> pack_q8k(const int8_t *qs, const float *d, int cols) {
    std::vector<q8_K> y(static_cast<size_t>(cols / 256));
    for (size_t b = 0; b < y.size(); ++b) {
        y[b].d = d[b];
        std::memcpy(y[b].qs, qs + b * 256, 256);
        for (int j = 0; j < 16; ++j) {
            int s = 0;
            for (int i = 0; i < 16; ++i) s += y[b].qs[16 * j + i];
            y[b].bsums[j] = static_cast<int16_t>(s);
        }
    }
    return y;
}

std::vector<q8_0> pack_q80(const int8_t *qs, const uint16_t *d, int cols) {
    std::vector<q8_0> y(static_cast<size_t>(cols / 32));
    for (size_t b = 0; b < y.size(); ++b) {
        y[b].d = d[b];
        std::memcpy(y[b].qs, qs + b * 32, 32);
    }
    return y;
}

int to_block_type(int ggml_type) { return block_type_from_ggml(ggml_type); }

std::unique_ptr<ThreadPool> g_pool;
int g_pool_threads = 0;

ThreadPool &pool(int threads) {
    if (!g_pool || g_pool_threads != threads) {
        g_pool.reset(new ThreadPool(threads));
        g_pool_threads = threads;
    }
    return *g_pool;
}

}  // namespace

extern "C" {

int wdref_thread_count() { return thread_count(); }
const uint32_t *wdref_iq3s_grid() { return kIq3sGrid; }
const uint64_t *wdref_iq2s_grid() { return kIq2sGrid; }
float wdref_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t wdref_f32_to_f16(float v) { return f32_to_f16_bits(v); }
float wdref_exp(float x) { return ggml_avx2_exp_f32(x); }
float wdref_silu(float x) { return silu_ggml(x); }
float wdref_sigmoid(float x) { return sigmoid_ggml(x); }
float wdref_dot_f32(const float *a, const float *b, int n) { return dot_f32_avx2(a, b, n); }
// src/qwen38_precision.hpp:32-55 (the host branches)
float wdref_moe_branch_f32(float routed, float shared, float gate) { return wd::q38_moe_branch_f32(routed, shared, gate); }
float wdref_residual_add_f32(float residual, float branch, float weight) { return wd::q38_residual_add_f32(residual, branch, weight); }
float wdref_round_half(float value) { return wd::q38_round_half(value); }

void wdref_quantize_q8_0(const float *x, int n, int8_t *qs, uint16_t *d) {
    std::vector<q8_0> y(static_cast<size_t>(n / 32));
    quantize_q8_0(x, y.data(), n / 32);
    for (size_t b = 0; b < y.size(); ++b) {
        d[b] = y[b].d;
        std::memcpy(qs + b * 32, y[b].qs, 32);
    }
}

void wdref_quantize_q8_K(const float *x, int n, int8_t *qs, float *d, int16_t *bsums) {
    std::vector<q8_K> y(static_cast<size_t>(n / 256));
    quantize_q8_K(x, y.data(), n / 256);
    for (size_t b = 0; b < y.size(); ++b) {
        d[b] = y[b].d;
        std::memcpy(qs + b * 256, y[b].qs, 256);
        std::memcpy(bsums + b * 16, y[b].bsums, 32);
    }
}

// scalar != 0 selects the reference's scalar twin instead of its AVX2 kernel.
float wdref_row(int ggml_type, const uint8_t *w, const int8_t *qs, const void *d, int cols, int scalar) {
    switch (to_block_type(ggml_type)) {
        case kIq3S: {
            auto y = pack_q8k(qs, static_cast<const float *>(d), cols);
            return scalar ? scalar_iq3_s_q8_K(w, y.data(), cols) : row_iq3_s_q8_K(w, y.data(), cols);
        }
        case kIq2S: {
            auto y = pack_q8k(qs, static_cast<const float *>(d), cols);
            return scalar ? scalar_iq2_s_q8_K(w, y.data(), cols) : row_iq2_s_q8_K(w, y.data(), cols);
        }
        case kQ8_0: {
            auto y = pack_q80(qs, static_cast<const uint16_t *>(d), cols);
            return scalar ? scalar_q8_0_q8_0(w, y.data(), cols) : row_q8_0_q8_0(w, y.data(), cols);
        }
        case kIq4Nl: {
            auto y = pack_q80(qs, static_cast<const uint16_t *>(d), cols);
            return scalar ? scalar_iq4_nl_q8_0(w, y.data(), cols) : row_iq4_nl_q8_0(w, y.data(), cols);
        }
        default: return 0.0f / 0.0f;
    }
}

void wdref_gemv(int ggml_type, const uint8_t *w, int rows, int cols, const int8_t *qs, const void *d,
                float *out) {
    const int bt = to_block_type(ggml_type);
    const size_t rb = row_bytes(bt, cols);
    if (bt == kIq3S || bt == kIq2S) {
        auto y = pack_q8k(qs, static_cast<const float *>(d), cols);
        for (int r = 0; r < rows; ++r) out[r] = dot_row(bt, w + static_cast<size_t>(r) * rb, y.data(), cols);
    } else {
        auto y = pack_q80(qs, static_cast<const uint16_t *>(d), cols);
        for (int r = 0; r < rows; ++r) out[r] = dot_row(bt, w + static_cast<size_t>(r) * rb, y.data(), cols);
    }
}

// Routed experts of one layer through the reference's run_layer (gate/up must be
// IQ2_S or IQ3_S: the reference always feeds them Q8_K).  out is zeroed first.
void wdref_run_layer(const uint8_t *gate, const uint8_t *up, const uint8_t *down, int gate_type, int up_type,
                     int down_type, int hidden, int ffn, const float *x, const int *ids, const float *weights,
                     int k, int threads, float *out) {
    LayerWeights w;
    w.gate = gate;
    w.up = up;
    w.down = down;
    w.hidden = hidden;
    w.expert_ffn = ffn;
    w.gate_type = to_block_type(gate_type);
    w.up_type = to_block_type(up_type);
    w.down_type = to_block_type(down_type);
    w.gate_expert_stride = static_cast<size_t>(ffn) * row_bytes(w.gate_type, hidden);
    w.up_expert_stride = static_cast<size_t>(ffn) * row_bytes(w.up_type, hidden);
    w.down_expert_stride = static_cast<size_t>(hidden) * row_bytes(w.down_type, ffn);
    static thread_local LayerScratch scratch;
    static thread_local int sk = 0, sh = 0, sf = 0;
    if (sk != k || sh != hidden || sf != ffn) {
        scratch.reset(k, hidden, ffn);
        sk = k;
        sh = hidden;
        sf = ffn;
    }
    std::memset(out, 0, sizeof(float) * static_cast<size_t>(hidden));
    run_layer(w, pool(threads), x, ids, weights, k, scratch, out);
}

// Q8_0 expert chain on a f32 input, composed from the reference primitives in the
// order of the shared-expert runner: quantize_q8_0 -> gate/up rows -> silu*up ->
// quantize_q8_0 -> down rows.
void wdref_q8_0_chain(const uint8_t *gate, const uint8_t *up, const uint8_t *down, int hidden, int ffn,
                      const float *x, float *out) {
    std::vector<q8_0> xq(static_cast<size_t>(hidden / 32));
    quantize_q8_0(x, xq.data(), hidden / 32);
    const size_t rb_h = row_bytes(kQ8_0, hidden);
    const size_t rb_f = row_bytes(kQ8_0, ffn);
    std::vector<float> act(static_cast<size_t>(ffn));
    for (int r = 0; r < ffn; ++r) {
        const float g = row_q8_0_q8_0(gate + static_cast<size_t>(r) * rb_h, xq.data(), hidden);
        const float u = row_q8_0_q8_0(up + static_cast<size_t>(r) * rb_h, xq.data(), hidden);
        act[static_cast<size_t>(r)] = silu_ggml(g) * u;
    }
    std::vector<q8_0> aq(static_cast<size_t>(ffn / 32));
    quantize_q8_0(act.data(), aq.data(), ffn / 32);
    for (int r = 0; r < hidden; ++r) out[r] = row_q8_0_q8_0(down + static_cast<size_t>(r) * rb_f, aq.data(), ffn);
}

// out[i] = add_rn(out[i], mul_rn(src[i], w)): the reference's combine step.
void wdref_accumulate(float *out, const float *src, float w, int n) {
    for (int i = 0; i < n; ++i) out[i] = add_rn(out[i], mul_rn(src[i], w));
}

}  // extern "C"
