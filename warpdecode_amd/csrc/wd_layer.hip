// Whole-layer entry points: scratch object and the staged layer pass (one launch per stage,
// every stage a stand-alone operator of wd_ops.hip resolved against the device-side ids).
#include "wd_profile.hpp"
#include "wd_common.h"
#include "wd_tokens.cuh"
#include "wd_resident.cuh"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

using namespace wd;

struct wd_moe_scratch {
    int hidden = 0, ffn = 0, n_experts = 0, max_k = 0;
    uint8_t *block = nullptr;
    float *logits = nullptr;
    int32_t *ids = nullptr;
    float *weights = nullptr;
    int8_t *xk_qs = nullptr;
    float *xk_d = nullptr;
    int16_t *xk_bs = nullptr;
    int8_t *x0_qs = nullptr;
    uint16_t *x0_d = nullptr;
    float *gate_up = nullptr;
    float *act = nullptr;
    int8_t *act_qs = nullptr;
    uint16_t *act_d = nullptr;
    float *expert_out = nullptr;
    float *accum = nullptr;
    float *down_f32 = nullptr;
    float *shared_gate = nullptr;
    int32_t *gup = nullptr;
    int32_t *dp = nullptr;
    int gup_type = -1, dp_type = -1;
    unsigned *arrive = nullptr;           // device counter used inside the fused dispatch A
    unsigned long long *trace = nullptr;  // device [3][16][8] time stamps, see wd_moe_scratch_trace
    int trace_wg = 0;
    int32_t *h_ids = nullptr;             // pinned [32]: [0..15] routed ids for callers that must see them on the host,
                                          // [16] mirror of the status word, written by the resident launch when a wait runs out
    uint32_t *tagged = nullptr;           // [kTagRecords][kTagCopies][16] ids published inside the merged dispatch
    unsigned *status = nullptr;           // [0] != 0: a bounded wait inside a dispatch ran out
    unsigned spin_limit = kSpinLimit;
    int compute_units = 256;              // of the device the scratch lives on
    // the resident stack kernel (wd_resident.cuh): hand-off buffers, device copy of the layer descriptors
    uint8_t *res_block = nullptr;
    // Device copies of the layer descriptors of the stacks this scratch has run ([kResMaxLayers], then one ResidentViews
    // each).  A copy is never overwritten: a captured graph keeps the address of the copy it was recorded with.
    struct ResDescSet {
        std::vector<ResidentLayer> shadow;
        ResidentLayer *dev = nullptr;
    };
    std::vector<ResDescSet> res_sets;
    int res_fits = -1;                            // -1 not asked yet; 1: the device holds the whole grid at once
    int trace_layer = 0;
    bool trace_all = false;                       // the trace buffer has the resident kernel's size
    // wd_moe_layer_tokens_pairs_f32: a ring of pointer tables (pinned staging + device copy), kPairRing x [kPairEntries][3]
    const uint8_t **pair_host = nullptr, **pair_dev = nullptr;
    hipEvent_t pair_done[4] = {nullptr, nullptr, nullptr, nullptr};
    bool pair_used[4] = {false, false, false, false};
    int pair_next = 0;
};
constexpr int kPairRing = 4;

namespace {
constexpr int kTagRecords = 64;  // one record per layer of a stack (modulo), so that a chain of layers needs no reset in between
}

namespace {

struct Carver {
    size_t off = 0;
    size_t take(size_t bytes) {
        const size_t at = off;
        off += (bytes + 255) & ~static_cast<size_t>(255);
        return at;
    }
};

}  // namespace

extern "C" {

int wd_moe_scratch_create(wd_moe_scratch **out, int hidden, int expert_ffn, int n_experts, int max_k) {
    WD_REQUIRE(out != nullptr, "wd_moe_scratch_create: null output pointer");
    WD_REQUIRE(hidden > 0 && hidden % 256 == 0, "MoE scratch: hidden must be a positive multiple of 256 (got %d)", hidden);
    WD_REQUIRE(expert_ffn > 0 && expert_ffn % 32 == 0, "MoE scratch: expert_ffn must be a positive multiple of 32 (got %d)",
               expert_ffn);
    WD_REQUIRE(n_experts > 0 && max_k > 0 && max_k <= 16, "MoE scratch: invalid expert counts (%d experts, k=%d)",
               n_experts, max_k);
    wd_moe_scratch *s = new (std::nothrow) wd_moe_scratch;
    WD_REQUIRE(s != nullptr, "MoE scratch: out of host memory");
    s->hidden = hidden, s->ffn = expert_ffn, s->n_experts = n_experts, s->max_k = max_k;
    const size_t H = hidden, F = expert_ffn, K1 = max_k + 1;
    Carver c;
    const size_t o_logits = c.take(sizeof(float) * n_experts), o_ids = c.take(sizeof(int32_t) * 16),
                 o_w = c.take(sizeof(float) * 16), o_xkq = c.take(H), o_xkd = c.take(sizeof(float) * (H / 256)),
                 o_xkb = c.take(sizeof(int16_t) * (H / 16)), o_x0q = c.take(H),
                 o_x0d = c.take(sizeof(uint16_t) * (H / 32)), o_gu = c.take(sizeof(float) * K1 * 2 * F),
                 o_act = c.take(sizeof(float) * K1 * F), o_aq = c.take(K1 * F),
                 o_ad = c.take(sizeof(uint16_t) * K1 * (F / 32)), o_eo = c.take(sizeof(float) * K1 * H),
                 o_acc = c.take(sizeof(float) * H), o_dn = c.take(sizeof(float) * H), o_sg = c.take(256),
                 o_arr = c.take(256),
                 o_tag = c.take(sizeof(uint32_t) * kTagRecords * kTagCopies * 16), o_status = c.take(256);
    const hipError_t e = hipMalloc(reinterpret_cast<void **>(&s->block), c.off);
    if (e != hipSuccess) {
        delete s;
        return fail(WD_ERR_HIP, "hipMalloc MoE scratch (%zu bytes) failed: %s", c.off, hipGetErrorString(e));
    }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
        s->compute_units = cus;
    uint8_t *b = s->block;
    s->logits = reinterpret_cast<float *>(b + o_logits);
    s->ids = reinterpret_cast<int32_t *>(b + o_ids);
    s->weights = reinterpret_cast<float *>(b + o_w);
    s->xk_qs = reinterpret_cast<int8_t *>(b + o_xkq);
    s->xk_d = reinterpret_cast<float *>(b + o_xkd);
    s->xk_bs = reinterpret_cast<int16_t *>(b + o_xkb);
    s->x0_qs = reinterpret_cast<int8_t *>(b + o_x0q);
    s->x0_d = reinterpret_cast<uint16_t *>(b + o_x0d);
    s->gate_up = reinterpret_cast<float *>(b + o_gu);
    s->act = reinterpret_cast<float *>(b + o_act);
    s->act_qs = reinterpret_cast<int8_t *>(b + o_aq);
    s->act_d = reinterpret_cast<uint16_t *>(b + o_ad);
    s->expert_out = reinterpret_cast<float *>(b + o_eo);
    s->accum = reinterpret_cast<float *>(b + o_acc);
    s->down_f32 = reinterpret_cast<float *>(b + o_dn);
    s->shared_gate = reinterpret_cast<float *>(b + o_sg);
    s->arrive = reinterpret_cast<unsigned *>(b + o_arr);
    s->tagged = reinterpret_cast<uint32_t *>(b + o_tag);
    s->status = reinterpret_cast<unsigned *>(b + o_status);
    (void)hipMemset(s->block, 0, c.off);
    (void)hipMemset(s->tagged, 0xff, sizeof(uint32_t) * kTagRecords * kTagCopies * 16);
    if (hipHostMalloc(reinterpret_cast<void **>(&s->h_ids), sizeof(int32_t) * 32, hipHostMallocDefault) != hipSuccess) {
        (void)hipFree(s->block);
        delete s;
        return fail(WD_ERR_HIP, "hipHostMalloc MoE scratch ids failed");
    }
    std::memset(s->h_ids, 0, sizeof(int32_t) * 32);
    *out = s;
    return WD_OK;
}

int wd_moe_scratch_destroy(wd_moe_scratch *s) {
    if (!s) return WD_OK;
    (void)hipFree(s->block);
    (void)hipFree(s->gup);
    (void)hipFree(s->dp);
    (void)hipFree(s->trace);
    (void)hipFree(s->res_block);
    for (wd_moe_scratch::ResDescSet &d : s->res_sets) (void)hipFree(d.dev);
    (void)hipHostFree(s->h_ids);
    (void)hipFree(s->pair_dev);
    (void)hipHostFree(s->pair_host);
    for (hipEvent_t ev : s->pair_done)
        if (ev) (void)hipEventDestroy(ev);
    delete s;
    return WD_OK;
}

int wd_moe_scratch_status(wd_moe_scratch *s) {
    if (!s) return -1;
    unsigned v = 0;
    if (hipMemcpy(&v, s->status, sizeof(v), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    return static_cast<int>(v);
}
const unsigned *wd_moe_scratch_status_word(wd_moe_scratch *s) { return s ? s->status : nullptr; }
int wd_moe_scratch_set_wait_limit(wd_moe_scratch *s, unsigned polls) {
    WD_REQUIRE(s != nullptr, "wd_moe_scratch_set_wait_limit: null scratch");
    s->spin_limit = polls ? polls : kSpinLimit;
    // a fresh start: clear the status word and make the published ids invalid again
    WD_HIP(hipDeviceSynchronize());  // (a launch that gave up may still be running and would set the words again)
    WD_HIP(hipMemset(s->status, 0, sizeof(unsigned)));
    reinterpret_cast<volatile int32_t *>(s->h_ids)[16] = 0;
    WD_HIP(hipMemset(s->tagged, 0xff, sizeof(uint32_t) * kTagRecords * kTagCopies * 16));
    if (s->res_block) WD_HIP(hipMemset(s->res_block, 0xff, kHandEpoch));
    return WD_OK;
}
float *wd_moe_scratch_logits(wd_moe_scratch *s) { return s->logits; }
int32_t *wd_moe_scratch_ids(wd_moe_scratch *s) { return s->ids; }
float *wd_moe_scratch_weights(wd_moe_scratch *s) { return s->weights; }
float *wd_moe_scratch_gate_up(wd_moe_scratch *s) { return s->gate_up; }
float *wd_moe_scratch_act(wd_moe_scratch *s) { return s->act; }
int8_t *wd_moe_scratch_act_qs(wd_moe_scratch *s) { return s->act_qs; }
uint16_t *wd_moe_scratch_act_scales(wd_moe_scratch *s) { return s->act_d; }
float *wd_moe_scratch_expert_out(wd_moe_scratch *s) { return s->expert_out; }
float *wd_moe_scratch_accum(wd_moe_scratch *s) { return s->accum; }
float *wd_moe_scratch_down_f32(wd_moe_scratch *s) { return s->down_f32; }
float *wd_moe_scratch_shared_gate(wd_moe_scratch *s) { return s->shared_gate; }
int32_t *wd_moe_scratch_gate_up_partials(wd_moe_scratch *s) { return s->gup; }
int32_t *wd_moe_scratch_down_partials(wd_moe_scratch *s) { return s->dp; }

// Profiling aid: allocates (once) a buffer of 3 x 16 x 8 time stamps (100 MHz counter) that the fused
// dispatches A, B, C fill for workgroup `wg` (per wave, per marked point); returns its device address.
unsigned long long *wd_moe_scratch_trace(wd_moe_scratch *s, int wg) {
    if (!s) return nullptr;
    if (!s->trace) {
        if (hipMalloc(reinterpret_cast<void **>(&s->trace), sizeof(unsigned long long) * 3 * 16 * 8) != hipSuccess) return nullptr;
        (void)hipMemset(s->trace, 0, sizeof(unsigned long long) * 3 * 16 * 8);
    }
    for (int d = 0; d < 3; ++d) {  // earliest-start cells start at the maximum
        const unsigned long long big = ~0ull;
        (void)hipMemcpy(s->trace + (d * 16 + 15) * 8, &big, sizeof(big), hipMemcpyHostToDevice);
        (void)hipMemset(s->trace + (d * 16 + 15) * 8 + 1, 0, sizeof(big));
    }
    s->trace_wg = wg;
    return s->trace;
}

// Profiling aid of the resident stack kernel: 12 x 16 time stamps (100 MHz counter; per wave, per marked point) of
// workgroup `wg` in layer `layer`; returns the device address of the buffer (shared with wd_moe_scratch_trace).
unsigned long long *wd_moe_scratch_trace_resident(wd_moe_scratch *s, int wg, int layer) {
    if (!s) return nullptr;
    const size_t bytes = sizeof(unsigned long long) * kResWgs * 4 * 16;  // also covers the per-layer kernels' 3 x 16 x 8
    if (s->trace && !s->trace_all) {
        (void)hipFree(s->trace);
        s->trace = nullptr;
    }
    if (!s->trace) {
        if (hipMalloc(reinterpret_cast<void **>(&s->trace), bytes) != hipSuccess) return nullptr;
        s->trace_all = true;
    }
    (void)hipMemset(s->trace, 0, bytes);
    s->trace_wg = wg, s->trace_layer = layer;
    return s->trace;
}

int wd_moe_scratch_enable_partials(wd_moe_scratch *s, int gate_type, int down_type) {
    WD_REQUIRE(s != nullptr, "enable partials: null scratch");
    const int pg = partials_per_row(gate_type, s->hidden), pd = partials_per_row(down_type, s->ffn);
    WD_REQUIRE(pg > 0 && pd > 0, "enable partials: unsupported tensor types %d / %d", gate_type, down_type);
    (void)hipFree(s->gup);
    (void)hipFree(s->dp);
    s->gup = s->dp = nullptr;
    WD_HIP(hipMalloc(reinterpret_cast<void **>(&s->gup), sizeof(int32_t) * s->max_k * 2 * s->ffn * pg));
    WD_HIP(hipMalloc(reinterpret_cast<void **>(&s->dp), sizeof(int32_t) * s->max_k * s->hidden * pd));
    s->gup_type = gate_type, s->dp_type = down_type;
    return WD_OK;
}

}  // extern "C"

namespace {

int check_layer(const wd_moe_layer *L, const wd_moe_scratch *s, unsigned flags) {
    WD_REQUIRE(L && s, "MoE layer: null layer or scratch");
    WD_REQUIRE(L->hidden == s->hidden && L->expert_ffn == s->ffn, "MoE layer geometry mismatch: layer %d/%d, scratch %d/%d",
               L->hidden, L->expert_ffn, s->hidden, s->ffn);
    WD_REQUIRE(L->n_experts > 0 && L->n_experts <= s->n_experts, "MoE layer: %d experts exceed the scratch (%d)",
               L->n_experts, s->n_experts);
    WD_REQUIRE(L->top_k > 0 && L->top_k <= s->max_k && L->top_k <= L->n_experts, "MoE layer: top_k %d out of range",
               L->top_k);
    WD_REQUIRE(L->gate_type == L->up_type, "MoE layer: gate and up tensors must share a type (%d vs %d)", L->gate_type,
               L->up_type);
    WD_REQUIRE(consumes_q8k(L->gate_type) || L->gate_type == WD_TYPE_Q8_0 || L->gate_type == WD_TYPE_IQ4_NL,
               "MoE layer: unsupported gate/up type %d", L->gate_type);
    WD_REQUIRE(L->down_type == WD_TYPE_Q8_0 || L->down_type == WD_TYPE_IQ4_NL, "MoE layer: unsupported down type %d",
               L->down_type);
    WD_REQUIRE(L->router != nullptr, "MoE layer: null router");
    // the selection sums the probabilities in groups of eight experts and holds at most 1024 of them (src/qwen38_moe.cuh:686-688)
    if (!(flags & WD_MOE_PRESELECTED))
        WD_REQUIRE(L->n_experts % 8 == 0 && L->n_experts <= 1024,
                   "MoE layer: the router's selection needs n_experts (%d) to be a multiple of 8, at most 1024", L->n_experts);
    if (L->slot_of_expert) {
        WD_REQUIRE(L->slot_pool != nullptr && L->slot_bytes > 0, "MoE layer: slot table without a slot pool");
    } else {
        WD_REQUIRE(L->gate && L->up && L->down, "MoE layer: null expert tensors");
    }
    if (L->shared_gate_inp) WD_REQUIRE(L->shared_gate && L->shared_up && L->shared_down, "MoE layer: incomplete shared expert");
    return WD_OK;
}

MatSrc routed_src(const wd_moe_layer *L, const wd_moe_scratch *s, const int32_t *ids, bool down) {
    MatSrc m{};
    m.ids = ids;
    m.slot_status = s->status;
    m.per_expert = down ? 1 : 2;
    if (L->slot_of_expert) {
        m.slot_of_expert = L->slot_of_expert;
        m.pool = L->slot_pool;
        m.slot_bytes = L->slot_bytes;
        if (down) {
            m.slot_off[0] = L->slot_gate_bytes + L->slot_up_bytes;
        } else {
            m.slot_off[0] = 0;
            m.slot_off[1] = L->slot_gate_bytes;
        }
    } else if (down) {
        m.base[0] = L->down;
        m.stride[0] = L->down_stride;
    } else {
        m.base[0] = L->gate, m.base[1] = L->up;
        m.stride[0] = L->gate_stride, m.stride[1] = L->up_stride;
    }
    return m;
}

template <int TYPE>
void launch_iq(bool part, dim3 grid, hipStream_t st, MatSrc src, int rows, int cols, const int8_t *qs, const float *d,
               float *out, int32_t *partials, int ppr) {
    if (part)
        k_gemv_iq<TYPE, true><<<grid, dim3(256), 0, st>>>(src, rows, cols, qs, d, out, partials, ppr);
    else
        k_gemv_iq<TYPE, false><<<grid, dim3(256), 0, st>>>(src, rows, cols, qs, d, out, nullptr, 0);
}

template <int KIND>
void launch_q8(bool part, dim3 grid, hipStream_t st, MatSrc src, int rows, int cols, const int8_t *qs,
               const uint16_t *d, int act_stride, float *out, int32_t *partials, int ppr) {
    if (part)
        k_gemv_q8<KIND, true><<<grid, dim3(256), 0, st>>>(src, rows, cols, qs, d, act_stride, out, partials, ppr);
    else
        k_gemv_q8<KIND, false><<<grid, dim3(256), 0, st>>>(src, rows, cols, qs, d, act_stride, out, nullptr, 0);
}

// One grouped GEMV of `mats` matrices of `type` ([rows][cols]) against the layer's quantised input
// (shared activation) or against per-matrix Q8_0 activations (act_stride != 0).
int grouped_gemv(int type, MatSrc src, int mats, int rows, int cols, const wd_moe_scratch *s, const int8_t *q0,
                 const uint16_t *d0, int act_stride, float *out, int32_t *partials, hipStream_t st) {
    const dim3 grid((rows + 15) / 16, mats);
    const int ppr = partials_per_row(type, cols);
    const bool part = partials != nullptr;
    switch (type) {
        case WD_TYPE_IQ3_S: launch_iq<21>(part, grid, st, src, rows, cols, s->xk_qs, s->xk_d, out, partials, ppr); break;
        case WD_TYPE_IQ2_S: launch_iq<22>(part, grid, st, src, rows, cols, s->xk_qs, s->xk_d, out, partials, ppr); break;
        case WD_TYPE_Q8_0: launch_q8<0>(part, grid, st, src, rows, cols, q0, d0, act_stride, out, partials, ppr); break;
        case WD_TYPE_IQ4_NL: launch_q8<1>(part, grid, st, src, rows, cols, q0, d0, act_stride, out, partials, ppr); break;
        default: return fail(WD_ERR_UNSUPPORTED, "grouped GEMV: unsupported type %d", type);
    }
    WD_LAUNCH_CHECK();
    return WD_OK;
}

}  // namespace

namespace {

// The hyper-connection form of the residual update: residual is [hc][hidden] and stream c receives
// out * 2 sigmoid(inject[c] / hc) (src/qwen38_hc.cuh:2530-2547).
struct HcSpec {
    const float *inject;
    int hc, round_half;
};

// One layer, one launch per stage.  ids_override (device, k ids) replaces the router's ids while
// keeping its weights; residual (device f32[hidden]) receives residual += layer output.
int layer_staged(const wd_moe_layer *L, const float *d_x, float *d_out, wd_moe_scratch *s, unsigned flags,
                 const int32_t *ids_override, float *residual, float residual_scale, hipStream_t st,
                 const HcSpec *hc = nullptr) {
    const int H = L->hidden, F = L->expert_ffn, E = L->n_experts, k = L->top_k;
    const bool shared = L->shared_gate_inp != nullptr;
    const bool pre = (flags & WD_MOE_PRESELECTED) != 0;

    // 1. router logits (+ the shared expert's gate logit as one more row), softmax/top-k, sigmoid
    if (!pre) {
        {
            SiteScope site(WD_SITE_ROUTER_GEMV, st);
            k_router_gemv<<<dim3((E + (shared ? 1 : 0) + 7) / 8), dim3(256), 0, st>>>(
                L->router, d_x, s->logits, E, H, shared ? L->shared_gate_inp : nullptr, s->shared_gate);
            WD_LAUNCH_CHECK();
        }
        SiteScope site(WD_SITE_ROUTER_TOPK, st);
        k_topk_softmax<<<dim3(1), dim3(64), 0, st>>>(s->logits, E, k, L->expert_scale, s->ids, s->weights,
                                                     shared ? s->shared_gate : nullptr, ids_override);
        WD_LAUNCH_CHECK();
    } else if (shared) {
        SiteScope site(WD_SITE_SHARED_GATE, st);
        k_router_gemv<<<dim3(1), dim3(256), 0, st>>>(L->router, d_x, s->logits, 0, H, L->shared_gate_inp, s->shared_gate);
        WD_LAUNCH_CHECK();
        k_sigmoid1<<<dim3(1), dim3(64), 0, st>>>(s->shared_gate);
        WD_LAUNCH_CHECK();
    }

    // 2. quantise the layer input for the consumers that need it
    {
        SiteScope site(WD_SITE_RX_QUANT, st);
        if (consumes_q8k(L->gate_type)) {
            k_q8_k_quantize<<<dim3((H / 256 + 3) / 4), dim3(256), 0, st>>>(d_x, H / 256, s->xk_qs, s->xk_d, s->xk_bs);
            WD_LAUNCH_CHECK();
        }
        if (!consumes_q8k(L->gate_type) || shared) {
            k_q8_0_quantize<<<dim3((H / 32 + 31) / 32), dim3(256), 0, st>>>(d_x, H / 32, s->x0_qs, s->x0_d);
            WD_LAUNCH_CHECK();
        }
    }

    // 3. gate/up of the k selected experts in one dispatch (2k matrices), then the shared expert's
    const bool part = s->gup != nullptr && s->gup_type == L->gate_type && s->dp_type == L->down_type;
    {
        SiteScope site(WD_SITE_GATE_UP_GEMV, st);
        if (const int rc = grouped_gemv(L->gate_type, routed_src(L, s, s->ids, false), 2 * k, F, H, s, s->x0_qs, s->x0_d, 0,
                                        s->gate_up, part ? s->gup : nullptr, st))
            return rc;
    }
    if (shared) {
        SiteScope site(WD_SITE_SHARED, st);
        MatSrc g{}, u{};
        g.single = L->shared_gate, u.single = L->shared_up;
        float *gu = s->gate_up + static_cast<size_t>(2) * k * F;
        if (const int rc = grouped_gemv(WD_TYPE_Q8_0, g, 1, F, H, s, s->x0_qs, s->x0_d, 0, gu, nullptr, st)) return rc;
        if (const int rc = grouped_gemv(WD_TYPE_Q8_0, u, 1, F, H, s, s->x0_qs, s->x0_d, 0, gu + F, nullptr, st)) return rc;
    }

    // 4. SwiGLU in f32, 5. Q8_0 re-quantisation, for k (+1) experts at once
    const int n_act = k + (shared ? 1 : 0);
    {
        SiteScope site(WD_SITE_SILU, st);
        k_silu_mul_experts<<<dim3((F + 255) / 256, n_act), dim3(256), 0, st>>>(s->gate_up, s->act, F);
        WD_LAUNCH_CHECK();
    }
    {
        SiteScope site(WD_SITE_Q8_QUANT, st);
        k_q8_0_quantize<<<dim3((n_act * F / 32 + 31) / 32), dim3(256), 0, st>>>(s->act, n_act * F / 32, s->act_qs, s->act_d);
        WD_LAUNCH_CHECK();
    }

    // 6. down projections: k routed matrices with their own activations, then the shared expert
    {
        SiteScope site(WD_SITE_DOWN_GEMV, st);
        if (const int rc = grouped_gemv(L->down_type, routed_src(L, s, s->ids, true), k, H, F, s, s->act_qs, s->act_d, F,
                                        s->expert_out, part ? s->dp : nullptr, st))
            return rc;
    }
    if (shared) {
        SiteScope site(WD_SITE_SHARED, st);
        MatSrc d{};
        d.single = L->shared_down;
        if (const int rc = grouped_gemv(WD_TYPE_Q8_0, d, 1, H, F, s, s->act_qs + static_cast<size_t>(k) * F,
                                        s->act_d + static_cast<size_t>(k) * (F / 32), 0, s->down_f32, nullptr, st))
            return rc;
    }

    // 7. ordered weighted sum and the shared branch
    {
        SiteScope site(WD_SITE_ACCUM, st);
        k_combine<<<dim3((H + 255) / 256), dim3(256), 0, st>>>(s->expert_out, s->weights, k, shared ? s->down_f32 : nullptr,
                                                                s->shared_gate, s->accum, d_out, hc ? nullptr : residual,
                                                                residual_scale, H);
        WD_LAUNCH_CHECK();
    }
    if (hc && residual) {
        SiteScope site(WD_SITE_HC_COMBINE, st);
        k_hc_combine<0><<<dim3((H * hc->hc + 255) / 256), dim3(256), 0, st>>>(residual, d_out, nullptr, nullptr, hc->inject, H,
                                                                             hc->hc, hc->round_half);
        WD_LAUNCH_CHECK();
    }
    return WD_OK;
}

LayerArgs fused_args(const wd_moe_layer *L, const float *d_x, float *d_out, wd_moe_scratch *s, unsigned flags,
                     const int32_t *ids_override, float *residual, float residual_scale, int rec = 0,
                     const HcSpec *hc = nullptr) {
    const bool shared = L->shared_gate_inp != nullptr;
    LayerArgs a{};
    a.H = L->hidden, a.F = L->expert_ffn, a.E = L->n_experts, a.k = L->top_k;
    a.w_scale = L->expert_scale;
    a.x = d_x;
    a.router = L->router;
    a.gate_up = routed_src(L, s, s->ids, false);
    a.down = routed_src(L, s, s->ids, true);
    a.sh_inp = L->shared_gate_inp;
    a.sh_gate = L->shared_gate, a.sh_up = L->shared_up, a.sh_down = L->shared_down;
    a.logits = s->logits, a.ids = s->ids, a.weights = s->weights;
    a.ids_override = ids_override;
    a.act = s->act;
    a.shared_gate = s->shared_gate;
    a.expert_out = (flags & WD_MOE_KEEP_EXPERT_OUT) ? s->expert_out : nullptr;
    a.accum = s->accum, a.down_f32 = s->down_f32, a.out = d_out;
    a.residual = residual, a.residual_scale = residual_scale;
    if (hc) a.hc_inject = hc->inject, a.hc = hc->hc, a.hc_round_half = hc->round_half;
    a.preselected = (flags & WD_MOE_PRESELECTED) ? 1 : 0;
    a.dry = (flags & WD_MOE_DRY) ? 1 : 0;
    const int router_rows_n = (a.preselected ? 0 : a.E) + (shared ? 1 : 0);
    a.n_router_wgs = (router_rows_n + 15) / 16;
    a.trace = s->trace, a.trace_wg = s->trace_wg;
    a.arrive = s->arrive;
    a.ids_tagged = s->tagged + static_cast<size_t>(rec % kTagRecords) * kTagCopies * 16;
    a.clear_tagged = 1;
    a.status = s->status;
    a.spin_limit = s->spin_limit;
    // the chunk sums go out of the fused dispatches when the scratch was asked to keep them and the gate/up rows are of
    // the kinds whose fused kernels export them (other layers take the staged dispatches for that)
    if (s->gup && !(flags & WD_MOE_STAGED) && consumes_q8k(L->gate_type) && s->gup_type == L->gate_type && s->dp_type == L->down_type)
        a.gup_part = s->gup, a.down_part = s->dp;
    return a;
}

// Dispatch A: router logits (+ selection by the last router workgroup) and the shared expert's gate/up.
int launch_a(const LayerArgs &a, hipStream_t st) {
    const int grid_a = a.n_router_wgs + (a.sh_inp ? (a.F + 7) / 8 : 0);
    if (grid_a > 0) {
        k_layer_a<<<dim3(grid_a), dim3(512), static_cast<size_t>(a.H) + a.H / 16, st>>>(a);
        WD_LAUNCH_CHECK();
    }
    return WD_OK;
}

// One layer in three dispatches (router + shared gate/up, routed gate/up, down + combine).
template <int TYPE, bool COAL, int NB>
void launch_layer_ab(bool loop, dim3 grid, dim3 block, size_t lds, hipStream_t st, const LayerArgs &m) {
    const bool part = m.gup_part != nullptr;  // the variants that also store the int32 chunk sums
    // (the time stamps are a variant of their own, so that the others run without their tests; no stamps are taken
    // while the chunk sums are exported)
    const bool trace = m.trace != nullptr && !part;
    if (loop && part)
        k_layer_ab<TYPE, COAL, NB, true, true><<<grid, block, lds, st>>>(m);
    else if (loop && trace)
        k_layer_ab<TYPE, COAL, NB, true, false, true><<<grid, block, lds, st>>>(m);
    else if (loop)
        k_layer_ab<TYPE, COAL, NB, true><<<grid, block, lds, st>>>(m);
    else if (part)
        k_layer_ab<TYPE, COAL, NB, false, true><<<grid, block, lds, st>>>(m);
    else if (trace)
        k_layer_ab<TYPE, COAL, NB, false, false, true><<<grid, block, lds, st>>>(m);
    else
        k_layer_ab<TYPE, COAL, NB, false><<<grid, block, lds, st>>>(m);
}
template <int KIND, bool COAL, int NB, bool TWO>
void launch_layer_c(dim3 grid, dim3 block, size_t lds, hipStream_t st, const LayerArgs &a) {
    if (a.down_part)
        k_layer_c<KIND, COAL, NB, TWO, true><<<grid, block, lds, st>>>(a);
    else if (a.trace)
        k_layer_c<KIND, COAL, NB, TWO, false, true><<<grid, block, lds, st>>>(a);
    else
        k_layer_c<KIND, COAL, NB, TWO><<<grid, block, lds, st>>>(a);
}

int layer_fused(const wd_moe_layer *L, const float *d_x, float *d_out, wd_moe_scratch *s, unsigned flags,
                const int32_t *ids_override, float *residual, float residual_scale, hipStream_t st, int rec = 0,
                const HcSpec *hc = nullptr) {
    const int H = L->hidden, F = L->expert_ffn, k = L->top_k;
    const bool shared = L->shared_gate_inp != nullptr;
    const LayerArgs a = fused_args(L, d_x, d_out, s, flags, ids_override, residual, residual_scale, rec, hc);
    const unsigned only = flags & (WD_MOE_ONLY_A | WD_MOE_ONLY_B | WD_MOE_ONLY_C);
    const bool run_a = !only || (only & WD_MOE_ONLY_A), run_b = !only || (only & WD_MOE_ONLY_B);
    const bool iq = consumes_q8k(L->gate_type);
    // router + selection + shared gate/up + routed gate/up in one launch (the routed workgroups wait for the ids
    // inside the dispatch) unless the ids are given, the tensor type has no 512-thread kernel, or the caller
    // asked for the two dispatches apart
    const bool merged = run_a && run_b && !a.preselected && !(flags & WD_MOE_SPLIT_AB) &&
                        (iq || L->gate_type == WD_TYPE_Q8_0);
    if (merged) {
        SiteScope site(WD_SITE_FUSED_AB, st);
        LayerArgs m = a;
        m.n_router_wgs = (a.E + (shared ? 1 : 0) + 7) / 8;  // one router row per wave in the merged dispatch
        // A compute unit holds three of these workgroups.  The router and shared ones leave well before the ids are
        // published, so a few routed ones that have to wait for their places still start in time.  But when the routed
        // ones alone are more than the device holds at once (hidden 2560: 800 against 768), the surplus would start -
        // quantise x, stage the codebooks - only after others have finished: the grid is then cut to what the device
        // holds and the routed workgroups walk the items in a loop (measured at hidden 2560: 36.4 against 37.4 us per layer).
        m.n_routed_items = k * ((F + 7) / 8);
        const int fixed_wgs = m.n_router_wgs + (shared ? (F + 7) / 8 : 0);
        const int capacity = 3 * s->compute_units;
        const int routed_wgs = m.n_routed_items <= capacity - 8 ? m.n_routed_items
                                                                : std::min(m.n_routed_items, std::max(capacity - fixed_wgs, (F + 7) / 8));
        // rows of eight super-blocks on 16-byte boundaries: coalesced fetch with a per-wave staging area behind lds_ab
        auto al16_ = [](const void *p_, size_t v) { return reinterpret_cast<uintptr_t>(p_) % 16 == 0 && v % 16 == 0; };
        // (rows of ten super-blocks are 4-byte aligned then, and F rows end on a 16-byte boundary)
        const bool coal_ab = iq && (H == 2048 || H == 2560) &&
                             (L->slot_of_expert ? al16_(L->slot_pool, L->slot_bytes) && L->slot_gate_bytes % 16 == 0
                                                : al16_(L->gate, L->gate_stride) && al16_(L->up, L->up_stride));
        if (coal_ab && H == 2560) {
            // these variants give a router row two waves, every weight of the row requested at once: twice the router
            // workgroups (they leave long before the routed ones stop waiting, so the routed workgroups keep their number)
            m.n_router_wgs = (a.E + (shared ? 1 : 0) + 3) / 4;
        }
        const int grid_ab = m.n_router_wgs + (shared ? (F + 7) / 8 : 0) + routed_wgs;
        const size_t lds_ab = sizeof(float) * static_cast<size_t>(H) + 16;  // f32 x of the router rows; the quantised x of the others fits inside
        const size_t lds_stage = 16 + 8 * 2 * static_cast<size_t>(H == 2048 ? kIqStageBytes : kIqStage10Bytes);
        const dim3 grid(grid_ab), block(512);
        const bool loop = routed_wgs < m.n_routed_items;
        switch (L->gate_type) {
            case WD_TYPE_IQ3_S:
                if (coal_ab && H == 2048) launch_layer_ab<21, true, 8>(loop, grid, block, lds_ab + lds_stage, st, m);
                else if (coal_ab) launch_layer_ab<21, true, 10>(loop, grid, block, lds_ab + lds_stage, st, m);
                else launch_layer_ab<21, false, 8>(loop, grid, block, lds_ab, st, m);
                break;
            case WD_TYPE_IQ2_S:
                if (coal_ab && H == 2048) launch_layer_ab<22, true, 8>(loop, grid, block, lds_ab + lds_stage, st, m);
                else if (coal_ab) launch_layer_ab<22, true, 10>(loop, grid, block, lds_ab + lds_stage, st, m);
                else launch_layer_ab<22, false, 8>(loop, grid, block, lds_ab, st, m);
                break;
            default: launch_layer_ab<8, false, 8>(loop, grid, block, lds_ab, st, m); break;
        }
        WD_LAUNCH_CHECK();
    } else if (run_a) {
        SiteScope site(WD_SITE_FUSED_A, st);
        if (const int rc = launch_a(a, st)) return rc;
    }
    const size_t lds_b = H + (iq ? sizeof(float) * (H / 256) : sizeof(uint16_t) * (H / 32));
    const int grid_b = k * (L->gate_type == WD_TYPE_IQ4_NL ? (F + 15) / 16 : (F + 7) / 8);
    if (run_b && !merged) {
        SiteScope site(WD_SITE_FUSED_B, st);
        switch (L->gate_type) {
            case WD_TYPE_IQ3_S:
                if (a.gup_part) k_layer_b<21, true><<<dim3(grid_b), dim3(512), lds_b, st>>>(a);
                else k_layer_b<21><<<dim3(grid_b), dim3(512), lds_b, st>>>(a);
                break;
            case WD_TYPE_IQ2_S:
                if (a.gup_part) k_layer_b<22, true><<<dim3(grid_b), dim3(512), lds_b, st>>>(a);
                else k_layer_b<22><<<dim3(grid_b), dim3(512), lds_b, st>>>(a);
                break;
            case WD_TYPE_Q8_0: k_layer_b<8><<<dim3(grid_b), dim3(512), lds_b, st>>>(a); break;
            case WD_TYPE_IQ4_NL: k_layer_b<20><<<dim3(grid_b), dim3(256), lds_b, st>>>(a); break;
            default: return fail(WD_ERR_UNSUPPORTED, "fused layer: unsupported gate/up type %d", L->gate_type);
        }
        WD_LAUNCH_CHECK();
    }
    if (only && !(only & WD_MOE_ONLY_C)) return WD_OK;
    const int n_act = k + (shared ? 1 : 0);
    const int grid_c = (H + 3) / 4;
    // One wave per matrix (k routed and the shared one).  A compute unit holds two such workgroups; when the grid has
    // more than the chip holds at once (hidden > 2048), waves take two matrices each instead, so that the smaller
    // workgroups all run together rather than in two rounds.
    // (With k = 16 and a shared expert there are 17 matrices, more than the 16 waves of a workgroup: halved as well.)
    int waves_c = n_act;
    if (grid_c > 512 || n_act > 16) waves_c = (n_act + 1) / 2;
    const size_t per_wave = (static_cast<size_t>(F) + F / 16 + 15) & ~static_cast<size_t>(15);
    const bool two = waves_c < n_act;  // halved above: n_act <= 2 * waves_c
    // such a wave keeps both quantised activations and the second row group (at most 4 rows of F / 32 34-byte blocks) in LDS
    const size_t lds_c = waves_c * (two ? 2 * per_wave + static_cast<size_t>(4) * (F / 32) * 34 : per_wave) + sizeof(float) * 4 * n_act;
    auto al16 = [](const void *p_, size_t v) { return reinterpret_cast<uintptr_t>(p_) % 16 == 0 && v % 16 == 0; };
    // rows of 16 or 20 blocks in 16-byte aligned groups of four: the coalesced fetch
    const bool coal = (F == 512 || F == 640) && H % 4 == 0 && al16(L->shared_down, 0) &&
                      (L->slot_of_expert ? al16(L->slot_pool, L->slot_bytes) && (L->slot_gate_bytes + L->slot_up_bytes) % 16 == 0
                                         : al16(L->down, L->down_stride));
    const dim3 grid(grid_c), block(64 * waves_c);
    const bool q8 = L->down_type == WD_TYPE_Q8_0;
    SiteScope site(WD_SITE_FUSED_C, st);
    if (coal && two) {
        if (waves_c > 9) return fail(WD_ERR_ARG, "fused layer: %d waves in the paired down dispatch (at most 9)", waves_c);
        if (F == 512 && q8) launch_layer_c<0, true, 16, true>(grid, block, lds_c, st, a);
        else if (F == 512) launch_layer_c<1, true, 16, true>(grid, block, lds_c, st, a);
        else if (q8) launch_layer_c<0, true, 20, true>(grid, block, lds_c, st, a);
        else launch_layer_c<1, true, 20, true>(grid, block, lds_c, st, a);
    } else if (coal && F == 512 && q8)
        launch_layer_c<0, true, 16, false>(grid, block, lds_c, st, a);
    else if (coal && F == 512)
        launch_layer_c<1, true, 16, false>(grid, block, lds_c, st, a);
    else if (coal && q8)
        launch_layer_c<0, true, 20, false>(grid, block, lds_c, st, a);
    else if (coal)
        launch_layer_c<1, true, 20, false>(grid, block, lds_c, st, a);
    else if (q8)
        launch_layer_c<0, false, 16, false>(grid, block, lds_c, st, a);
    else
        launch_layer_c<1, false, 16, false>(grid, block, lds_c, st, a);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

int layer_dispatch(const wd_moe_layer *L, const float *d_x, float *d_out, wd_moe_scratch *s, unsigned flags,
                   const int32_t *ids_override, float *residual, float residual_scale, hipStream_t st, int rec = 0,
                   const HcSpec *hc = nullptr) {
    const bool want_partials = s->gup != nullptr;
    const bool fused_exports = consumes_q8k(L->gate_type) && s->gup_type == L->gate_type && s->dp_type == L->down_type;
    if ((flags & WD_MOE_STAGED) || (want_partials && !fused_exports))
        return layer_staged(L, d_x, d_out, s, flags, ids_override, residual, residual_scale, st, hc);
    return layer_fused(L, d_x, d_out, s, flags, ids_override, residual, residual_scale, st, rec, hc);
}

}  // namespace

extern "C" int wd_moe_layer_f32(const wd_moe_layer *L, const float *d_x, float *d_out, wd_moe_scratch *s,
                                unsigned flags, void *stream) {
    if (const int rc = check_layer(L, s, flags)) return rc;
    WD_REQUIRE(d_x && d_out, "MoE layer: null activation or output pointer");
    SiteScope site(WD_SITE_ROUTED_TOTAL, as_stream(stream));
    return layer_dispatch(L, d_x, d_out, s, flags, nullptr, nullptr, 0.0f, as_stream(stream));
}

extern "C" int wd_moe_layer_hc_f32(const wd_moe_layer *L, const float *d_x, float *d_out, float *d_residual,
                                   const float *d_inject, int hc, int round_half, wd_moe_scratch *s, unsigned flags,
                                   void *stream) {
    if (const int rc = check_layer(L, s, flags)) return rc;
    WD_REQUIRE(d_x && d_out && d_residual && d_inject, "MoE layer with combine: null activation, output, residual or inject pointer");
    WD_REQUIRE(hc >= 1 && hc <= 16, "MoE layer with combine: 1..16 residual streams (got %d)", hc);
    WD_REQUIRE(!(flags & (WD_MOE_ONLY_A | WD_MOE_ONLY_B | WD_MOE_ONLY_C | WD_MOE_DRY)), "MoE layer with combine: measurement flags are not supported");
    const HcSpec spec{d_inject, hc, round_half ? 1 : 0};
    SiteScope site(WD_SITE_ROUTED_TOTAL, as_stream(stream));
    return layer_dispatch(L, d_x, d_out, s, flags, nullptr, d_residual, 0.0f, as_stream(stream), 0, &spec);
}

extern "C" int wd_hc_combine_f32(float *d_residual, const float *d_block_out, const float *d_inject, int hidden, int hc,
                                 int round_half, void *stream) {
    WD_REQUIRE(d_residual && d_block_out && d_inject, "combine: null pointer");
    WD_REQUIRE(hidden > 0 && hc > 0 && static_cast<long long>(hidden) * hc < (1LL << 31), "combine: bad geometry %d x %d", hc, hidden);
    SiteScope site(WD_SITE_HC_COMBINE, as_stream(stream));
    k_hc_combine<0><<<dim3((hidden * hc + 255) / 256), dim3(256), 0, as_stream(stream)>>>(d_residual, d_block_out, nullptr, nullptr,
                                                                                          d_inject, hidden, hc, round_half ? 1 : 0);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

extern "C" int wd_hc_combine_moe_f32(float *d_residual, const float *d_routed, const void *d_shared, int shared_is_half,
                                     const float *d_shared_gate, const float *d_inject, int hidden, int hc, int round_half,
                                     void *stream) {
    WD_REQUIRE(d_residual && d_routed && d_shared && d_shared_gate && d_inject, "combine: null pointer");
    WD_REQUIRE(hidden > 0 && hc > 0 && static_cast<long long>(hidden) * hc < (1LL << 31), "combine: bad geometry %d x %d", hc, hidden);
    SiteScope site(WD_SITE_HC_COMBINE, as_stream(stream));
    const dim3 grid((hidden * hc + 255) / 256), block(256);
    if (shared_is_half)
        k_hc_combine<2><<<grid, block, 0, as_stream(stream)>>>(d_residual, d_routed, d_shared, d_shared_gate, d_inject, hidden, hc, round_half ? 1 : 0);
    else
        k_hc_combine<1><<<grid, block, 0, as_stream(stream)>>>(d_residual, d_routed, d_shared, d_shared_gate, d_inject, hidden, hc, round_half ? 1 : 0);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

extern "C" int wd_shared_expert_f32(const wd_moe_layer *L, const float *d_x, wd_moe_scratch *s, void *stream) {
    WD_REQUIRE(L && s && d_x, "shared expert: null layer, scratch or activation");
    WD_REQUIRE(L->hidden == s->hidden && L->expert_ffn == s->ffn, "shared expert geometry mismatch: layer %d/%d, scratch %d/%d",
               L->hidden, L->expert_ffn, s->hidden, s->ffn);
    WD_REQUIRE(L->shared_gate_inp && L->shared_gate && L->shared_up && L->shared_down, "shared expert: incomplete weights");
    const int H = L->hidden, F = L->expert_ffn, slot = s->max_k;
    const hipStream_t st = as_stream(stream);
    SiteScope site(WD_SITE_SHARED, st);
    k_router_gemv<<<dim3(1), dim3(256), 0, st>>>(L->router, d_x, s->logits, 0, H, L->shared_gate_inp, s->shared_gate);
    WD_LAUNCH_CHECK();
    k_sigmoid1<<<dim3(1), dim3(64), 0, st>>>(s->shared_gate);
    WD_LAUNCH_CHECK();
    k_q8_0_quantize<<<dim3((H / 32 + 31) / 32), dim3(256), 0, st>>>(d_x, H / 32, s->x0_qs, s->x0_d);
    WD_LAUNCH_CHECK();
    MatSrc g{}, u{}, d{};
    g.single = L->shared_gate, u.single = L->shared_up, d.single = L->shared_down;
    float *gu = s->gate_up + static_cast<size_t>(2) * slot * F;
    float *act = s->act + static_cast<size_t>(slot) * F;
    int8_t *aq = s->act_qs + static_cast<size_t>(slot) * F;
    uint16_t *ad = s->act_d + static_cast<size_t>(slot) * (F / 32);
    if (const int rc = grouped_gemv(WD_TYPE_Q8_0, g, 1, F, H, s, s->x0_qs, s->x0_d, 0, gu, nullptr, st)) return rc;
    if (const int rc = grouped_gemv(WD_TYPE_Q8_0, u, 1, F, H, s, s->x0_qs, s->x0_d, 0, gu + F, nullptr, st)) return rc;
    k_silu_mul_experts<<<dim3((F + 255) / 256, 1), dim3(256), 0, st>>>(gu, act, F);
    WD_LAUNCH_CHECK();
    k_q8_0_quantize<<<dim3((F / 32 + 31) / 32), dim3(256), 0, st>>>(act, F / 32, aq, ad);
    WD_LAUNCH_CHECK();
    return grouped_gemv(WD_TYPE_Q8_0, d, 1, H, F, s, aq, ad, 0, s->down_f32, nullptr, st);
}

namespace {

// The hand-off buffers of the resident stack kernel, allocated on first use.
int resident_prepare(wd_moe_scratch *s) {
    if (s->res_block) return WD_OK;
    uint8_t *b = nullptr;
    WD_HIP(hipMalloc(reinterpret_cast<void **>(&b), kHandBytes));
    (void)hipMemset(b, 0xff, kHandEpoch);                        // every hand-off word of both sets "not yet written"
    (void)hipMemset(b + kHandEpoch, 0, kHandBytes - kHandEpoch);  // launches finished
    s->res_block = b;
    return WD_OK;
}

// The device copy of these layer descriptors: the one made for an equal stack before, or a new one (null: none may be
// made now - a graph is being recorded, or the scratch already holds kResMaxDescSets different stacks).
constexpr size_t kResMaxDescSets = 32;
ResidentLayer *resident_descriptors(wd_moe_scratch *s, const std::vector<ResidentLayer> &want, bool capturing) {
    for (const wd_moe_scratch::ResDescSet &d : s->res_sets)
        if (d.shadow.size() == want.size() && std::memcmp(d.shadow.data(), want.data(), sizeof(ResidentLayer) * want.size()) == 0) return d.dev;
    if (capturing || s->res_sets.size() >= kResMaxDescSets) return nullptr;
    wd_moe_scratch::ResDescSet d;
    const size_t desc_bytes = sizeof(ResidentLayer) * kResMaxLayers + sizeof(ResidentViews);
    if (hipMalloc(reinterpret_cast<void **>(&d.dev), desc_bytes) != hipSuccess) return nullptr;
    const ResidentViews v{s->logits, s->weights, s->accum, s->down_f32, s->shared_gate, s->ids};
    if (hipMemcpy(d.dev, want.data(), sizeof(ResidentLayer) * want.size(), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(d.dev + kResMaxLayers, &v, sizeof(v), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(d.dev);
        return nullptr;
    }
    d.shadow = want;
    s->res_sets.push_back(d);
    return d.dev;
}

bool aligned16(const void *p, size_t stride) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && stride % 16 == 0; }

// Whether the stack can run as one resident launch (see wd_resident.cuh for the geometry it is written for).
bool resident_shape(const wd_moe_layer *layers, int n_layers, const wd_moe_scratch *s, unsigned flags) {
    if (flags != 0 || n_layers > kResMaxLayers || s->gup != nullptr) return false;
    const wd_moe_layer &f = layers[0];
    if (f.hidden != kResH || f.expert_ffn != kResF || f.n_experts > 512 || f.n_experts % 8 != 0 || f.top_k > kResMaxK) return false;
    if (!consumes_q8k(f.gate_type) && f.gate_type != WD_TYPE_Q8_0) return false;
    for (int l = 0; l < n_layers; ++l) {
        const wd_moe_layer &L = layers[l];
        if (L.hidden != f.hidden || L.expert_ffn != f.expert_ffn || L.n_experts != f.n_experts || L.top_k != f.top_k) return false;
        if (L.gate_type != f.gate_type || L.up_type != f.gate_type || L.down_type != WD_TYPE_Q8_0 || L.slot_of_expert) return false;
        if (L.gate_stride != f.gate_stride || L.up_stride != f.up_stride || L.down_stride != f.down_stride) return false;
        if ((L.shared_gate_inp != nullptr) != (f.shared_gate_inp != nullptr)) return false;
        if (!aligned16(L.gate, L.gate_stride) || !aligned16(L.up, L.up_stride) || !aligned16(L.down, L.down_stride)) return false;
        if (reinterpret_cast<uintptr_t>(L.router) % 16 != 0) return false;
        if (L.shared_gate_inp && (!aligned16(L.shared_down, 0) || reinterpret_cast<uintptr_t>(L.shared_gate_inp) % 4 != 0)) return false;
    }
    return true;
}

constexpr int kTakePerLayer = 1;  // (not an error code) the stack cannot run as one resident launch

template <int TYPE>
int resident_launch(const ResidentArgs &a, wd_moe_scratch *s, hipStream_t st) {
    if (s->res_fits < 0) {  // both variants of the kernel (with and without the time stamps) must fit
        int plain = 0, stamped = 0;
        // (more dynamic LDS than a kernel may have without asking)
        const hipError_t a0 = hipFuncSetAttribute(reinterpret_cast<const void *>(k_stack_resident<TYPE, false>), hipFuncAttributeMaxDynamicSharedMemorySize, kResLdsBytes);
        const hipError_t a1 = hipFuncSetAttribute(reinterpret_cast<const void *>(k_stack_resident<TYPE, true>), hipFuncAttributeMaxDynamicSharedMemorySize, kResLdsBytes);
        const hipError_t e0 = hipOccupancyMaxActiveBlocksPerMultiprocessor(&plain, k_stack_resident<TYPE, false>, kResThreads, kResLdsBytes);
        const hipError_t e1 = hipOccupancyMaxActiveBlocksPerMultiprocessor(&stamped, k_stack_resident<TYPE, true>, kResThreads, kResLdsBytes);
        s->res_fits = (a0 == hipSuccess && a1 == hipSuccess && e0 == hipSuccess && e1 == hipSuccess && std::min(plain, stamped) * s->compute_units >= kResWgs) ? 1 : 0;
    }
    if (!s->res_fits) return kTakePerLayer;  // the workgroups would wait for each other without all being on the device
    SiteScope site(WD_SITE_STACK_RESIDENT, st);
    if (a.trace)  // (the variant with the time stamps only when they are asked for)
        k_stack_resident<TYPE, true><<<dim3(kResWgs), dim3(kResThreads), kResLdsBytes, st>>>(a);
    else
        k_stack_resident<TYPE, false><<<dim3(kResWgs), dim3(kResThreads), kResLdsBytes, st>>>(a);
    WD_LAUNCH_CHECK();
    return WD_OK;
}

// Routed experts in a slot pool (see ResidentArgs): the layers' gate/up/down point into the pool, their strides are a slot.
struct ResidentSlots {
    const int32_t *rows_trace;   // device [n_layers][k] slot numbers
    const uint32_t *fill_need;   // device [n_layers]
    const uint32_t *fill_done;   // device [n_layers]
    unsigned n_slots;
};

// Returns kTakePerLayer when the stack has to take the per-layer dispatches instead.
int stack_resident(const wd_moe_layer *layers, int n_layers, float *d_x, float *d_layer_out, wd_moe_scratch *s,
                   const int32_t *d_ids_trace, float residual_scale, hipStream_t st, const ResidentSlots *slots = nullptr) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) return kTakePerLayer;
    const bool capturing = cap != hipStreamCaptureStatusNone;
    if (!s->res_block) {
        if (capturing) return kTakePerLayer;  // nothing may be allocated while a graph is recorded
        if (const int rc = resident_prepare(s)) return rc;
    }
    std::vector<ResidentLayer> want(n_layers);
    for (int l = 0; l < n_layers; ++l) {
        const wd_moe_layer &L = layers[l];
        ResidentLayer &d = want[l];
        std::memset(&d, 0, sizeof(d));
        d.router = L.router, d.sh_inp = L.shared_gate_inp;
        d.sh_gate = L.shared_gate, d.sh_up = L.shared_up, d.sh_down = L.shared_down;
        d.gate = L.gate, d.up = L.up, d.down = L.down;
        d.w_scale = L.expert_scale;
    }
    ResidentLayer *const descriptors = resident_descriptors(s, want, capturing);
    if (!descriptors) return kTakePerLayer;
    // a wait of an earlier launch on this scratch ran out: its results were NaN, and so would this launch's be
    if (reinterpret_cast<const volatile int32_t *>(s->h_ids)[16] != 0)
        return fail(WD_ERR_STATE, "MoE stack: a wait inside an earlier resident launch on this scratch ran out (is other work resident on the device?); "
                                  "wd_moe_scratch_set_wait_limit resets the scratch");
    ResidentArgs a{};
    a.layers = descriptors, a.n_layers = n_layers, a.E = layers[0].n_experts, a.k = layers[0].top_k;
    a.shared = layers[0].shared_gate_inp != nullptr;
    a.gate_stride = layers[0].gate_stride, a.up_stride = layers[0].up_stride, a.down_stride = layers[0].down_stride;
    a.x = d_x, a.out = d_layer_out, a.residual_scale = residual_scale, a.ids_trace = d_ids_trace;
    a.row_limit = static_cast<unsigned>(a.E);
    if (slots) {
        if (!d_ids_trace) return kTakePerLayer;  // (the slots of a layer are known before the launch only with a routing trace)
        a.rows_trace = slots->rows_trace, a.fill_need = slots->fill_need, a.fill_done = slots->fill_done, a.row_limit = slots->n_slots;
    }
    a.views = reinterpret_cast<const ResidentViews *>(descriptors + kResMaxLayers);
    a.hand = s->res_block, a.status = s->status, a.spin_limit = s->spin_limit;
    a.status_host = reinterpret_cast<unsigned *>(s->h_ids + 16);
    a.trace = s->trace, a.trace_wg = s->trace_wg, a.trace_layer = s->trace_layer;
    switch (layers[0].gate_type) {
        case WD_TYPE_IQ3_S: return resident_launch<21>(a, s, st);
        case WD_TYPE_IQ2_S: return resident_launch<22>(a, s, st);
        default: return resident_launch<8>(a, s, st);  // Q8_0 gate/up rows
    }
}

}  // namespace

extern "C" int wd_moe_stack_f32(const wd_moe_layer *layers, int n_layers, float *d_x, float *d_layer_out,
                                wd_moe_scratch *s, const int32_t *d_ids_trace, float residual_scale, unsigned flags,
                                void *stream) {
    WD_REQUIRE(layers && n_layers > 0, "MoE stack: no layers");
    WD_REQUIRE(d_x && d_layer_out, "MoE stack: null activation or output pointer");
    for (int l = 0; l < n_layers; ++l) {
        if (const int rc = check_layer(&layers[l], s, flags)) return rc;
    }
    SiteScope site(WD_SITE_STACK_TOTAL, as_stream(stream));
    if (resident_shape(layers, n_layers, s, flags)) {
        const int rc = stack_resident(layers, n_layers, d_x, d_layer_out, s, d_ids_trace, residual_scale, as_stream(stream));
        if (rc != kTakePerLayer) return rc;
    }
    flags &= ~WD_MOE_PER_LAYER;
    const unsigned only = flags & (WD_MOE_ONLY_A | WD_MOE_ONLY_B | WD_MOE_ONLY_C);
    for (int l = 0; l < n_layers; ++l) {
        const int32_t *trace = d_ids_trace ? d_ids_trace + static_cast<size_t>(l) * layers[l].top_k : nullptr;
        if (only && !(only & WD_MOE_ONLY_C) && l % kTagRecords == 0) {
            // no dispatch C to invalidate the published ids: reset all records before they are used again
            const size_t n = static_cast<size_t>(kTagRecords) * kTagCopies * 16;
            k_fill_u32<<<dim3((n + 255) / 256), dim3(256), 0, as_stream(stream)>>>(s->tagged, kTagInvalid, n);
            WD_LAUNCH_CHECK();
        }
        SiteScope layer_site(WD_SITE_ROUTED_TOTAL, as_stream(stream));
        if (const int rc = layer_dispatch(&layers[l], d_x, d_layer_out, s, flags, trace, d_x, residual_scale, as_stream(stream), l))
            return rc;
    }
    return WD_OK;
}

namespace {
// gu_table / down_table: null, or device tables of pointers ([entry][2] gate and up, [entry] down) that take the place of
// the layer's routed tensors, the ids of the pass being entry numbers; tables_aligned: every pointer in them is 16-byte aligned.
int tokens_pass(const wd_moe_layer *L, const float *d_x, float *d_out, int tokens, wd_moe_scratch *const *scratch_per_token,
                unsigned flags, void *stream, const uint8_t *const *gu_table, const uint8_t *const *down_table, bool tables_aligned) {
    WD_REQUIRE(tokens > 0 && tokens <= kMaxTokens, "multi-token pass: 1..%d tokens (got %d)", kMaxTokens, tokens);
    WD_REQUIRE(scratch_per_token != nullptr && d_x && d_out, "multi-token pass: null pointer");
    for (int t = 0; t < tokens; ++t) {
        WD_REQUIRE(scratch_per_token[t] != nullptr, "multi-token pass: null scratch for token %d", t);
        for (int q = 0; q < t; ++q)
            WD_REQUIRE(scratch_per_token[q] != scratch_per_token[t], "multi-token pass: tokens %d and %d share a scratch", q, t);
        if (const int rc = check_layer(L, scratch_per_token[t], flags)) return rc;
    }
    hipStream_t st = as_stream(stream);
    const int H = L->hidden, F = L->expert_ffn, k = L->top_k;
    SiteScope total_site(WD_SITE_TOKENS_TOTAL, st);
    // the union pass over the gate/up tensors needs the IQ types; the multi-token down dispatch needs Q8_0 rows of at
    // most 16 blocks (other down tensors take the one-token dispatch per token, on the activations the union pass left)
    const bool union_path = !(flags & WD_MOE_STAGED) && consumes_q8k(L->gate_type) && tokens * k <= 128 &&
                            scratch_per_token[0]->gup == nullptr &&
                            !(flags & (WD_MOE_ONLY_A | WD_MOE_ONLY_B | WD_MOE_ONLY_C | WD_MOE_DRY));
    const bool down_tokens = L->down_type == WD_TYPE_Q8_0 && F <= 512;
    if (gu_table) WD_REQUIRE(union_path, "multi-token pass on a pointer table: IQ3_S / IQ2_S gate and up tensors, at most 128 (token, expert) pairs, no staging flags");
    if (!union_path) {
        // same results, one pass per token (every pass reads its own experts)
        for (int t = 0; t < tokens; ++t)
            if (const int rc = layer_dispatch(L, d_x + static_cast<size_t>(t) * H, d_out + static_cast<size_t>(t) * H,
                                              scratch_per_token[t], flags, nullptr, nullptr, 0.0f, st))
                return rc;
        return WD_OK;
    }
    TokenArgs ta{};
    ta.T = tokens;
    ta.common = fused_args(L, d_x, d_out, scratch_per_token[0], flags, nullptr, nullptr, 0.0f);
    ta.common.gate_up = routed_src(L, scratch_per_token[0], nullptr, false);  // the kernels pass the expert id themselves
    ta.common.down = routed_src(L, scratch_per_token[0], nullptr, true);
    if (gu_table) {
        ta.common.gate_up.table = gu_table, ta.common.gate_up.per_expert = 2;
        ta.common.down.table = down_table, ta.common.down.per_expert = 1;
    }
    for (int t = 0; t < tokens; ++t) {
        wd_moe_scratch *s = scratch_per_token[t];
        TokenSlots &k_ = ta.tok[t];
        k_.x = d_x + static_cast<size_t>(t) * H, k_.out = d_out + static_cast<size_t>(t) * H;
        k_.logits = s->logits, k_.ids = s->ids, k_.weights = s->weights, k_.act = s->act;
        k_.shared_gate = s->shared_gate, k_.arrive = s->arrive;
        k_.expert_out = (flags & WD_MOE_KEEP_EXPERT_OUT) ? s->expert_out : nullptr;
        k_.accum = s->accum, k_.down_f32 = s->down_f32;
    }
    LayerArgs &a = ta.common;
    a.n_router_wgs = ((a.preselected ? 0 : a.E) + (a.sh_inp ? 1 : 0) + 7) / 8;  // one router row per wave
    const int grid_a = tokens_a_grid(a.n_router_wgs, a.sh_inp ? (F + 7) / 8 : 0).total(tokens);
    if (grid_a > 0) {  // router, selection and shared gate/up of every token
        SiteScope site(WD_SITE_TOKENS_A, st);
        k_tokens_a<<<dim3(grid_a), dim3(512), static_cast<size_t>(H) * 4 + 16, st>>>(ta);
        WD_LAUNCH_CHECK();
    }
    const size_t lds_b = static_cast<size_t>(tokens) * (H + sizeof(float) * (H / 256));
    const int items_b = tokens * k * ((F + 7) / 8);
    const int grid_b = items_b < 512 ? items_b : 512;  // persistent: two workgroups per compute unit walk the items
    // rows of eight or ten super-blocks of aligned tensors: the aligned fetch, one item ahead
    auto al16b = [](const void *p_, size_t v) { return reinterpret_cast<uintptr_t>(p_) % 16 == 0 && v % 16 == 0; };
    const bool coal_b = (H == 2048 || H == 2560) &&
                        (gu_table ? tables_aligned
                                  : (L->slot_of_expert ? al16b(L->slot_pool, L->slot_bytes) && L->slot_gate_bytes % 16 == 0
                                                       : al16b(L->gate, L->gate_stride) && al16b(L->up, L->up_stride)));
    const size_t lds_b_coal = ((lds_b + 15) & ~static_cast<size_t>(15)) + 8 * 2 * static_cast<size_t>(H == 2048 ? kIqStageBytes : kIqStage10Bytes);
    const dim3 gb(grid_b), bb(512);
#define WD_TOKENS_B(TYPE_)                                                                              \
    do {                                                                                                \
        if (coal_b && H == 2048) {                                                                      \
            if (tokens <= 4) k_tokens_b<TYPE_, 4, 8><<<gb, bb, lds_b_coal, st>>>(ta);                   \
            else k_tokens_b<TYPE_, kMaxTokens, 8><<<gb, bb, lds_b_coal, st>>>(ta);                      \
        } else if (coal_b) {                                                                            \
            if (tokens <= 4) k_tokens_b<TYPE_, 4, 10><<<gb, bb, lds_b_coal, st>>>(ta);                  \
            else k_tokens_b<TYPE_, kMaxTokens, 10><<<gb, bb, lds_b_coal, st>>>(ta);                     \
        } else {                                                                                        \
            if (tokens <= 4) k_tokens_b<TYPE_, 4><<<gb, bb, lds_b, st>>>(ta);                           \
            else k_tokens_b<TYPE_, kMaxTokens><<<gb, bb, lds_b, st>>>(ta);                              \
        }                                                                                               \
    } while (0)
    {
        SiteScope site(WD_SITE_TOKENS_B, st);
        if (L->gate_type == WD_TYPE_IQ3_S)
            WD_TOKENS_B(21);
        else
            WD_TOKENS_B(22);
        WD_LAUNCH_CHECK();
    }
#undef WD_TOKENS_B
    // down tensors in aligned groups of four 16- or 20-block rows (either type): the dispatch with the aligned fetch
    auto al16t = [](const void *p_, size_t v) { return reinterpret_cast<uintptr_t>(p_) % 16 == 0 && v % 16 == 0; };
    const bool down_tokens_nb = (F == 512 || F == 640) && H % 8 == 0 && tokens <= 16 &&
                                (!L->shared_down || al16t(L->shared_down, 0)) &&
                                (down_table ? tables_aligned
                                            : (L->slot_of_expert ? al16t(L->slot_pool, L->slot_bytes) && (L->slot_gate_bytes + L->slot_up_bytes) % 16 == 0
                                                                 : al16t(L->down, L->down_stride)));
    SiteScope c_site(WD_SITE_TOKENS_C, st);
    if (down_tokens_nb) {
        const size_t per_wave_n = (static_cast<size_t>(F) + F / 16 + 15) & ~static_cast<size_t>(15);
        const size_t lds_n = 16 * per_wave_n + sizeof(float) * 8 * tokens * (k + 1);
        const dim3 grid(H / 8), block(1024);
        const bool q8 = L->down_type == WD_TYPE_Q8_0;
        if (F == 512 && !q8) k_tokens_c_nb<1, 16><<<grid, block, lds_n, st>>>(ta);
        else if (F == 512) k_tokens_c_nb<0, 16><<<grid, block, lds_n, st>>>(ta);
        else if (q8) k_tokens_c_nb<0, 20><<<grid, block, lds_n, st>>>(ta);
        else k_tokens_c_nb<1, 20><<<grid, block, lds_n, st>>>(ta);
        WD_LAUNCH_CHECK();
        return WD_OK;
    }
    if (!down_tokens) {
        WD_REQUIRE(!down_table, "multi-token pass on a pointer table: this down tensor (type %d, %d columns) has no multi-token dispatch", L->down_type, F);
        for (int t = 0; t < tokens; ++t)
            if (const int rc = layer_fused(L, d_x + static_cast<size_t>(t) * H, d_out + static_cast<size_t>(t) * H, scratch_per_token[t],
                                           flags | WD_MOE_ONLY_C, nullptr, nullptr, 0.0f, st))
                return rc;
        return WD_OK;
    }
    const int waves_c = 16;
    const size_t per_wave = (static_cast<size_t>(F) + F / 16 + 15) & ~static_cast<size_t>(15);
    const size_t lds_c = waves_c * per_wave + sizeof(float) * 8 * tokens * (k + 1);
    k_tokens_c<<<dim3((H + 7) / 8), dim3(64 * waves_c), lds_c, st>>>(ta);
    WD_LAUNCH_CHECK();
    return WD_OK;
}
}  // namespace

extern "C" int wd_moe_layer_tokens_f32(const wd_moe_layer *L, const float *d_x, float *d_out, int tokens,
                                       wd_moe_scratch *const *scratch_per_token, unsigned flags, void *stream) {
    return tokens_pass(L, d_x, d_out, tokens, scratch_per_token, flags, stream, nullptr, nullptr, false);
}

extern "C" int wd_moe_layer_tokens_pairs_f32(const wd_moe_layer *L, const uint8_t *const *h_gate, const uint8_t *const *h_up,
                                             const uint8_t *const *h_down, int n_entries, const float *d_x, float *d_out, int tokens,
                                             wd_moe_scratch *const *scratch_per_token, unsigned flags, void *stream) {
    WD_REQUIRE(L && h_gate && h_up && h_down && scratch_per_token && scratch_per_token[0], "multi-token pass on a pointer table: null argument");
    WD_REQUIRE(n_entries > 0 && n_entries <= kPairEntries, "multi-token pass on a pointer table: 1..%d entries (got %d)", kPairEntries, n_entries);
    WD_REQUIRE(flags & WD_MOE_PRESELECTED, "multi-token pass on a pointer table: the selection (entry numbers) must be in the scratches");
    bool aligned = true;
    for (int i = 0; i < n_entries; ++i) {
        WD_REQUIRE(h_gate[i] && h_up[i] && h_down[i], "multi-token pass on a pointer table: entry %d has a null pointer", i);
        WD_REQUIRE((reinterpret_cast<uintptr_t>(h_gate[i]) | reinterpret_cast<uintptr_t>(h_up[i]) | reinterpret_cast<uintptr_t>(h_down[i])) % 2 == 0,
                   "multi-token pass on a pointer table: entry %d is not 2-byte aligned", i);
        aligned = aligned && (reinterpret_cast<uintptr_t>(h_gate[i]) | reinterpret_cast<uintptr_t>(h_up[i]) | reinterpret_cast<uintptr_t>(h_down[i])) % 16 == 0;
    }
    wd_moe_layer Lt = *L;  // the routed tensors come from the table: the descriptor's own are placeholders for the checks
    Lt.slot_of_expert = nullptr;
    Lt.gate = h_gate[0], Lt.up = h_up[0], Lt.down = h_down[0];
    Lt.n_experts = n_entries < Lt.top_k ? Lt.top_k : n_entries;
    wd_moe_scratch *s = scratch_per_token[0];
    hipStream_t st = as_stream(stream);
    // the table goes up through a ring of pinned entries that this call may have to wait for: not something a graph
    // can record
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    WD_HIP(hipStreamIsCapturing(st, &cap));
    WD_REQUIRE(cap == hipStreamCaptureStatusNone, "multi-token pass on a pointer table: the stream is being captured (the table upload cannot be recorded)");
    if (!s->pair_host)  // once per scratch
        WD_HIP(hipHostMalloc(reinterpret_cast<void **>(&s->pair_host), sizeof(void *) * 3 * kPairEntries * kPairRing, hipHostMallocDefault));
    if (!s->pair_dev) WD_HIP(hipMalloc(reinterpret_cast<void **>(&s->pair_dev), sizeof(void *) * 3 * kPairEntries * kPairRing));
    for (hipEvent_t &ev : s->pair_done)
        if (!ev) WD_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    const int slot = s->pair_next;
    s->pair_next = (slot + 1) % kPairRing;
    if (s->pair_used[slot]) WD_HIP(hipEventSynchronize(s->pair_done[slot]));  // the pass that read this entry of the ring has run
    const uint8_t **h = s->pair_host + static_cast<size_t>(slot) * 3 * kPairEntries, **d = s->pair_dev + static_cast<size_t>(slot) * 3 * kPairEntries;
    for (int i = 0; i < kPairEntries; ++i) {  // entries the caller did not give point at entry 0
        const int from = i < n_entries ? i : 0;
        h[2 * i] = h_gate[from], h[2 * i + 1] = h_up[from], h[2 * kPairEntries + i] = h_down[from];
    }
    WD_HIP(hipMemcpyAsync(d, h, sizeof(void *) * 3 * kPairEntries, hipMemcpyHostToDevice, st));
    const int rc = tokens_pass(&Lt, d_x, d_out, tokens, scratch_per_token, flags, stream, d, d + 2 * kPairEntries, aligned);
    WD_HIP(hipEventRecord(s->pair_done[slot], st));
    s->pair_used[slot] = true;
    return rc;
}
