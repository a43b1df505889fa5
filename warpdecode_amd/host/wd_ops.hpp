// C++ operator surface of the MoE decode path, header-only, over the C ABI of
// include/warpdecode_amd.h.  The names, argument order and error behaviour are those of the
// reference's inline C++ API (namespace wd), so that a caller written against it compiles against
// this header: owning objects are move-only and free device memory in their destructors, cache views
// are borrowed, geometry/type mismatches and device errors throw std::runtime_error, the grouped
// launchers return false when they launched nothing.  A stream is an opaque handle (hipStream_t
// passed as void*), a half scale is 16-bit storage (uint16_t).
//
// Link with -lwarpdecode_amd.  No HIP header is needed to include this file.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <type_traits>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "warpdecode_amd.h"

namespace wd {

using Stream = void *;
using half_bits = uint16_t;

// src/gguf.hpp:26-44
enum class GgmlType : uint32_t {
    F32 = 0,
    F16 = 1,
    Q4_0 = 2,
    Q8_0 = 8,
    Q6_K = 14,
    IQ4_NL = 20,
    IQ3_S = 21,
    IQ2_S = 22,
    BF16 = 30,
};

inline void check(int rc, const char *what) {
    if (rc != WD_OK) throw std::runtime_error(std::string(what) + ": " + wd_last_error());
}

// src/gguf.hpp:268-310
struct TensorInfo {
    std::string name;
    std::vector<uint64_t> dims;  // GGUF order: dims[0] = columns, dims[1] = rows, dims[2] = experts
    GgmlType type = GgmlType::F32;
    uint64_t relative_offset = 0;
    const uint8_t *data = nullptr;

    uint64_t elements() const {
        uint64_t n = 1;
        for (uint64_t d : dims) n *= d;
        return n;
    }
    size_t byte_size() const {
        const uint64_t n = elements();
        if (type == GgmlType::F32) return static_cast<size_t>(n * 4);
        if (type == GgmlType::F16 || type == GgmlType::BF16) return static_cast<size_t>(n * 2);
        const uint64_t cols = dims.empty() ? 0 : dims[0];
        const size_t row = wd_row_bytes(static_cast<int>(type), static_cast<int>(cols));
        if (row == 0 || cols == 0) throw std::runtime_error("tensor size is not a whole number of blocks, or unsupported type: " + name);
        return static_cast<size_t>(n / cols) * row;
    }
};

// Owning device array (DeviceFloatArray of the reference, src/device_buffer.cuh).
template <typename T>
struct DeviceArray {
    T *data = nullptr;
    size_t count = 0;
    DeviceArray() = default;
    explicit DeviceArray(size_t n) { allocate(n); }
    DeviceArray(const DeviceArray &) = delete;
    DeviceArray &operator=(const DeviceArray &) = delete;
    DeviceArray(DeviceArray &&o) noexcept : data(o.data), count(o.count) { o.data = nullptr, o.count = 0; }
    DeviceArray &operator=(DeviceArray &&o) noexcept {
        if (this != &o) {
            reset();
            data = o.data, count = o.count;
            o.data = nullptr, o.count = 0;
        }
        return *this;
    }
    ~DeviceArray() { reset(); }
    void allocate(size_t n) {
        reset();
        void *p = nullptr;
        check(wd_malloc(&p, n * sizeof(T)), "device allocation failed");
        data = static_cast<T *>(p), count = n;
    }
    void upload(const T *host, size_t n) {
        if (n != count) allocate(n);
        check(wd_memcpy_h2d(data, host, n * sizeof(T), nullptr), "host to device copy failed");
    }
    void download(T *host) const { check(wd_memcpy_d2h(host, data, count * sizeof(T), nullptr), "device to host copy failed"); }
    void reset() {
        if (data) wd_free(data);
        data = nullptr, count = 0;
    }
    bool empty() const { return data == nullptr; }
};
using DeviceFloatArray = DeviceArray<float>;

// src/lowbit.cuh:20-66
struct LowBitMatrix {
    int rows = 0;
    int cols = 0;
    GgmlType type = GgmlType::F32;
    uint8_t *data = nullptr;
    size_t bytes = 0;
    bool owns = true;

    LowBitMatrix() = default;
    LowBitMatrix(const LowBitMatrix &) = delete;
    LowBitMatrix &operator=(const LowBitMatrix &) = delete;
    LowBitMatrix(LowBitMatrix &&o) noexcept { take(o); }
    LowBitMatrix &operator=(LowBitMatrix &&o) noexcept {
        if (this != &o) {
            reset();
            take(o);
        }
        return *this;
    }
    ~LowBitMatrix() { reset(); }
    void reset() {
        if (data && owns) wd_free(data);
        data = nullptr, rows = cols = 0, bytes = 0, owns = true;
    }

private:
    void take(LowBitMatrix &o) {
        rows = o.rows, cols = o.cols, type = o.type, data = o.data, bytes = o.bytes, owns = o.owns;
        o.data = nullptr, o.rows = o.cols = 0, o.bytes = 0, o.owns = true;
    }
};

inline bool lowbit_gemv_supported(GgmlType t) {
    return t == GgmlType::Q8_0 || t == GgmlType::IQ4_NL || t == GgmlType::IQ2_S || t == GgmlType::IQ3_S || t == GgmlType::Q4_0 ||
           t == GgmlType::Q6_K;
}

// src/lowbit.cuh:72-86
inline LowBitMatrix borrow_lowbit_matrix(uint8_t *data, int rows, int cols, GgmlType type, size_t bytes) {
    LowBitMatrix out;
    out.data = data, out.rows = rows, out.cols = cols, out.type = type, out.bytes = bytes, out.owns = false;
    return out;
}

// src/lowbit.cuh:88-117
inline LowBitMatrix upload_lowbit_matrix(const TensorInfo &t) {
    if (t.dims.size() != 2) throw std::runtime_error("low-bit GEMV requires a 2D tensor: " + t.name);
    if (!lowbit_gemv_supported(t.type)) throw std::runtime_error("unsupported low-bit GEMV tensor type: " + t.name);
    LowBitMatrix out;
    out.cols = static_cast<int>(t.dims[0]);
    out.rows = static_cast<int>(t.dims[1]);
    out.type = t.type;
    const int quantum = (t.type == GgmlType::IQ2_S || t.type == GgmlType::IQ3_S || t.type == GgmlType::Q6_K) ? 256 : 32;
    if (out.cols <= 0 || out.rows <= 0 || out.cols % quantum != 0) throw std::runtime_error("invalid low-bit matrix shape: " + t.name);
    out.bytes = t.byte_size();
    void *p = nullptr;
    check(wd_malloc(&p, out.bytes), "low-bit matrix allocation failed");
    out.data = static_cast<uint8_t *>(p);
    if (wd_memcpy_h2d(out.data, t.data, out.bytes, nullptr) != WD_OK) {
        out.reset();
        throw std::runtime_error(std::string("low-bit matrix upload failed: ") + wd_last_error());
    }
    return out;
}

// src/matrix.cuh:15-31 (the f16 mirror of the reference is not kept: F32 tensors stay F32)
struct GpuMatrix {
    int rows = 0;
    int cols = 0;
    GgmlType type = GgmlType::F32;
    bool lowbit = false;
    LowBitMatrix low;
    DeviceFloatArray dense_f32;
    GpuMatrix() = default;
    GpuMatrix(const GpuMatrix &) = delete;
    GpuMatrix &operator=(const GpuMatrix &) = delete;
    GpuMatrix(GpuMatrix &&) noexcept = default;
    GpuMatrix &operator=(GpuMatrix &&) noexcept = default;
};

inline bool matrix_has_f32_weights(const GpuMatrix &m) { return !m.lowbit && !m.dense_f32.empty(); }

inline GpuMatrix upload_matrix(const TensorInfo &t) {
    if (t.dims.size() != 2) throw std::runtime_error("matrix upload requires a 2D tensor: " + t.name);
    GpuMatrix m;
    m.cols = static_cast<int>(t.dims[0]), m.rows = static_cast<int>(t.dims[1]), m.type = t.type;
    if (t.type == GgmlType::F32) {
        m.dense_f32.upload(reinterpret_cast<const float *>(t.data), static_cast<size_t>(m.rows) * m.cols);
    } else {
        m.lowbit = true;
        m.low = upload_lowbit_matrix(t);
    }
    return m;
}

// src/expert_cache.cuh:2107-2146
struct ExpertHostSlice {
    const uint8_t *data = nullptr;
    size_t bytes = 0;
    int rows = 0, cols = 0;
    GgmlType type = GgmlType::F32;
};
inline ExpertHostSlice expert_slice(const TensorInfo &t, int expert) {
    if (t.dims.size() != 3) throw std::runtime_error("expert tensor must be 3D: " + t.name);
    const int n_expert = static_cast<int>(t.dims[2]);
    if (expert < 0 || expert >= n_expert) throw std::runtime_error("expert index out of range: " + t.name);
    if (!lowbit_gemv_supported(t.type)) throw std::runtime_error("expert tensor has unsupported low-bit type: " + t.name);
    TensorInfo one;
    one.name = t.name, one.dims = {t.dims[0], t.dims[1]}, one.type = t.type;
    const size_t slice_bytes = one.byte_size();
    if (slice_bytes * static_cast<size_t>(n_expert) != t.byte_size()) throw std::runtime_error("expert tensor is not slice-contiguous: " + t.name);
    ExpertHostSlice out;
    out.data = t.data + slice_bytes * static_cast<size_t>(expert);
    out.bytes = slice_bytes, out.cols = static_cast<int>(t.dims[0]), out.rows = static_cast<int>(t.dims[1]), out.type = t.type;
    return out;
}

// src/qwen38_moe.cuh:547-562
struct Qwen38SharedExpertWeights {
    DeviceFloatArray gate_input_f32;  // f32 [hidden]
    LowBitMatrix gate, up, down;      // Q8_0
};

constexpr int kMoeBatchTokenMax = 8;  // tokens of one batch pass (src/qwen38_moe.cuh:2711 allows 32; larger batches take the serial loop)

// src/qwen38_moe.cuh:1701-2150.  The device buffers belong to the library's scratch object; the accessors
// keep the reference's names for the views a caller reads after a layer pass.
class Qwen38MoeScratch {
public:
    Qwen38MoeScratch() = default;
    Qwen38MoeScratch(const Qwen38MoeScratch &) = delete;
    Qwen38MoeScratch &operator=(const Qwen38MoeScratch &) = delete;
    ~Qwen38MoeScratch() { reset(); }

    void initialize(int n_experts, int k, int hidden, int expert_ffn) {
        if (s_) throw std::runtime_error("MoE scratch already initialized");
        if (n_experts <= 0 || n_experts > 4096 || k <= 0 || k > 16 || k > n_experts || hidden <= 0 || expert_ffn <= 0)
            throw std::runtime_error("invalid MoE scratch geometry");
        check(wd_moe_scratch_create(&s_, hidden, expert_ffn, n_experts, k), "MoE scratch allocation failed");
        n_experts_ = n_experts, k_ = k, hidden_ = hidden, expert_ffn_ = expert_ffn;
        void *p = nullptr;
        // room for a token batch's ids and weights ([kMoeBatchTokenMax][k], as the reference's batch buffers); the word
        // behind the ids receives the status word
        check(wd_malloc_host(&p, sizeof(int) * (kMoeBatchTokenMax * k + 1)), "pinned allocation failed");
        h_ids_ = static_cast<int *>(p);
        h_ids_[kMoeBatchTokenMax * k] = 0;
        check(wd_malloc_host(&p, sizeof(float) * kMoeBatchTokenMax * k), "pinned allocation failed");
        h_weights_ = static_cast<float *>(p);
    }
    void reset() {
        if (s_) wd_moe_scratch_destroy(s_);
        if (h_ids_) wd_free_host(h_ids_);
        if (h_weights_) wd_free_host(h_weights_);
        s_ = nullptr, h_ids_ = nullptr, h_weights_ = nullptr;
        moe_out_.reset(), x_f32_.reset(), trace_.reset();
    }
    float *moe_out_f32() {
        if (moe_out_.empty()) moe_out_.allocate(static_cast<size_t>(hidden_));
        return moe_out_.data;
    }
    // the layer's input widened to float, for callers that hold it as half
    float *x_f32() {
        if (x_f32_.empty()) x_f32_.allocate(static_cast<size_t>(hidden_));
        return x_f32_.data;
    }
    // src/qwen38_moe.cuh:1769-1775: half [k][hidden], the selected experts' down outputs of a capturing run
    half_bits *selected_output_trace() {
        if (trace_.empty()) trace_.allocate(static_cast<size_t>(k_) * hidden_);
        return trace_.data;
    }
    int n_experts() const { return n_experts_; }
    int k() const { return k_; }
    int hidden() const { return hidden_; }
    int expert_ffn() const { return expert_ffn_; }
    float *d_logits() const { return wd_moe_scratch_logits(s_); }
    int *d_ids() const { return wd_moe_scratch_ids(s_); }
    float *d_weights() const { return wd_moe_scratch_weights(s_); }
    float *d_accum() const { return wd_moe_scratch_accum(s_); }
    float *d_shared_gate() const { return wd_moe_scratch_shared_gate(s_); }
    float *down_f32() const { return wd_moe_scratch_down_f32(s_); }
    float *rx_batch_gate_up() const { return wd_moe_scratch_gate_up(s_); }
    float *rx_batch_act() const { return wd_moe_scratch_act(s_); }
    int8_t *rx_batch_q8_0_values() const { return wd_moe_scratch_act_qs(s_); }
    half_bits *rx_batch_q8_0_scales() const { return wd_moe_scratch_act_scales(s_); }
    float *rx_batch_down() const { return wd_moe_scratch_expert_out(s_); }
    int *h_ids() const { return h_ids_; }
    // The scratch's status word travels to the host with the next synchronisation of `stream`; afterwards
    // throw_if_failed() reports a layer pass on this scratch whose results are invalid (a bounded wait that ran out,
    // an expert that had no slot).
    void queue_status_copy(Stream stream) {
        check(wd_memcpy_d2h(h_ids_ + kMoeBatchTokenMax * k_, wd_moe_scratch_status_word(s_), sizeof(int), stream), "status copy failed");
    }
    void throw_if_failed() const {
        const int st = h_ids_[kMoeBatchTokenMax * k_];
        if (st == 1) throw std::runtime_error("MoE layer pass failed: a wait between its workgroups ran out");
        if (st == 2) throw std::runtime_error("MoE layer pass failed: an expert without a cache slot was selected");
        if (st != 0) throw std::runtime_error("MoE layer pass failed");
    }
    float *h_weights() const { return h_weights_; }
    wd_moe_scratch *handle() const { return s_; }

private:
    wd_moe_scratch *s_ = nullptr;
    int n_experts_ = 0, k_ = 0, hidden_ = 0, expert_ffn_ = 0;
    int *h_ids_ = nullptr;
    float *h_weights_ = nullptr;
    DeviceFloatArray moe_out_, x_f32_;
    DeviceArray<half_bits> trace_;
};

// src/expert_cache.cuh:76-115 (the file-backed staging knobs have no meaning here: sources are host memory)
struct ExpertCacheOptions {
    bool stats = false;
    bool layer_evict = false;
    int layer_count = 0;
    int prefetch_depth = 0;  // layers of read-ahead for file-backed experts (src/expert_cache.cuh:105-112); 0 = off
    int prefetch_slots = 0;  // 0 = prefetch_depth * 16
};

// src/expert_cache.cuh:2148-2154
struct ExpertDeviceWeights {
    LowBitMatrix gate, up, down;  // borrowed views of one slot
    bool cache_hit = false;
    size_t slot = 0;
};

// src/expert_cache.cuh:2156-2536
class GpuExpertCache {
public:
    GpuExpertCache() = default;
    GpuExpertCache(const GpuExpertCache &) = delete;
    GpuExpertCache &operator=(const GpuExpertCache &) = delete;
    GpuExpertCache(GpuExpertCache &&o) noexcept { *this = std::move(o); }
    GpuExpertCache &operator=(GpuExpertCache &&o) noexcept {
        if (this != &o) {
            release();
            c_ = o.c_, n_slots_ = o.n_slots_, slot_bytes_ = o.slot_bytes_, gate_bytes_ = o.gate_bytes_, up_bytes_ = o.up_bytes_,
            down_bytes_ = o.down_bytes_, n_experts_ = o.n_experts_, n_layers_ = o.n_layers_;
            g_ = o.g_, u_ = o.u_, d_ = o.d_;
            reg_ = std::move(o.reg_);
            o.c_ = nullptr;
        }
        return *this;
    }
    ~GpuExpertCache() { release(); }

    void initialize(size_t capacity_mib, const TensorInfo &sample_gate, const TensorInfo &sample_up, const TensorInfo &sample_down,
                    size_t gate_capacity_bytes = 0, size_t up_capacity_bytes = 0, size_t down_capacity_bytes = 0,
                    const ExpertCacheOptions &options = ExpertCacheOptions{}) {
        if (c_) throw std::runtime_error("expert cache already initialized");
        if (capacity_mib == 0) throw std::runtime_error("expert cache capacity is zero");
        g_ = expert_slice(sample_gate, 0), u_ = expert_slice(sample_up, 0), d_ = expert_slice(sample_down, 0);
        gate_bytes_ = gate_capacity_bytes ? gate_capacity_bytes : g_.bytes;
        up_bytes_ = up_capacity_bytes ? up_capacity_bytes : u_.bytes;
        down_bytes_ = down_capacity_bytes ? down_capacity_bytes : d_.bytes;
        if (gate_bytes_ < g_.bytes || up_bytes_ < u_.bytes || down_bytes_ < d_.bytes)
            throw std::runtime_error("expert cache slot capacity is smaller than sample tensors");
        slot_bytes_ = gate_bytes_ + up_bytes_ + down_bytes_;
        if (slot_bytes_ == 0) throw std::runtime_error("expert cache slot is empty");
        const size_t capacity_bytes = capacity_mib * 1024ull * 1024ull;
        if (capacity_bytes / slot_bytes_ == 0) throw std::runtime_error("expert cache capacity is smaller than one expert slot");
        n_experts_ = static_cast<int>(sample_gate.dims[2]);
        n_layers_ = options.layer_count > 0 ? options.layer_count : 128;
        check(wd_expert_cache_create(&c_, capacity_bytes, gate_bytes_, up_bytes_, down_bytes_, n_layers_, n_experts_,
                                     options.layer_evict ? 1 : 0),
              "expert cache allocation failed");
        wd_expert_cache_stats st{};
        wd_expert_cache_get_stats(c_, &st);
        n_slots_ = static_cast<size_t>(st.slots);
        if (options.prefetch_depth > 0)
            check(wd_expert_cache_set_read_ahead(c_, options.prefetch_depth, options.prefetch_slots), "expert read-ahead setup failed");
    }
    // layers of read-ahead in force (src/expert_cache.cuh:2229)
    void set_prefetch_depth(int depth, int slots = 0) { check(wd_expert_cache_set_read_ahead(c_, depth, slots), "expert read-ahead setup failed"); }

    size_t slot_count() const { return n_slots_; }
    size_t slot_bytes() const { return slot_bytes_; }
    size_t resident_count() const {
        wd_expert_cache_stats st{};
        if (c_) wd_expert_cache_get_stats(c_, &st);
        return static_cast<size_t>(st.resident);
    }
    wd_expert_cache_stats stats() const {
        wd_expert_cache_stats st{};
        if (c_) wd_expert_cache_get_stats(c_, &st);
        return st;
    }

    // Host sources of a layer's 3-D expert tensors (pinned memory makes the fills asynchronous).
    void register_layer_experts(int layer, const TensorInfo &gate, const TensorInfo &up, const TensorInfo &down) {
        if (layer < 0) return;
        if (!c_) throw std::runtime_error("expert cache is not initialized");
        if (registered(layer)) return;
        expert_slice(gate, 0), expert_slice(up, 0), expert_slice(down, 0);
        check(wd_expert_cache_register_layer(c_, layer, gate.data, up.data, down.data), "expert cache layer registration failed");
        if (reg_.size() <= static_cast<size_t>(layer)) reg_.resize(static_cast<size_t>(layer) + 1, 0);
        reg_[static_cast<size_t>(layer)] = 1;
    }

    // Fused gate_up tensor (dims {hidden, 2 * ffn, experts}: gate rows, then up rows, per expert) as the source of
    // a layer (reference: GpuFusedExpertCache, src/expert_cache.cuh:2546-2882).  The slot keeps gate | up | down.
    void register_layer_fused(int layer, const TensorInfo &gate_up, const TensorInfo &down) {
        if (layer < 0) return;
        if (!c_) throw std::runtime_error("expert cache is not initialized");
        if (registered(layer)) return;
        const ExpertHostSlice gu = expert_slice(gate_up, 0);
        expert_slice(down, 0);
        if (gu.rows % 2 != 0 || gu.bytes != gate_bytes_ + up_bytes_) throw std::runtime_error("fused gate_up tensor does not match the cache's slot layout: " + gate_up.name);
        check(wd_expert_cache_register_layer_strided(c_, layer, gate_up.data, gate_up.data + gate_bytes_, down.data, gu.bytes, gu.bytes, down_bytes_),
              "expert cache layer registration failed");
        if (reg_.size() <= static_cast<size_t>(layer)) reg_.resize(static_cast<size_t>(layer) + 1, 0);
        reg_[static_cast<size_t>(layer)] = 1;
    }

    // Makes every expert of a registered layer resident.  With room for all experts of all layers (the
    // normal case with 288 GB of HBM) nothing is ever evicted and layer passes need no host round trip.
    void preload_layer(int layer, Stream stream) {
        if (!registered(layer)) throw std::runtime_error("expert cache layer is not registered");
        for (int e0 = 0; e0 < n_experts_; e0 += 16) {
            int32_t ids[16];
            const int n = std::min(16, n_experts_ - e0);
            for (int i = 0; i < n; ++i) ids[i] = e0 + i;
            check(wd_expert_cache_acquire(c_, layer, ids, n, nullptr, stream), "expert cache preload failed");
        }
        reg_[static_cast<size_t>(layer)] = 2;
    }
    // True when the layer was preloaded and no slot has been recycled since the cache was created.
    bool layer_resident(int layer) const { return registered(layer) && reg_[static_cast<size_t>(layer)] == 2 && stats().evictions == 0; }

    // One expert; the views stay valid until the slot is recycled by a later acquire.
    ExpertDeviceWeights acquire(int layer, int expert, const TensorInfo &gate, const TensorInfo &up, const TensorInfo &down, Stream stream) {
        if (!c_) throw std::runtime_error("expert cache is not initialized");
        register_layer_experts(layer, gate, up, down);
        const int32_t id = expert;
        uint8_t hit = 0;
        check(wd_expert_cache_acquire(c_, layer, &id, 1, &hit, stream), "expert cache acquire failed");
        return view(layer, expert, hit != 0);
    }

    // The k experts of one layer pass at once (they are guaranteed to stay resident together).
    void acquire_ids(int layer, const int *h_ids, int k, Stream stream, uint8_t *hit_out = nullptr) {
        if (!c_) throw std::runtime_error("expert cache is not initialized");
        check(wd_expert_cache_acquire(c_, layer, h_ids, k, hit_out, stream), "expert cache acquire failed");
    }

    ExpertDeviceWeights view(int layer, int expert, bool hit) const {
        const long long slot = wd_expert_cache_slot_of(c_, layer, expert);
        if (slot < 0) throw std::runtime_error("expert is not resident");
        uint8_t *base = const_cast<uint8_t *>(wd_expert_cache_pool(c_)) + static_cast<size_t>(slot) * slot_bytes_;
        ExpertDeviceWeights w;
        w.gate = borrow_lowbit_matrix(base, g_.rows, g_.cols, g_.type, g_.bytes);
        w.up = borrow_lowbit_matrix(base + gate_bytes_, u_.rows, u_.cols, u_.type, u_.bytes);
        w.down = borrow_lowbit_matrix(base + gate_bytes_ + up_bytes_, d_.rows, d_.cols, d_.type, d_.bytes);
        w.cache_hit = hit, w.slot = static_cast<size_t>(slot);
        return w;
    }

    const int32_t *slot_table(int layer) const { return wd_expert_cache_slot_table(c_, layer); }
    const uint8_t *pool() const { return wd_expert_cache_pool(c_); }
    size_t gate_bytes() const { return gate_bytes_; }
    size_t up_bytes() const { return up_bytes_; }
    wd_expert_cache *handle() const { return c_; }

private:
    bool registered(int layer) const { return layer >= 0 && static_cast<size_t>(layer) < reg_.size() && reg_[static_cast<size_t>(layer)] != 0; }
    void release() {
        if (c_) wd_expert_cache_destroy(c_);
        c_ = nullptr;
    }
    wd_expert_cache *c_ = nullptr;
    size_t n_slots_ = 0, slot_bytes_ = 0, gate_bytes_ = 0, up_bytes_ = 0, down_bytes_ = 0;
    int n_experts_ = 0, n_layers_ = 0;
    ExpertHostSlice g_, u_, d_;
    std::vector<char> reg_;
};

// ---- operators -----------------------------------------------------------------------------------

// src/lowbit.cuh:873-891
inline void launch_q8_k_quantize_f32(const float *x, int elements, int8_t *qs, float *scales, int16_t *bsums, Stream stream, int /*threads*/ = 256) {
    if (elements <= 0 || elements % 256 != 0) throw std::runtime_error("Q8_K activation quantisation needs a multiple of 256 elements");
    check(wd_q8_k_quantize_f32(x, elements, qs, scales, bsums, stream), "Q8_K quantisation failed");
}

// src/qwen38_moe.cuh:1470-1481
inline void q38_moe_quantize_activation_q8_0(const float *input, int elements, int8_t *quantized, half_bits *scales, Stream stream) {
    check(wd_q8_0_quantize_f32(input, elements, quantized, scales, stream), "Q8_0 quantisation failed");
}

// src/warodecode.cu:1504-1520 (the dense Q4_0 path's activation quantiser: half input)
inline void launch_q8_0_quantize_half(const half_bits *x, int elements, int8_t *quantized, half_bits *scales, Stream stream) {
    check(wd_q8_0_quantize_f16(x, elements, quantized, scales, stream), "Q8_0 quantisation of half input failed");
}

// src/lowbit.cuh:251-285: the activation buffer of the plain Q8_0 x Q8_1 GEMV
class Q8_1Buffer {
public:
    Q8_1Buffer() = default;
    Q8_1Buffer(const Q8_1Buffer &) = delete;
    Q8_1Buffer &operator=(const Q8_1Buffer &) = delete;
    ~Q8_1Buffer() { reset(); }

    void initialize(int elements) {
        if (values_) throw std::runtime_error("Q8_1 buffer already initialized");
        if (elements <= 0 || elements % 32 != 0) throw std::runtime_error("Q8_1 input must be a positive multiple of 32");
        void *p = nullptr;
        check(wd_malloc(&p, static_cast<size_t>(elements)), "Q8_1 values allocation failed");
        values_ = static_cast<int8_t *>(p);
        if (wd_malloc(&p, static_cast<size_t>(elements / 32) * sizeof(half_bits)) != WD_OK) {
            reset();
            throw std::runtime_error(std::string("Q8_1 scales allocation failed: ") + wd_last_error());
        }
        scales_ = static_cast<half_bits *>(p);
        elements_ = elements;
    }
    int elements() const { return elements_; }
    int8_t *values() const { return values_; }
    half_bits *scales() const { return scales_; }

private:
    void reset() {
        if (values_) wd_free(values_);
        if (scales_) wd_free(scales_);
        values_ = nullptr, scales_ = nullptr, elements_ = 0;
    }
    int elements_ = 0;
    int8_t *values_ = nullptr;
    half_bits *scales_ = nullptr;
};

// src/lowbit.cuh:343-362: quantise the input to Q8_1, then one row sum per output (blocks in ascending order)
inline void launch_q8_0_gemv_q8_1_f32(const LowBitMatrix &weights, const float *input, float *output, Q8_1Buffer &scratch, Stream stream) {
    if (weights.type != GgmlType::Q8_0 || weights.rows <= 0 || weights.cols > scratch.elements() || weights.cols % 32 != 0)
        throw std::runtime_error("Q8_0 x Q8_1 GEMV geometry mismatch");
    check(wd_q8_1_quantize_f32(input, weights.cols, scratch.values(), scratch.scales(), stream), "Q8_1 quantisation failed");
    check(wd_gemv_q8_0_q8_1_f32(weights.data, weights.rows, weights.cols, scratch.values(), scratch.scales(), output, nullptr, stream),
          "Q8_0 x Q8_1 GEMV failed");
}

// The slot pool's default size for a device with `vram_bytes` of memory: three quarters of the card minus 8 GiB, at least
// 512 MiB, at most 64 GiB; WARODECODE_EXPERT_CACHE_MIB overrides it (src/qwen38_tuning.hpp:88-116: 40 GB -> 22 GiB,
// 80 GB -> 52 GiB).  A device that holds the whole model needs no pool at all: the layer calls take resident tensors.
inline int default_expert_cache_mib(size_t vram_bytes) {
    long long cache = static_cast<long long>(vram_bytes >> 20) * 3 / 4 - 8 * 1024;
    if (cache < 512) cache = 512;
    if (cache > 64 * 1024) cache = 64 * 1024;
    if (const char *v = std::getenv("WARODECODE_EXPERT_CACHE_MIB")) {
        const int mib = std::atoi(v);
        if (mib > 0) cache = mib;
    }
    return static_cast<int>(cache);
}
// How many layers ahead the expert read-ahead works, by device memory (src/qwen38_tuning.hpp:97-112).
inline int default_expert_prefetch_depth(size_t vram_bytes) {
    const long long mib = static_cast<long long>(vram_bytes >> 20);
    return mib >= 120 * 1024 ? 3 : (mib >= 40 * 1024 ? 2 : 1);
}

// Site profiler (src/qwen38_moe.cuh:296-535): the reference's site numbers, its process-wide profiler object and its
// scope bracket, over the library's profiler.  As there, WARODECODE_MOE_PROFILE=1 switches it on when the object is
// first used and the summary goes to stderr when the process ends; the library brackets its own dispatches while it
// is on (the sites beyond kQ38MoeSiteCount), a caller brackets the regions of its own code with Q38MoeKernelScope and
// calls flush_token() once per token after its stream synchronisation.
enum Q38MoeSite : int {
    kQ38MoeSiteStageTotal = WD_SITE_STAGE_TOTAL,
    kQ38MoeSiteRoutedTotal = WD_SITE_ROUTED_TOTAL,
    kQ38MoeSiteRouter = WD_SITE_ROUTER,
    kQ38MoeSiteRouterQuant = WD_SITE_ROUTER_QUANT,
    kQ38MoeSiteRouterGemv = WD_SITE_ROUTER_GEMV,
    kQ38MoeSiteRouterTopk = WD_SITE_ROUTER_TOPK,
    kQ38MoeSiteRouterD2h = WD_SITE_ROUTER_D2H,
    kQ38MoeSiteRouterSync = WD_SITE_ROUTER_SYNC,
    kQ38MoeSiteAccumZero = WD_SITE_ACCUM_ZERO,
    kQ38MoeSiteRxQuant = WD_SITE_RX_QUANT,
    kQ38MoeSiteAcquire = WD_SITE_ACQUIRE,
    kQ38MoeSitePtrH2d = WD_SITE_PTR_H2D,
    kQ38MoeSiteBatchTotal = WD_SITE_BATCH_TOTAL,
    kQ38MoeSiteGateUpGemv = WD_SITE_GATE_UP_GEMV,
    kQ38MoeSiteSilu = WD_SITE_SILU,
    kQ38MoeSiteQ8Quant = WD_SITE_Q8_QUANT,
    kQ38MoeSiteDownGemv = WD_SITE_DOWN_GEMV,
    kQ38MoeSiteAccum = WD_SITE_ACCUM,
    kQ38MoeSiteCapture = WD_SITE_CAPTURE,
    kQ38MoeSiteLoopTotal = WD_SITE_LOOP_TOTAL,
    kQ38MoeSiteFinish = WD_SITE_FINISH,
    kQ38MoeSiteShared = WD_SITE_SHARED,
    kQ38MoeSiteSharedGate = WD_SITE_SHARED_GATE,
    kQ38MoeSiteMirror = WD_SITE_MIRROR,
    kQ38MoeSiteCount = WD_PROFILE_FIRST_OWN_SITE
};
inline const char *q38_moe_site_name(int site) { return wd_profile_site_name(site); }

struct Q38MoeSiteStat {
    unsigned long long calls = 0;
    double total_ms = 0.0;
    double total_host_ms = 0.0;
    unsigned long long overflow = 0;
    unsigned long long elapsed_fail = 0;
    unsigned long long recorded = 0;
};

class Q38MoeKernelProfiler {
public:
    static Q38MoeKernelProfiler &instance() {
        static Q38MoeKernelProfiler profiler;
        return profiler;
    }
    bool enabled() const { return wd_profile_enabled() != 0; }
    void mark_begin(int site, Stream stream) {
        if (site >= 0 && site < WD_PROFILE_SITE_COUNT) (void)wd_profile_begin(site, stream);
    }
    void mark_end(int site, Stream stream) {
        if (site >= 0 && site < WD_PROFILE_SITE_COUNT) (void)wd_profile_end(site, stream);
    }
    void flush_token() { check(wd_profile_flush_token(), "profiler flush"); }
    Q38MoeSiteStat site(int site_index) const {
        wd_profile_site_stat raw{};
        check(wd_profile_site(site_index, &raw, nullptr), "profiler site");
        Q38MoeSiteStat out;
        out.calls = raw.calls, out.total_ms = raw.device_ms, out.total_host_ms = raw.host_ms;
        out.overflow = raw.dropped, out.elapsed_fail = raw.unreadable, out.recorded = raw.recorded;
        return out;
    }
    std::string summary() const {
        std::string text(wd_profile_report(nullptr, 0), '\0');
        if (!text.empty()) wd_profile_report(&text[0], text.size() + 1);
        return text;
    }
    void print_summary() const {
        if (!enabled()) return;
        wd_profile_site_stat raw{};
        unsigned long long tokens = 0;
        if (wd_profile_site(0, &raw, &tokens) != WD_OK || tokens == 0) return;
        std::fputs(summary().c_str(), stderr);
    }

private:
    Q38MoeKernelProfiler() {
        const char *v = std::getenv("WARODECODE_MOE_PROFILE");
        if (v != nullptr && v[0] != '\0' && v[0] != '0') (void)wd_profile_enable(1);
    }
    ~Q38MoeKernelProfiler() { print_summary(); }
    Q38MoeKernelProfiler(const Q38MoeKernelProfiler &) = delete;
    Q38MoeKernelProfiler &operator=(const Q38MoeKernelProfiler &) = delete;
};

// RAII bracket for one region of a MoE layer.
class Q38MoeKernelScope {
public:
    Q38MoeKernelScope(int site, Stream stream) : site_(site), stream_(stream) {
        Q38MoeKernelProfiler::instance().mark_begin(site_, stream_);
    }
    ~Q38MoeKernelScope() { Q38MoeKernelProfiler::instance().mark_end(site_, stream_); }
    Q38MoeKernelScope(const Q38MoeKernelScope &) = delete;
    Q38MoeKernelScope &operator=(const Q38MoeKernelScope &) = delete;

private:
    int site_;
    Stream stream_;
};

// src/qwen38_moe.cuh:247-263
inline void launch_q38_router_gemv_f32(const GpuMatrix &w, const float *x, float *y, Stream stream, int threads = 256) {
    if (!matrix_has_f32_weights(w)) throw std::runtime_error("router F32 warp GEMV requires an F32 dense matrix");
    if (threads < 32 || threads % 32 != 0) throw std::runtime_error("router F32 warp GEMV threads must be a multiple of 32");
    check(wd_router_gemv_f32(w.dense_f32.data, x, y, w.rows, w.cols, stream), "router GEMV failed");
}

// src/qwen38_moe.cuh:1065-1090
inline void q38_launch_topk_softmax(const float *logits, int n_experts, int k, float expert_scale, int *ids, float *weights, Stream stream) {
    check(wd_topk_softmax(logits, n_experts, k, expert_scale, ids, weights, stream), "router top-k failed");
}

// src/lowbit.cuh:1483-1499, :1181-1197
inline void launch_iq3_s_gemv_q8_k_f32(const LowBitMatrix &w, const int8_t *act, const float *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    if (w.type != GgmlType::IQ3_S || w.rows <= 0 || w.cols <= 0 || w.cols % 256 != 0) throw std::runtime_error("IQ3_S x Q8_K GEMV geometry mismatch");
    check(wd_gemv_q8_k_f32(WD_TYPE_IQ3_S, w.data, w.rows, w.cols, act, act_scales, out, nullptr, stream), "IQ3_S GEMV failed");
}
inline void launch_iq2_s_gemv_q8_k_f32(const LowBitMatrix &w, const int8_t *act, const float *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    if (w.type != GgmlType::IQ2_S || w.rows <= 0 || w.cols <= 0 || w.cols % 256 != 0) throw std::runtime_error("IQ2_S x Q8_K GEMV geometry mismatch");
    check(wd_gemv_q8_k_f32(WD_TYPE_IQ2_S, w.data, w.rows, w.cols, act, act_scales, out, nullptr, stream), "IQ2_S GEMV failed");
}
// src/lowbit.cuh:2615-2636
inline void launch_q6_k_gemv_q8_k_f32(const LowBitMatrix &w, const int8_t *act, const float *act_scales, const int16_t *act_sums, float *out, Stream stream, int threads = 256) {
    if (w.type != GgmlType::Q6_K || w.rows <= 0 || w.cols <= 0 || w.cols % 256 != 0) throw std::runtime_error("Q6_K x Q8_K GEMV geometry mismatch");
    if (threads < 32 || threads % 32 != 0) throw std::runtime_error("Q6_K x Q8_K GEMV threads must be a multiple of 32");
    check(wd_gemv_q6_k_q8_k_f32(w.data, w.rows, w.cols, act, act_scales, act_sums, out, nullptr, stream), "Q6_K GEMV failed");
}

// Q8_K image of the head's activation; a few kilobytes kept for the life of the process and never shrunk or moved
// while a launch may still read it (a larger request allocates a new one and leaves the old in place).
// src/lowbit.cuh:2638-2710
struct LowBitHeadQ8KScratch {
    int cols = 0;
    int8_t *quants = nullptr;
    float *scales = nullptr;
    int16_t *sums = nullptr;
};
inline LowBitHeadQ8KScratch &lowbit_head_q8_k_scratch() {
    static LowBitHeadQ8KScratch scratch;
    return scratch;
}
inline void lowbit_head_q8_k_reserve(int cols) {
    LowBitHeadQ8KScratch &s = lowbit_head_q8_k_scratch();
    if (cols <= s.cols) return;
    LowBitHeadQ8KScratch n;
    void *q = nullptr, *d = nullptr, *b = nullptr;
    if (wd_malloc(&q, static_cast<size_t>(cols)) != WD_OK || wd_malloc(&d, sizeof(float) * (cols / 256)) != WD_OK ||
        wd_malloc(&b, sizeof(int16_t) * (cols / 16)) != WD_OK) {
        wd_free(q), wd_free(d), wd_free(b);
        throw std::runtime_error(std::string("Q8_K head scratch allocation failed: ") + wd_last_error());
    }
    n.cols = cols, n.quants = static_cast<int8_t *>(q), n.scales = static_cast<float *>(d), n.sums = static_cast<int16_t *>(b);
    s = n;  // the previous buffers stay allocated: a launch in flight may still read them
}
// src/lowbit.cuh:2712-2716
inline bool lowbit_q6_k_head_q8_k_eligible(const LowBitMatrix &w) {
    return w.type == GgmlType::Q6_K && w.rows > 0 && w.cols > 0 && w.cols % 256 == 0;
}
// The output head from the caller's F32 activation: Q8_K quantisation, then the Q6_K x Q8_K GEMV into F32 logits.
// src/lowbit.cuh:2724-2744
inline void launch_q6_k_head_gemv_q8_k_from_f32(const LowBitMatrix &w, const float *activation, float *out, Stream stream, int threads = 256) {
    if (!lowbit_q6_k_head_q8_k_eligible(w)) throw std::runtime_error("Q6_K x Q8_K output head path is not available for this matrix");
    if (threads < 32 || threads % 32 != 0) throw std::runtime_error("Q6_K x Q8_K GEMV threads must be a multiple of 32");
    lowbit_head_q8_k_reserve(w.cols);
    LowBitHeadQ8KScratch &s = lowbit_head_q8_k_scratch();
    launch_q8_k_quantize_f32(activation, w.cols, s.quants, s.scales, s.sums, stream, threads);
    launch_q6_k_gemv_q8_k_f32(w, s.quants, s.scales, s.sums, out, stream, threads);
}

// src/lowbit.cuh:1787-1810
inline void launch_iq4_nl_gemv_q8_0_f32(const LowBitMatrix &w, const int8_t *act, const half_bits *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    if (w.type != GgmlType::IQ4_NL || w.rows <= 0 || w.cols <= 0 || w.cols % 64 != 0) throw std::runtime_error("IQ4_NL x Q8_0 GEMV geometry mismatch");
    check(wd_gemv_q8_0_f32(WD_TYPE_IQ4_NL, w.data, w.rows, w.cols, act, act_scales, out, nullptr, stream), "IQ4_NL GEMV failed");
}
// src/qwen38_hc.cuh:1020-1049
inline void q38_hc_launch_exact_q8_0_gemv_f32(const uint8_t *weight, const int8_t *act, const half_bits *act_scales, float *out, int rows, int cols, Stream stream) {
    check(wd_gemv_q8_0_f32(WD_TYPE_Q8_0, weight, rows, cols, act, act_scales, out, nullptr, stream), "Q8_0 GEMV failed");
}
// The same for a list of projections of one row length in one launch (no counterpart in the reference, which launches
// q38_hc_launch_exact_q8_0_gemv_f32 once per projection; the results are the same bits as those calls).
inline void q38_hc_launch_exact_q8_0_gemv_batch_f32(const wd_gemv_item *items, int n_items, int cols, Stream stream) {
    check(wd_gemv_q8_0_batch_f32(WD_TYPE_Q8_0, items, n_items, cols, stream), "batched Q8_0 GEMV failed");
}
// src/warodecode.cu:1746-1768 (raw Q4_0 blocks; no planar prepack)
inline void launch_q4_float(const LowBitMatrix &w, const int8_t *act, const half_bits *act_scales, float *out, Stream stream) {
    if (w.type != GgmlType::Q4_0 || w.cols % 32 != 0) throw std::runtime_error("Q4_0 x Q8_0 GEMV geometry mismatch");
    check(wd_gemv_q8_0_f32(WD_TYPE_Q4_0, w.data, w.rows, w.cols, act, act_scales, out, nullptr, stream), "Q4_0 GEMV failed");
}

// Grouped launchers over a DEVICE table of expert pointers; false = nothing launched
// (src/lowbit.cuh:2352-2418, :2427-2460).
inline bool launch_iq3_s_gemv_q8_k_experts_f32(const uint8_t *const *w_experts, int experts, int rows, int cols, const int8_t *act, const float *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    return wd_gemv_q8_k_experts_f32(WD_TYPE_IQ3_S, w_experts, experts, rows, cols, act, act_scales, out, nullptr, stream) == WD_OK;
}
inline bool launch_iq2_s_gemv_q8_k_experts_f32(const uint8_t *const *w_experts, int experts, int rows, int cols, const int8_t *act, const float *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    return wd_gemv_q8_k_experts_f32(WD_TYPE_IQ2_S, w_experts, experts, rows, cols, act, act_scales, out, nullptr, stream) == WD_OK;
}
inline bool launch_iq4_nl_gemv_q8_0_experts_f32(const uint8_t *const *w_experts, int experts, int rows, int cols, const int8_t *act, const half_bits *act_scales, float *out, Stream stream, int /*threads*/ = 256) {
    return wd_gemv_q8_0_experts_f32(WD_TYPE_IQ4_NL, w_experts, experts, rows, cols, act, act_scales, out, nullptr, stream) == WD_OK;
}
inline bool launch_q8_0_gemv_q8_0_experts_f32(const uint8_t *const *w_experts, int experts, int rows, int cols, const int8_t *act, const half_bits *act_scales, float *out, Stream stream) {
    return wd_gemv_q8_0_experts_f32(WD_TYPE_Q8_0, w_experts, experts, rows, cols, act, act_scales, out, nullptr, stream) == WD_OK;
}

// src/qwen38_moe.cuh:2425-2436
inline void q38_moe_add_shared_f32(float *routed_in_out, const float *shared, const float *gate, int n, Stream stream) {
    check(wd_add_shared_f32(routed_in_out, shared, gate, n, stream), "shared expert add failed");
}

// ---- layer -------------------------------------------------------------------------------------------

namespace detail {
inline void fill_routed(wd_moe_layer &L, int layer, const GpuMatrix &router, const TensorInfo &gate, const TensorInfo &up, const TensorInfo &down,
                        const GpuExpertCache &cache, const Qwen38MoeScratch &scratch, float expert_scale) {
    if (!matrix_has_f32_weights(router)) throw std::runtime_error("MoE router must be an F32 matrix");
    const ExpertHostSlice g = expert_slice(gate, 0), u = expert_slice(up, 0), d = expert_slice(down, 0);
    if (g.cols != router.cols || u.cols != g.cols || u.rows != g.rows || d.cols != g.rows || d.rows != g.cols)
        throw std::runtime_error("MoE expert tensor geometry mismatch");
    std::memset(&L, 0, sizeof(L));
    L.hidden = g.cols, L.expert_ffn = g.rows, L.n_experts = router.rows, L.top_k = scratch.k();
    L.expert_scale = expert_scale;
    L.gate_type = static_cast<int>(g.type), L.up_type = static_cast<int>(u.type), L.down_type = static_cast<int>(d.type);
    L.router = router.dense_f32.data;
    L.slot_of_expert = cache.slot_table(layer);
    L.slot_pool = cache.pool();
    L.slot_bytes = cache.slot_bytes(), L.slot_gate_bytes = cache.gate_bytes(), L.slot_up_bytes = cache.up_bytes();
    if (!L.slot_of_expert) throw std::runtime_error("MoE layer is outside the expert cache's layer range");
}
// The layer pass for a layer whose experts are not all in the slot pool: dispatch A (router, selection, the shared
// expert's first half), the ids to the host, the cache acquires them, then the routed dispatches on that selection.
// The wait for the ids is also where a failure recorded by an earlier pass on this scratch surfaces.
inline void routed_through_host(const wd_moe_layer &L, int layer, const float *x, const TensorInfo &gate, const TensorInfo &up,
                                const TensorInfo &down, GpuExpertCache &cache, Qwen38MoeScratch &scratch, float *dst, bool run_a,
                                Stream stream, unsigned extra_flags = 0u) {
    {   // the reference's brackets of this stretch (src/qwen38_moe.cuh:2323-2380): selection, ids to the host, the wait
        Q38MoeKernelScope select_scope(kQ38MoeSiteRouter, stream);
        if (run_a) check(wd_moe_layer_f32(&L, x, dst, scratch.handle(), WD_MOE_ONLY_A, stream), "MoE router failed");
        {
            Q38MoeKernelScope d2h_scope(kQ38MoeSiteRouterD2h, stream);
            check(wd_memcpy_d2h(scratch.h_ids(), scratch.d_ids(), sizeof(int) * L.top_k, stream), "routed ids copy failed");
            scratch.queue_status_copy(stream);
        }
        Q38MoeKernelScope sync_scope(kQ38MoeSiteRouterSync, stream);
        check(wd_stream_sync(stream), "stream synchronisation failed");
    }
    scratch.throw_if_failed();
    cache.register_layer_experts(layer, gate, up, down);
    cache.acquire_ids(layer, scratch.h_ids(), L.top_k, stream);
    check(wd_moe_layer_f32(&L, x, dst, scratch.handle(), WD_MOE_PRESELECTED | WD_MOE_ONLY_B | WD_MOE_ONLY_C | extra_flags, stream), "MoE experts failed");
}
}  // namespace detail

// Routed experts of one layer: router -> top-k -> (host ids, cache acquire) -> grouped gate/up -> SwiGLU ->
// grouped down -> ordered weighted sum into scratch.d_accum() and `out`.
// src/qwen38_moe.cuh:3650-3779.  When every expert of the layer is already resident the host never
// waits: the selection stays on the device and the kernels index the slot table themselves.
inline void run_qwen38_routed_moe_separate_f32_x(int layer, const float *x, const GpuMatrix &router, const TensorInfo &gate_exps,
                                                 const TensorInfo &up_exps, const TensorInfo &down_exps, GpuExpertCache &cache,
                                                 Qwen38MoeScratch &scratch, float *out, float expert_scale, Stream stream,
                                                 bool preselected = false, bool keep_expert_outputs = false) {
    wd_moe_layer L;
    detail::fill_routed(L, layer, router, gate_exps, up_exps, down_exps, cache, scratch, expert_scale);
    float *dst = out ? out : scratch.moe_out_f32();
    const unsigned keep = keep_expert_outputs ? WD_MOE_KEEP_EXPERT_OUT : 0u;  // scratch.rx_batch_down(): [k][hidden]
    Q38MoeKernelScope routed_scope(kQ38MoeSiteRoutedTotal, stream);  // (the library's own brackets of this site nest inside)
    if (cache.layer_resident(layer)) {
        check(wd_moe_layer_f32(&L, x, dst, scratch.handle(), (preselected ? WD_MOE_PRESELECTED : 0u) | keep, stream), "MoE layer failed");
        return;
    }
    detail::routed_through_host(L, layer, x, gate_exps, up_exps, down_exps, cache, scratch, dst, !preselected, stream, keep);
}

// The same with the gate and up projections stored as one tensor of 2 * ffn rows per expert
// (run_qwen38_routed_moe_fused, src/qwen38_moe.cuh:3522-3647).
inline void run_qwen38_routed_moe_fused_f32_x(int layer, const float *x, const GpuMatrix &router, const TensorInfo &gate_up_exps,
                                              const TensorInfo &down_exps, GpuExpertCache &cache, Qwen38MoeScratch &scratch, float *out,
                                              float expert_scale, Stream stream, bool preselected = false, bool keep_expert_outputs = false) {
    if (gate_up_exps.dims.size() != 3 || gate_up_exps.dims[1] % 2 != 0) throw std::runtime_error("fused gate_up tensor must be 3D with an even row count: " + gate_up_exps.name);
    TensorInfo half = gate_up_exps;   // geometry of one projection; the data pointer is only used for registration
    half.dims[1] = gate_up_exps.dims[1] / 2;
    cache.register_layer_fused(layer, gate_up_exps, down_exps);
    // the slot pool holds gate | up | down per expert, so from here on the separate runner applies unchanged
    // (its own registration call is a no-op for a layer that is registered already)
    half.dims[2] = gate_up_exps.dims[2];
    TensorInfo g = half, u = half;
    g.data = gate_up_exps.data, u.data = gate_up_exps.data;
    // expert_slice() checks contiguity against byte_size(): give it tensors of the half geometry
    run_qwen38_routed_moe_separate_f32_x(layer, x, router, g, u, down_exps, cache, scratch, out, expert_scale, stream, preselected,
                                         keep_expert_outputs);
}

// The reference's runners by element type (src/qwen38_moe.cuh:3521-3534, :3650-3668): XT the type of the layer's input
// (half bits or float), OutT that of the routed output, CaptureSelectedOutput the k selected experts' down outputs as half
// into selected_output_trace [k][hidden].  Half input is widened once (every half is a float, so the result is that of the
// float runner on the widened input - the reference's own statement, :3607-3610); half output is the F32 routed sum
// rounded once, as the reference's F32-mid lifetime rounds it (q38_finish_moe, :2401-2453).
namespace detail {
template <typename XT>
inline const float *widened_input(const XT *x, Qwen38MoeScratch &scratch, Stream stream) {
    if constexpr (std::is_same<XT, float>::value) {
        return x;
    } else {
        static_assert(std::is_same<XT, half_bits>::value, "MoE input is float or half bits");
        check(wd_convert_f16_to_f32(x, scratch.x_f32(), static_cast<size_t>(scratch.hidden()), stream), "widening the MoE input failed");
        return scratch.x_f32();
    }
}
template <bool Capture, typename OutT>
inline void narrowed_output(Qwen38MoeScratch &scratch, const float *routed, OutT *out, half_bits *trace, Stream stream) {
    if constexpr (!std::is_same<OutT, float>::value) {
        static_assert(std::is_same<OutT, half_bits>::value, "MoE output is float or half bits");
        check(wd_convert_f32_to_f16(routed, out, static_cast<size_t>(scratch.hidden()), stream), "rounding the MoE output failed");
    }
    if constexpr (Capture)
        check(wd_convert_f32_to_f16(scratch.rx_batch_down(), trace, static_cast<size_t>(scratch.k()) * scratch.hidden(), stream),
              "selected expert trace failed");
}
}  // namespace detail

template <bool CaptureSelectedOutput = false, typename OutT = half_bits, typename XT = half_bits>
inline void run_qwen38_routed_moe_separate(int layer, const XT *x, const GpuMatrix &router, const TensorInfo &gate_exps,
                                           const TensorInfo &up_exps, const TensorInfo &down_exps, GpuExpertCache &cache,
                                           Qwen38MoeScratch &scratch, OutT *out, float expert_scale, Stream stream,
                                           bool preselected = false, half_bits *selected_output_trace = nullptr) {
    if (CaptureSelectedOutput && !selected_output_trace) throw std::runtime_error("selected expert trace buffer is null");
    if (!out) throw std::runtime_error("MoE output buffer is null");
    const float *xf = detail::widened_input<XT>(x, scratch, stream);
    float *routed = std::is_same<OutT, float>::value ? reinterpret_cast<float *>(out) : scratch.moe_out_f32();
    run_qwen38_routed_moe_separate_f32_x(layer, xf, router, gate_exps, up_exps, down_exps, cache, scratch, routed, expert_scale, stream,
                                         preselected, CaptureSelectedOutput);
    detail::narrowed_output<CaptureSelectedOutput, OutT>(scratch, routed, out, selected_output_trace, stream);
}
template <bool CaptureSelectedOutput = false, typename OutT = half_bits, typename XT = half_bits>
inline void run_qwen38_routed_moe_fused(int layer, const XT *x, const GpuMatrix &router, const TensorInfo &gate_up_exps,
                                        const TensorInfo &down_exps, GpuExpertCache &cache, Qwen38MoeScratch &scratch, OutT *out,
                                        float expert_scale, Stream stream, bool preselected = false,
                                        half_bits *selected_output_trace = nullptr) {
    if (CaptureSelectedOutput && !selected_output_trace) throw std::runtime_error("selected expert trace buffer is null");
    if (!out) throw std::runtime_error("MoE output buffer is null");
    const float *xf = detail::widened_input<XT>(x, scratch, stream);
    float *routed = std::is_same<OutT, float>::value ? reinterpret_cast<float *>(out) : scratch.moe_out_f32();
    run_qwen38_routed_moe_fused_f32_x(layer, xf, router, gate_up_exps, down_exps, cache, scratch, routed, expert_scale, stream, preselected,
                                      CaptureSelectedOutput);
    detail::narrowed_output<CaptureSelectedOutput, OutT>(scratch, routed, out, selected_output_trace, stream);
}
// src/qwen38_moe.cuh:3588-3604: float output from half input
template <bool CaptureSelectedOutput = false>
inline void run_qwen38_routed_moe_fused_f32(int layer, const half_bits *x, const GpuMatrix &router, const TensorInfo &gate_up_exps,
                                            const TensorInfo &down_exps, GpuExpertCache &cache, Qwen38MoeScratch &scratch, float *out,
                                            float expert_scale, Stream stream, bool preselected = false,
                                            half_bits *selected_output_trace = nullptr) {
    run_qwen38_routed_moe_fused<CaptureSelectedOutput, float, half_bits>(layer, x, router, gate_up_exps, down_exps, cache, scratch, out,
                                                                         expert_scale, stream, preselected, selected_output_trace);
}

// src/qwen38_moe.cuh:3963-3969
inline void run_qwen38_shared_expert_f32_x(const float *x, const Qwen38SharedExpertWeights &shared, Qwen38MoeScratch &scratch, Stream stream) {
    if (shared.gate.type != GgmlType::Q8_0 || shared.up.type != GgmlType::Q8_0 || shared.down.type != GgmlType::Q8_0)
        throw std::runtime_error("shared expert weights must be Q8_0");
    if (shared.gate.cols != scratch.hidden() || shared.gate.rows != scratch.expert_ffn() || shared.down.rows != scratch.hidden() ||
        shared.down.cols != scratch.expert_ffn() || shared.gate_input_f32.count != static_cast<size_t>(scratch.hidden()))
        throw std::runtime_error("shared expert geometry mismatch");
    wd_moe_layer L;
    std::memset(&L, 0, sizeof(L));
    L.hidden = scratch.hidden(), L.expert_ffn = scratch.expert_ffn();
    L.shared_gate_inp = shared.gate_input_f32.data;
    L.shared_gate = shared.gate.data, L.shared_up = shared.up.data, L.shared_down = shared.down.data;
    check(wd_shared_expert_f32(&L, x, scratch.handle(), stream), "shared expert failed");
}

// out = routed weighted sum + shared expert * gate (src/qwen38_moe.cuh:2442-2453)
inline void q38_finish_moe_f32(Qwen38MoeScratch &scratch, float *out, Stream stream) {
    if (out == scratch.d_accum()) throw std::runtime_error("F32 MoE output must not alias the routed accumulation buffer");
    Q38MoeKernelScope finish_scope(kQ38MoeSiteFinish, stream);
    check(wd_memcpy_d2d(out, scratch.d_accum(), sizeof(float) * scratch.hidden(), stream), "routed sum copy failed");
    q38_moe_add_shared_f32(out, scratch.down_f32(), scratch.d_shared_gate(), scratch.hidden(), stream);
}

// The three calls above in the fused dispatches (router and shared expert overlap, the selection never
// leaves the device): the fast path when the layer's experts are resident in `cache` or in plain device
// tensors.  No single counterpart in the reference (its caller issues the three calls,
// src/qwen38_forward.cuh:3330-3371).
inline void run_qwen38_moe_layer_f32_x(int layer, const float *x, const GpuMatrix &router, const TensorInfo &gate_exps, const TensorInfo &up_exps,
                                       const TensorInfo &down_exps, GpuExpertCache &cache, const Qwen38SharedExpertWeights &shared,
                                       Qwen38MoeScratch &scratch, float *out, float expert_scale, Stream stream) {
    wd_moe_layer L;
    detail::fill_routed(L, layer, router, gate_exps, up_exps, down_exps, cache, scratch, expert_scale);
    L.shared_gate_inp = shared.gate_input_f32.data;
    L.shared_gate = shared.gate.data, L.shared_up = shared.up.data, L.shared_down = shared.down.data;
    if (!cache.layer_resident(layer)) {  // the device cannot resolve every selection by itself: the ids go through the host
        detail::routed_through_host(L, layer, x, gate_exps, up_exps, down_exps, cache, scratch, out, true, stream);
        return;
    }
    check(wd_moe_layer_f32(&L, x, out, scratch.handle(), 0u, stream), "MoE layer failed");
}

// M tokens through one layer, every selected expert read once for all the tokens that chose it (the MTP block's
// block_moe, src/qwen38_mtp.cuh:674-795, with Qwen38MoeTokenBatch, src/qwen38_moe.cuh:2743-3237: router and selection of
// every token, the union of their experts acquired from the cache, one batch pass, then the shared expert and the
// combine per token).  x and out are [tokens][hidden]; every token has a scratch of its own, which afterwards holds that
// token's ids, weights, routed sum and shared-expert output exactly as after a one-token call.  When the layer's experts
// are all resident nothing leaves the device; otherwise the ids of all tokens go to the host once, the union is acquired
// (the cache must have room for it) and the pass runs on the given selection.
inline void run_qwen38_moe_tokens_f32_x(int layer, const float *x, int tokens, const GpuMatrix &router, const TensorInfo &gate_exps,
                                        const TensorInfo &up_exps, const TensorInfo &down_exps, GpuExpertCache &cache,
                                        const Qwen38SharedExpertWeights &shared, const std::vector<Qwen38MoeScratch *> &scratch, float *out,
                                        float expert_scale, Stream stream) {
    if (tokens <= 0 || static_cast<size_t>(tokens) != scratch.size()) throw std::runtime_error("token batch: one scratch per token is required");
    wd_moe_layer L;
    detail::fill_routed(L, layer, router, gate_exps, up_exps, down_exps, cache, *scratch[0], expert_scale);
    L.shared_gate_inp = shared.gate_input_f32.data;
    L.shared_gate = shared.gate.data, L.shared_up = shared.up.data, L.shared_down = shared.down.data;
    std::vector<wd_moe_scratch *> handles;
    for (const Qwen38MoeScratch *s : scratch) handles.push_back(s->handle());
    if (cache.layer_resident(layer)) {
        check(wd_moe_layer_tokens_f32(&L, x, out, tokens, handles.data(), 0u, stream), "MoE token batch failed");
        return;
    }
    const int k = L.top_k, H = L.hidden;
    for (int t = 0; t < tokens; ++t) {
        check(wd_moe_layer_f32(&L, x + static_cast<size_t>(t) * H, out + static_cast<size_t>(t) * H, handles[t], WD_MOE_ONLY_A, stream),
              "MoE router failed");
        check(wd_memcpy_d2h(scratch[t]->h_ids(), scratch[t]->d_ids(), sizeof(int) * k, stream), "routed ids copy failed");
        scratch[t]->queue_status_copy(stream);
    }
    check(wd_stream_sync(stream), "stream synchronisation failed");
    for (const Qwen38MoeScratch *s : scratch) s->throw_if_failed();
    std::vector<int> unique;
    for (int t = 0; t < tokens; ++t)
        for (int j = 0; j < k; ++j) {
            const int e = scratch[t]->h_ids()[j];
            if (std::find(unique.begin(), unique.end(), e) == unique.end()) unique.push_back(e);
        }
    cache.register_layer_experts(layer, gate_exps, up_exps, down_exps);
    for (size_t at = 0; at < unique.size(); at += 16)  // most recently acquired experts are the last to be recycled
        cache.acquire_ids(layer, unique.data() + at, static_cast<int>(std::min<size_t>(16, unique.size() - at)), stream);
    for (int e : unique)
        if (wd_expert_cache_slot_of(cache.handle(), layer, e) < 0) throw std::runtime_error("token batch: the expert cache is too small for the union of the tokens' experts");
    check(wd_moe_layer_tokens_f32(&L, x, out, tokens, handles.data(), WD_MOE_PRESELECTED, stream), "MoE token batch failed");
}

// The MTP block's token batch with the reference's interface (Qwen38MoeTokenBatch, src/qwen38_moe.cuh:2743-3237; its
// caller: src/qwen38_mtp.cuh:674-795): open_all selects the experts of every token with one synchronisation, the caller
// acquires the union of the experts and names each pair's (token * k + rank) views with set_pair_weights, resolved()
// decides whether the pass may run, run() computes every token's routed sum with each distinct expert read once, and
// write_output() hands the sums on as float or half.  After open_all, scratch.h_ids() / h_weights() hold [tokens][k].
class Qwen38MoeTokenBatch {
public:
    Qwen38MoeTokenBatch() = default;
    Qwen38MoeTokenBatch(const Qwen38MoeTokenBatch &) = delete;
    Qwen38MoeTokenBatch &operator=(const Qwen38MoeTokenBatch &) = delete;

    int batch_k() const { return 16; }
    int tokens() const { return tokens_; }

    // src/qwen38_moe.cuh:2767-2791: the pass exists for IQ2_S / IQ3_S gate and up tensors; the down tensors this library
    // batches are Q8_0 rows of at most 16 blocks and aligned IQ4_NL / Q8_0 rows of 16 or 20 blocks.  The slot bound is the
    // reference's (8 slots per selection).
    bool compatible(const GpuExpertCache &cache, const Qwen38MoeScratch &scratch, const TensorInfo &gate_exps, const TensorInfo &up_exps,
                    const TensorInfo &down_exps, int tokens) const {
        if (tokens < 1 || tokens > kMoeBatchTokenMax) return false;
        if (scratch.k() < 1 || scratch.k() > batch_k() || tokens * scratch.k() > 128) return false;
        auto iq = [](GgmlType t) { return t == GgmlType::IQ2_S || t == GgmlType::IQ3_S; };
        if (!iq(gate_exps.type) || gate_exps.type != up_exps.type) return false;
        const int F = scratch.expert_ffn();
        if (!(down_exps.type == GgmlType::Q8_0 && F <= 512) && !((down_exps.type == GgmlType::IQ4_NL || down_exps.type == GgmlType::Q8_0) && (F == 512 || F == 640)))
            return false;
        if (gate_exps.dims.size() != 3 || up_exps.dims.size() != 3 || down_exps.dims.size() != 3) return false;
        if (static_cast<int>(gate_exps.dims[0]) != scratch.hidden() || static_cast<int>(gate_exps.dims[1]) != F ||
            static_cast<int>(up_exps.dims[0]) != scratch.hidden() || static_cast<int>(up_exps.dims[1]) != F ||
            static_cast<int>(down_exps.dims[0]) != F || static_cast<int>(down_exps.dims[1]) != scratch.hidden())
            return false;
        return cache.slot_count() >= 8u * static_cast<size_t>(scratch.k());
    }

    // src/qwen38_moe.cuh:2798-2888.  activations: one device pointer per token (float [hidden]).  preselected: the caller
    // has put ids and weights into scratch.h_ids() / h_weights() ([tokens][k]) itself (or will, with set_pair_experts).
    void open_all(Qwen38MoeScratch &scratch, const GpuMatrix &router, const std::vector<const float *> &activations, float expert_scale,
                  Stream stream, bool preselected) {
        tokens_ = static_cast<int>(activations.size());
        if (tokens_ < 1 || tokens_ > kMoeBatchTokenMax) throw std::runtime_error("MoE token batch holds one to the batch bound of tokens");
        if (!(expert_scale > 0.0f)) throw std::runtime_error("MoE token batch needs a positive expert scale");
        for (const float *x : activations)
            if (!x) throw std::runtime_error("MoE token batch got a null activation");
        k_ = scratch.k(), hidden_ = scratch.hidden();
        activations_ = activations;
        ids_ = scratch.h_ids(), weights_ = scratch.h_weights();
        while (tok_.size() < static_cast<size_t>(tokens_)) {
            tok_.emplace_back(new Qwen38MoeScratch);
            tok_.back()->initialize(scratch.n_experts(), scratch.k(), scratch.hidden(), scratch.expert_ffn());
        }
        for (int p = 0; p < kMoeBatchTokenMax * 16; ++p) pair_[p] = Pair();
        router_ = router.dense_f32.data;
        if (preselected) return;
        if (!matrix_has_f32_weights(router)) throw std::runtime_error("MoE router must be an F32 matrix");
        if (router.rows != scratch.n_experts() || router.cols != hidden_) throw std::runtime_error("Qwen3.8 router matrix geometry mismatch");
        for (int t = 0; t < tokens_; ++t) {
            Qwen38MoeScratch &q = *tok_[static_cast<size_t>(t)];
            check(wd_router_gemv_f32(router.dense_f32.data, activations[static_cast<size_t>(t)], q.d_logits(), router.rows, router.cols, stream),
                  "MoE token batch router failed");
            check(wd_topk_softmax(q.d_logits(), router.rows, k_, expert_scale, q.d_ids(), q.d_weights(), stream), "MoE token batch selection failed");
            check(wd_memcpy_d2h(ids_ + t * k_, q.d_ids(), sizeof(int) * k_, stream), "MoE token batch ids copy failed");
            check(wd_memcpy_d2h(weights_ + t * k_, q.d_weights(), sizeof(float) * k_, stream), "MoE token batch weights copy failed");
        }
        check(wd_stream_sync(stream), "MoE token batch selection failed");
        queued_ = false;
    }

    // src/qwen38_moe.cuh:2897-2904
    void set_pair_experts(int pair, int expert, const std::vector<float> &weights_by_pair) {
        if (pair < 0 || pair >= kMoeBatchTokenMax * 16) throw std::runtime_error("MoE token batch pair index out of range");
        if (ids_) ids_[pair] = expert;
        if (weights_) weights_[pair] = weights_by_pair[static_cast<size_t>(pair)];
    }
    // src/qwen38_moe.cuh:2907-2922
    void set_pair_weights(int pair, const LowBitMatrix &gate, const LowBitMatrix &up, const LowBitMatrix &down) {
        if (pair < 0 || pair >= kMoeBatchTokenMax * 16) throw std::runtime_error("MoE token batch pair index out of range");
        pair_[pair].gate = gate.data, pair_[pair].up = up.data, pair_[pair].down = down.data;
        if (pair == 0) gate_type_ = gate.type, down_type_ = down.type, ffn_ = gate.rows;
    }
    // src/qwen38_moe.cuh:2933-2951: every pair has its three views, 2-byte aligned, of the types the pass takes; with
    // check_slots, two pairs that share a slot must name the same expert (otherwise a later acquire recycled the slot
    // under an earlier pair and the batch must give way to the serial loop).
    bool resolved(bool check_slots = false) {
        if (gate_type_ != GgmlType::IQ2_S && gate_type_ != GgmlType::IQ3_S) return false;
        const int pairs = tokens_ * k_;
        for (int p = 0; p < pairs; ++p) {
            const Pair &e = pair_[p];
            if (!e.gate || !e.up || !e.down) return false;
            if ((reinterpret_cast<uintptr_t>(e.gate) | reinterpret_cast<uintptr_t>(e.up) | reinterpret_cast<uintptr_t>(e.down)) & 1u) return false;
        }
        if (!check_slots || !ids_) return true;
        for (int a = 0; a < pairs; ++a)
            for (int b = a + 1; b < pairs; ++b)
                if (pair_[b].gate == pair_[a].gate && pair_[b].down == pair_[a].down && ids_[a] != ids_[b]) return false;
        return true;
    }

    // src/qwen38_moe.cuh:2955-3109: the routed experts of every token in one pass.  The tensors are named for the
    // interface's sake; the pass works on the views given pair by pair.
    void run(Qwen38MoeScratch &scratch, const TensorInfo &, const TensorInfo &, const TensorInfo &, Stream stream) {
        const int pairs = tokens_ * k_;
        if (tokens_ < 1 || k_ < 1 || pairs <= 0 || pairs > 128) throw std::runtime_error("MoE token batch pass is not staged");
        if (!resolved(false)) throw std::runtime_error("MoE token batch pass has unresolved pairs");
        if (queued_) check(wd_stream_sync(stream), "MoE token batch: waiting for the previous pass failed");  // its copies read the staging below
        // distinct experts in order of first appearance; a pair's id is the number of its expert's entry
        std::vector<const uint8_t *> g, u, d;
        if (!stage_) {
            void *p = nullptr;
            check(wd_malloc_host(&p, sizeof(int) * kMoeBatchTokenMax * 16), "pinned allocation failed");
            stage_ = static_cast<int *>(p);
        }
        for (int p = 0; p < pairs; ++p) {
            int entry = -1;
            for (size_t q = 0; q < g.size(); ++q)
                if (g[q] == pair_[p].gate && d[q] == pair_[p].down) entry = static_cast<int>(q);
            if (entry < 0) {
                entry = static_cast<int>(g.size());
                g.push_back(pair_[p].gate), u.push_back(pair_[p].up), d.push_back(pair_[p].down);
            }
            stage_[p] = entry;
        }
        if (static_cast<int>(g.size()) > scratch.n_experts()) throw std::runtime_error("MoE token batch: more distinct experts than the scratch was made for");
        std::vector<wd_moe_scratch *> handles;
        for (int t = 0; t < tokens_; ++t) {
            Qwen38MoeScratch &q = *tok_[static_cast<size_t>(t)];
            check(wd_memcpy_h2d(q.d_ids(), stage_ + t * k_, sizeof(int) * k_, stream), "MoE token batch ids upload failed");
            check(wd_memcpy_h2d(q.d_weights(), weights_ + t * k_, sizeof(float) * k_, stream), "MoE token batch weights upload failed");
            handles.push_back(q.handle());
        }
        if (x_.count < static_cast<size_t>(tokens_) * hidden_) x_.reset(), x_.allocate(static_cast<size_t>(kMoeBatchTokenMax) * hidden_);
        if (out_.count < static_cast<size_t>(tokens_) * hidden_) out_.reset(), out_.allocate(static_cast<size_t>(kMoeBatchTokenMax) * hidden_);
        for (int t = 0; t < tokens_; ++t)
            check(wd_memcpy_d2d(x_.data + static_cast<size_t>(t) * hidden_, activations_[static_cast<size_t>(t)], sizeof(float) * hidden_, stream),
                  "MoE token batch activation copy failed");
        wd_moe_layer L;
        std::memset(&L, 0, sizeof(L));
        L.hidden = hidden_, L.expert_ffn = ffn_, L.n_experts = scratch.n_experts(), L.top_k = k_, L.expert_scale = 1.0f;
        L.gate_type = L.up_type = static_cast<int>(gate_type_), L.down_type = static_cast<int>(down_type_);
        L.router = router_ ? router_ : reinterpret_cast<const float *>(g[0]);  // (not read: the selection is given)
        check(wd_moe_layer_tokens_pairs_f32(&L, g.data(), u.data(), d.data(), static_cast<int>(g.size()), x_.data, out_.data, tokens_, handles.data(),
                                            WD_MOE_PRESELECTED, stream),
              "MoE token batch pass failed");
        queued_ = true;
    }

    // src/qwen38_moe.cuh:3111-3113: float [tokens][hidden], every token's routed weighted sum
    float *accumulated(Qwen38MoeScratch &) { return out_.data; }

    // src/qwen38_moe.cuh:3119-3147: the sums as they are, or rounded to half once
    void write_output(Qwen38MoeScratch &scratch, float *out_f32_or_null, half_bits *out_half_or_null, Stream stream) {
        const size_t n = static_cast<size_t>(tokens_) * scratch.hidden();
        if (out_half_or_null)
            check(wd_convert_f32_to_f16(out_.data, out_half_or_null, n, stream), "MoE token batch output failed");
        else if (out_f32_or_null)
            check(wd_memcpy_d2d(out_f32_or_null, out_.data, sizeof(float) * n, stream), "MoE token batch output failed");
        else
            throw std::runtime_error("MoE token batch output failed: no output buffer");
    }

    ~Qwen38MoeTokenBatch() {
        if (stage_) wd_free_host(stage_);
    }

private:
    struct Pair {
        const uint8_t *gate = nullptr, *up = nullptr, *down = nullptr;
    };
    int tokens_ = 0, k_ = 0, hidden_ = 0, ffn_ = 0;
    int *ids_ = nullptr, *stage_ = nullptr;
    float *weights_ = nullptr;
    const float *router_ = nullptr;
    bool queued_ = false;
    GgmlType gate_type_ = GgmlType::F32, down_type_ = GgmlType::F32;
    std::vector<const float *> activations_;
    std::vector<std::unique_ptr<Qwen38MoeScratch>> tok_;
    Pair pair_[kMoeBatchTokenMax * 16];
    DeviceFloatArray x_, out_;
};

// The F32 inject projections of the hyper-connection combine (the part of the reference's Qwen38HcF32DebugScratch that
// the combine reads: hidden(), hc(), inject(); src/qwen38_hc.cuh:2263-2330).
class Qwen38HcF32DebugScratch {
public:
    void initialize(int hidden, int hc) {
        if (hidden <= 0 || hc <= 0) throw std::runtime_error("invalid hyper-connection scratch geometry");
        hidden_ = hidden, hc_ = hc;
        inject_.reset();
        inject_.allocate(static_cast<size_t>(hc));
    }
    int hidden() const { return hidden_; }
    int hc() const { return hc_; }
    float *inject() const { return inject_.data; }

private:
    int hidden_ = 0, hc_ = 0;
    DeviceFloatArray inject_;
};

// src/qwen38_hc.cuh:2561-2570
inline void run_qwen38_hc_combine_f32_block_f32_inject(float *residual, const float *block_out, const Qwen38HcF32DebugScratch &scratch,
                                                       Stream stream, bool round_half = false) {
    check(wd_hc_combine_f32(residual, block_out, scratch.inject(), scratch.hidden(), scratch.hc(), round_half ? 1 : 0, stream),
          "hyper-connection combine failed");
}
// src/qwen38_hc.cuh:2587-2600 (shared: the shared expert's output as half bits)
inline void run_qwen38_hc_combine_moe_f32_inject(float *residual, const float *routed, const half_bits *shared, const float *shared_gate,
                                                 const Qwen38HcF32DebugScratch &scratch, Stream stream, bool round_half = false) {
    check(wd_hc_combine_moe_f32(residual, routed, shared, 1, shared_gate, scratch.inject(), scratch.hidden(), scratch.hc(),
                                round_half ? 1 : 0, stream),
          "hyper-connection combine failed");
}
// The same with the shared expert's output in F32, as run_qwen38_shared_expert_f32_x leaves it in the scratch.
inline void run_qwen38_hc_combine_moe_f32_inject(float *residual, const float *routed, const float *shared, const float *shared_gate,
                                                 const Qwen38HcF32DebugScratch &scratch, Stream stream, bool round_half = false) {
    check(wd_hc_combine_moe_f32(residual, routed, shared, 0, shared_gate, scratch.inject(), scratch.hidden(), scratch.hc(),
                                round_half ? 1 : 0, stream),
          "hyper-connection combine failed");
}

// run_qwen38_moe_layer_f32_x followed by run_qwen38_hc_combine_f32_block_f32_inject on its output, the combine folded into
// the layer's last dispatch (src/qwen38_forward.cuh:3330-3371 issues them one after the other).
inline void run_qwen38_moe_layer_hc_f32_x(int layer, const float *x, const GpuMatrix &router, const TensorInfo &gate_exps,
                                          const TensorInfo &up_exps, const TensorInfo &down_exps, GpuExpertCache &cache,
                                          const Qwen38SharedExpertWeights &shared, Qwen38MoeScratch &scratch, float *out, float *residual,
                                          const Qwen38HcF32DebugScratch &hc, float expert_scale, Stream stream, bool round_half = false) {
    if (hc.hidden() != static_cast<int>(gate_exps.dims[0])) throw std::runtime_error("hyper-connection scratch does not match the layer's hidden size");
    wd_moe_layer L;
    detail::fill_routed(L, layer, router, gate_exps, up_exps, down_exps, cache, scratch, expert_scale);
    L.shared_gate_inp = shared.gate_input_f32.data;
    L.shared_gate = shared.gate.data, L.shared_up = shared.up.data, L.shared_down = shared.down.data;
    if (!cache.layer_resident(layer)) {  // the ids go through the host, the combine runs as a call of its own
        detail::routed_through_host(L, layer, x, gate_exps, up_exps, down_exps, cache, scratch, out, true, stream);
        run_qwen38_hc_combine_f32_block_f32_inject(residual, out, hc, stream, round_half);
        return;
    }
    check(wd_moe_layer_hc_f32(&L, x, out, residual, hc.inject(), hc.hc(), round_half ? 1 : 0, scratch.handle(), 0u, stream),
          "MoE layer with combine failed");
}

}  // namespace wd
