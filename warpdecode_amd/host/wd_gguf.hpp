// GGUF model file with the reference's names, on top of the C ABI's reader (wd_gguf_* in warpdecode_amd.h).
//   GgufFile                     src/gguf.hpp:312-491   (tensor / optional_tensor / tensors / string_meta / number_meta)
//   Qwen38MoeLayerTensors        src/qwen38_moe.cuh:535-545
//   qwen38_moe_tensors           src/qwen38_moe.cuh:601-612
//   load_qwen38_shared_expert    src/qwen38_moe.cuh:564-599
// Tensor views point into the read-only mapping, which lives as long as the GgufFile.
#pragma once
#include "wd_ops.hpp"

#include <cstdint>
#include <cstring>
#include <unordered_map>

namespace wd {

class GgufFile {
public:
    explicit GgufFile(const std::string &path) {
        check(wd_gguf_open(&g_, path.c_str()), "wd_gguf_open");
        const long long n = wd_gguf_tensor_count(g_);
        tensors_.reserve(static_cast<size_t>(n));
        for (long long i = 0; i < n; ++i) {
            wd_gguf_tensor_info ti;
            check(wd_gguf_tensor(g_, i, &ti), "wd_gguf_tensor");
            TensorInfo t;
            t.name = ti.name;
            t.dims.assign(ti.dims, ti.dims + ti.n_dims);
            t.type = static_cast<GgmlType>(ti.type);
            t.relative_offset = ti.relative_offset;
            t.data = ti.data;
            index_.emplace(t.name, tensors_.size());
            tensors_.push_back(std::move(t));
        }
    }
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;
    ~GgufFile() { wd_gguf_close(g_); }

    uint32_t version() const { return wd_gguf_version(g_); }
    size_t data_offset() const { return wd_gguf_data_offset(g_); }
    const std::vector<TensorInfo> &tensors() const { return tensors_; }

    const TensorInfo *optional_tensor(const std::string &name) const {
        const auto it = index_.find(name);
        return it == index_.end() ? nullptr : &tensors_[it->second];
    }
    const TensorInfo &tensor(const std::string &name) const {
        const TensorInfo *t = optional_tensor(name);
        if (!t) throw std::runtime_error("GGUF tensor not found: " + name);
        return *t;
    }
    // Position of a tensor's bytes in the file, for readers that bypass the mapping.
    uint64_t tensor_file_offset(const TensorInfo &t) const { return data_offset() + t.relative_offset; }

    std::string string_meta(const std::string &key, const std::string &fallback = "") const {
        const char *s = wd_gguf_meta_string(g_, key.c_str());
        return s ? std::string(s) : fallback;
    }
    double number_meta(const std::string &key, double fallback = 0.0) const {
        double v = 0.0;
        return wd_gguf_meta_number(g_, key.c_str(), &v) == WD_OK ? v : fallback;
    }
    // src/gguf.hpp:334-339: an unsigned scalar (a signed one when it is not negative), an exception otherwise
    uint64_t uint_meta(const std::string &key) const {
        double v = 0.0;
        if (wd_gguf_meta_number(g_, key.c_str(), &v) != WD_OK || v < 0.0 || v != static_cast<double>(static_cast<uint64_t>(v)))
            throw std::runtime_error("GGUF metadata is not an unsigned integer: " + key);
        return static_cast<uint64_t>(v);
    }
    // src/gguf.hpp:358-402: integer arrays convert between signed and unsigned when every value fits, float arrays are
    // numbers only; a missing key or an array of another kind throws.
    std::vector<uint64_t> uint_array_meta(const std::string &key) const {
        std::vector<uint64_t> out;
        read_array(key, false, [&](int kind, uint64_t u, int64_t i, double) {
            if (kind == 1 && i < 0) throw std::runtime_error("GGUF metadata array holds a negative value: " + key);
            out.push_back(kind == 0 ? u : static_cast<uint64_t>(i));
        });
        return out;
    }
    std::vector<int64_t> int_array_meta(const std::string &key) const {
        std::vector<int64_t> out;
        read_array(key, false, [&](int kind, uint64_t u, int64_t i, double) {
            if (kind == 0 && u > static_cast<uint64_t>(INT64_MAX)) throw std::runtime_error("GGUF metadata array value does not fit int64: " + key);
            out.push_back(kind == 0 ? static_cast<int64_t>(u) : i);
        });
        return out;
    }
    std::vector<double> number_array_meta(const std::string &key) const {
        std::vector<double> out;
        read_array(key, true, [&](int kind, uint64_t u, int64_t i, double f) {
            out.push_back(kind == 0 ? static_cast<double>(u) : (kind == 1 ? static_cast<double>(i) : f));
        });
        return out;
    }
    bool has_meta(const std::string &key) const {
        double v;
        uint32_t et;
        const void *p;
        return wd_gguf_meta_number(g_, key.c_str(), &v) == WD_OK || wd_gguf_meta_string(g_, key.c_str()) != nullptr ||
               wd_gguf_meta_array(g_, key.c_str(), &et, &p) >= 0;
    }
    // The read-only mapping of the whole file and its descriptor, for readers that bypass the mapping.
    const uint8_t *map_base() const { return wd_gguf_map_base(g_); }
    size_t map_bytes() const { return wd_gguf_map_bytes(g_); }
    int fd() const { return wd_gguf_fd(g_); }
    bool has_number_meta(const std::string &key) const {
        double v;
        return wd_gguf_meta_number(g_, key.c_str(), &v) == WD_OK;
    }

private:
    // Walks an array of fixed-size elements: f(kind, u, i, d) with kind 0 unsigned (and bool), 1 signed, 2 float.
    template <typename F>
    void read_array(const std::string &key, bool floats_allowed, F &&f) const {
        uint32_t et = 0;
        const void *p = nullptr;
        const long long n = wd_gguf_meta_array(g_, key.c_str(), &et, &p);
        if (n < 0) throw std::runtime_error("GGUF metadata array not found: " + key);
        const uint8_t *b = static_cast<const uint8_t *>(p);
        auto get = [&](auto tag, long long at) {
            decltype(tag) v;
            std::memcpy(&v, b + static_cast<size_t>(at) * sizeof(v), sizeof(v));
            return v;
        };
        for (long long at = 0; at < n; ++at) {
            switch (et) {
                case 0: case 7: f(0, get(uint8_t{}, at), 0, 0.0); break;
                case 1: f(1, 0, get(int8_t{}, at), 0.0); break;
                case 2: f(0, get(uint16_t{}, at), 0, 0.0); break;
                case 3: f(1, 0, get(int16_t{}, at), 0.0); break;
                case 4: f(0, get(uint32_t{}, at), 0, 0.0); break;
                case 5: f(1, 0, get(int32_t{}, at), 0.0); break;
                case 10: f(0, get(uint64_t{}, at), 0, 0.0); break;
                case 11: f(1, 0, get(int64_t{}, at), 0.0); break;
                case 6: case 12:
                    if (!floats_allowed) throw std::runtime_error("GGUF metadata array is not an integer array: " + key);
                    f(2, 0, 0, et == 6 ? static_cast<double>(get(float{}, at)) : get(double{}, at));
                    break;
                default: throw std::runtime_error("GGUF metadata array of an unsupported element type: " + key);
            }
        }
    }

    wd_gguf *g_ = nullptr;
    std::vector<TensorInfo> tensors_;
    std::unordered_map<std::string, size_t> index_;
};

// Misses of experts that live in this file are read with pread() into the cache's pinned ring (`threads` readers per
// expert) instead of a pageable copy from the mapping; call it once, before or after the layers are registered.
// reference: ExpertFileMap / ExpertPreadPool, src/expert_cache.cuh:204-508.
inline void attach_expert_file(GpuExpertCache &cache, const GgufFile &g, int threads = 4) {
    check(wd_expert_cache_attach_file(cache.handle(), g.map_base(), g.map_bytes(), g.fd(), threads), "wd_expert_cache_attach_file");
}

// The same without naming the file: every registered host tensor is looked up in /proc/self/maps and the files found
// are attached (returns how many).  reference: ExpertFileMap::resolve, src/expert_cache.cuh:221-243.
inline int attach_mapped_expert_files(GpuExpertCache &cache, int threads = 4) {
    int n = 0;
    check(wd_expert_cache_attach_mappings(cache.handle(), threads, &n), "wd_expert_cache_attach_mappings");
    return n;
}

struct Qwen38MoeLayerTensors {
    const TensorInfo *router = nullptr;
    const TensorInfo *gate_up = nullptr;  // one tensor of 2*ffn rows per expert, when the file stores it so
    const TensorInfo *gate = nullptr;
    const TensorInfo *up = nullptr;
    const TensorInfo *down = nullptr;
    bool fused_gate_up() const { return gate_up != nullptr; }
};

inline Qwen38MoeLayerTensors qwen38_moe_tensors(const GgufFile &g, int il) {
    const std::string blk = "blk." + std::to_string(il) + ".";
    Qwen38MoeLayerTensors t;
    t.router = &g.tensor(blk + "ffn_gate_inp.weight");
    t.down = &g.tensor(blk + "ffn_down_exps.weight");
    t.gate_up = g.optional_tensor(blk + "ffn_gate_up_exps.weight");
    if (!t.gate_up) {
        t.gate = &g.tensor(blk + "ffn_gate_exps.weight");
        t.up = &g.tensor(blk + "ffn_up_exps.weight");
    }
    return t;
}

inline Qwen38SharedExpertWeights load_qwen38_shared_expert(const GgufFile &g, int il, int hidden, int shared_ffn) {
    const std::string blk = "blk." + std::to_string(il) + ".";
    const TensorInfo &gate_input = g.tensor(blk + "ffn_gate_inp_shexp.weight");
    if (gate_input.dims.size() != 1 || static_cast<int>(gate_input.dims[0]) != hidden)
        throw std::runtime_error("shared expert gate-input shape mismatch");
    if (gate_input.type != GgmlType::F32)
        throw std::runtime_error("shared expert gate-input must be F32: " + gate_input.name);
    auto matrix = [&](const char *leaf, int rows, int cols) -> const TensorInfo & {
        const TensorInfo &t = g.tensor(blk + leaf);
        if (t.dims.size() != 2 || static_cast<int>(t.dims[0]) != cols || static_cast<int>(t.dims[1]) != rows)
            throw std::runtime_error("shared expert shape mismatch: " + t.name);
        if (t.type != GgmlType::Q8_0) throw std::runtime_error("shared expert low-bit type unsupported: " + t.name);
        return t;
    };
    const TensorInfo &gate = matrix("ffn_gate_shexp.weight", shared_ffn, hidden);
    const TensorInfo &up = matrix("ffn_up_shexp.weight", shared_ffn, hidden);
    const TensorInfo &down = matrix("ffn_down_shexp.weight", hidden, shared_ffn);
    Qwen38SharedExpertWeights out;
    out.gate_input_f32.upload(reinterpret_cast<const float *>(gate_input.data), static_cast<size_t>(hidden));
    out.gate = upload_lowbit_matrix(gate);
    out.up = upload_lowbit_matrix(up);
    out.down = upload_lowbit_matrix(down);
    return out;
}

}  // namespace wd
