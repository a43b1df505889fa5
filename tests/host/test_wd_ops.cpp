// Host-side test of the C++ operator surface (warpdecode_amd/host/wd_ops.hpp): a caller written in the
// style of the reference's own layer driver (routed experts, shared expert, finish;
// src/qwen38_forward.cuh:3330-3371) runs against the library and every result is compared bit for
// bit with the CPU oracle.  `--host-only` runs the checks that need no GPU (geometry errors, sizes).
//
// Built by warpdecode_amd/build.py (build_host_test) with g++ against libwarpdecode_amd.so and the oracle.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <random>

#include <unistd.h>

#include "wd_gguf.hpp"
#include "wd_ops.hpp"
#include "wd_oracle.h"

using namespace wd;

static int g_checks = 0, g_fail = 0;
#define CHECK(cond, ...)                          \
    do {                                          \
        ++g_checks;                               \
        if (!(cond)) {                            \
            ++g_fail;                             \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);             \
            std::printf("\n");                    \
        }                                         \
    } while (0)

static bool throws(const std::function<void()> &f) {
    try {
        f();
    } catch (const std::runtime_error &) {
        return true;
    }
    return false;
}

static bool same_bits(const float *a, const float *b, size_t n) { return std::memcmp(a, b, n * sizeof(float)) == 0; }

struct Rng {
    std::mt19937_64 g;
    explicit Rng(uint64_t s) : g(s) {}
    uint32_t u32() { return static_cast<uint32_t>(g()); }
    float normal() {
        const double u1 = (static_cast<double>(g() >> 11) + 1.0) / 9007199254740993.0, u2 = static_cast<double>(g() >> 11) / 9007199254740992.0;
        return static_cast<float>(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
    }
};

// Random GGUF block bytes with a sane fp16 scale at the head of every block.
static std::vector<uint8_t> random_blocks(Rng &r, int type, size_t rows, int cols, float scale) {
    const size_t bb = wdo_block_bytes(type), nb = rows * (cols / wdo_block_elems(type));
    std::vector<uint8_t> w(nb * bb);
    for (auto &b : w) b = static_cast<uint8_t>(r.u32());
    for (size_t i = 0; i < nb; ++i) {
        const uint16_t d = wdo_f32_to_f16(std::fabs(r.normal()) * scale);
        std::memcpy(&w[i * bb], &d, 2);
        if (type == WDO_Q8_0)
            for (size_t j = 2; j < bb; ++j)
                if (w[i * bb + j] == 0x80) w[i * bb + j] = 0x81;  // int8 quants in [-127, 127]
    }
    return w;
}

struct HostLayer {
    int H, F, E, k;
    std::vector<float> router, gate_inp;
    std::vector<uint8_t> gate, up, down, sg, su, sd;
    TensorInfo t_router, t_gate, t_up, t_down;
    wdo_layer o{};
};

static HostLayer make_layer(uint64_t seed, int H, int F, int E, int k) {
    HostLayer L;
    L.H = H, L.F = F, L.E = E, L.k = k;
    Rng r(seed);
    L.router.resize(static_cast<size_t>(E) * H);
    for (auto &v : L.router) v = r.normal() / std::sqrt(static_cast<float>(H));
    L.gate_inp.resize(H);
    for (auto &v : L.gate_inp) v = r.normal() * 0.02f;
    L.gate = random_blocks(r, WDO_IQ3_S, static_cast<size_t>(E) * F, H, 0.01f);
    L.up = random_blocks(r, WDO_IQ3_S, static_cast<size_t>(E) * F, H, 0.01f);
    L.down = random_blocks(r, WDO_Q8_0, static_cast<size_t>(E) * H, F, 0.02f / 127.0f);
    L.sg = random_blocks(r, WDO_Q8_0, F, H, 0.02f / 127.0f);
    L.su = random_blocks(r, WDO_Q8_0, F, H, 0.02f / 127.0f);
    L.sd = random_blocks(r, WDO_Q8_0, H, F, 0.02f / 127.0f);
    L.t_router = {"ffn_gate_inp.weight", {static_cast<uint64_t>(H), static_cast<uint64_t>(E)}, GgmlType::F32, 0, reinterpret_cast<const uint8_t *>(L.router.data())};
    L.t_gate = {"ffn_gate_exps.weight", {static_cast<uint64_t>(H), static_cast<uint64_t>(F), static_cast<uint64_t>(E)}, GgmlType::IQ3_S, 0, L.gate.data()};
    L.t_up = {"ffn_up_exps.weight", {static_cast<uint64_t>(H), static_cast<uint64_t>(F), static_cast<uint64_t>(E)}, GgmlType::IQ3_S, 0, L.up.data()};
    L.t_down = {"ffn_down_exps.weight", {static_cast<uint64_t>(F), static_cast<uint64_t>(H), static_cast<uint64_t>(E)}, GgmlType::Q8_0, 0, L.down.data()};
    L.o.hidden = H, L.o.expert_ffn = F, L.o.n_experts = E, L.o.top_k = k, L.o.w_scale = 1.0f;
    L.o.router = L.router.data();
    L.o.gate_type = L.o.up_type = WDO_IQ3_S, L.o.down_type = WDO_Q8_0;
    L.o.gate = L.gate.data(), L.o.up = L.up.data(), L.o.down = L.down.data();
    L.o.shared_gate_inp = L.gate_inp.data(), L.o.shared_type = WDO_Q8_0;
    L.o.shared_gate = L.sg.data(), L.o.shared_up = L.su.data(), L.o.shared_down = L.sd.data();
    return L;
}

// Minimal GGUF v3 writer for the layers above (the names a model file uses for one MoE block).
struct GgufOut {
    std::vector<uint8_t> head, data;
    uint64_t n_tensors = 0, n_kv = 0;
    template <typename T>
    void put(T v) {
        const uint8_t *p = reinterpret_cast<const uint8_t *>(&v);
        head.insert(head.end(), p, p + sizeof(T));
    }
    void str(const std::string &s) {
        put<uint64_t>(s.size());
        head.insert(head.end(), s.begin(), s.end());
    }
    void kv_u32(const std::string &k, uint32_t v) { str(k), put<uint32_t>(4), put<uint32_t>(v), ++n_kv; }
    void kv_f32(const std::string &k, float v) { str(k), put<uint32_t>(6), put<float>(v), ++n_kv; }
    void kv_str(const std::string &k, const std::string &v) { str(k), put<uint32_t>(8), str(v), ++n_kv; }
    void tensor(const std::string &name, std::vector<uint64_t> dims, GgmlType type, const void *bytes, size_t n) {
        str(name), put<uint32_t>(static_cast<uint32_t>(dims.size()));
        for (uint64_t d : dims) put<uint64_t>(d);
        put<uint32_t>(static_cast<uint32_t>(type)), put<uint64_t>(data.size());
        const uint8_t *b = static_cast<const uint8_t *>(bytes);
        data.insert(data.end(), b, b + n);
        data.resize((data.size() + 31) & ~size_t(31));
        ++n_tensors;
    }
    std::string write() {
        char path[] = "/tmp/wd_gguf_test_XXXXXX";
        const int fd = mkstemp(path);
        if (fd < 0) throw std::runtime_error("mkstemp failed");
        FILE *f = fdopen(fd, "wb");
        const uint32_t magic = 0x46554747u, version = 3;
        fwrite(&magic, 4, 1, f), fwrite(&version, 4, 1, f), fwrite(&n_tensors, 8, 1, f), fwrite(&n_kv, 8, 1, f);
        fwrite(head.data(), 1, head.size(), f);
        const std::vector<uint8_t> pad((32 - (24 + head.size()) % 32) % 32, 0);
        fwrite(pad.data(), 1, pad.size(), f);
        fwrite(data.data(), 1, data.size(), f);
        fclose(f);
        return path;
    }
};

static std::string write_model_file(const std::vector<HostLayer> &L) {
    GgufOut o;  // every key/value goes in before the first tensor: the directory follows the metadata in the file
    o.kv_str("general.architecture", "qwen38");
    o.kv_u32("qwen38.block_count", static_cast<uint32_t>(L.size()));
    o.kv_u32("qwen38.expert_count", static_cast<uint32_t>(L[0].E));
    o.kv_u32("qwen38.expert_used_count", static_cast<uint32_t>(L[0].k));
    o.kv_f32("qwen38.expert_weights_scale", 1.0f);
    for (size_t l = 0; l < L.size(); ++l) {
        const HostLayer &h = L[l];
        const std::string blk = "blk." + std::to_string(l) + ".";
        const uint64_t H = h.H, F = h.F, E = h.E;
        o.tensor(blk + "ffn_gate_inp.weight", {H, E}, GgmlType::F32, h.router.data(), h.router.size() * 4);
        o.tensor(blk + "ffn_gate_exps.weight", {H, F, E}, GgmlType::IQ3_S, h.gate.data(), h.gate.size());
        o.tensor(blk + "ffn_up_exps.weight", {H, F, E}, GgmlType::IQ3_S, h.up.data(), h.up.size());
        o.tensor(blk + "ffn_down_exps.weight", {F, H, E}, GgmlType::Q8_0, h.down.data(), h.down.size());
        o.tensor(blk + "ffn_gate_inp_shexp.weight", {H}, GgmlType::F32, h.gate_inp.data(), h.gate_inp.size() * 4);
        o.tensor(blk + "ffn_gate_shexp.weight", {H, F}, GgmlType::Q8_0, h.sg.data(), h.sg.size());
        o.tensor(blk + "ffn_up_shexp.weight", {H, F}, GgmlType::Q8_0, h.su.data(), h.su.size());
        o.tensor(blk + "ffn_down_shexp.weight", {F, H}, GgmlType::Q8_0, h.sd.data(), h.sd.size());
    }
    return o.write();
}

static std::vector<float> rms_normed(Rng &r, int n) {
    std::vector<float> x(n);
    double ss = 0;
    for (auto &v : x) v = r.normal(), ss += static_cast<double>(v) * v;
    const float inv = static_cast<float>(1.0 / std::sqrt(ss / n));
    for (auto &v : x) v *= inv;
    return x;
}

static void host_only_checks() {
    TensorInfo t{"w", {256, 4}, GgmlType::IQ3_S, 0, nullptr};
    CHECK(t.byte_size() == 4 * 110, "IQ3_S [4][256] is %zu bytes", t.byte_size());
    t.type = GgmlType::Q8_0;
    CHECK(t.byte_size() == 4 * 8 * 34, "Q8_0 [4][256] is %zu bytes", t.byte_size());
    t.dims = {100, 4};
    CHECK(throws([&] { t.byte_size(); }), "a ragged block count must throw");
    TensorInfo one{"w", {256}, GgmlType::IQ3_S, 0, nullptr};
    CHECK(throws([&] { upload_lowbit_matrix(one); }), "1-D tensor must be refused");
    TensorInfo f32{"w", {256, 4}, GgmlType::F32, 0, nullptr};
    CHECK(throws([&] { upload_lowbit_matrix(f32); }), "F32 tensor is not a low-bit matrix");
    TensorInfo bad{"w", {288, 4}, GgmlType::IQ3_S, 0, nullptr};
    CHECK(throws([&] { upload_lowbit_matrix(bad); }), "IQ3_S needs columns in multiples of 256");
    TensorInfo two{"w", {256, 4}, GgmlType::IQ3_S, 0, nullptr};
    CHECK(throws([&] { expert_slice(two, 0); }), "expert tensors are 3-D");
    TensorInfo three{"w", {256, 4, 2}, GgmlType::IQ3_S, 0, nullptr};
    CHECK(throws([&] { expert_slice(three, 2); }), "expert index out of range");
    CHECK(expert_slice(three, 1).bytes == 440 && expert_slice(three, 1).data == static_cast<const uint8_t *>(nullptr) + 440, "slice offset");
    Qwen38MoeScratch s;
    CHECK(throws([&] { s.initialize(8, 17, 256, 32); }), "k > 16 must be refused");
    CHECK(throws([&] { s.initialize(8, 9, 256, 32); }), "k > n_experts must be refused");
    GpuExpertCache c;
    CHECK(throws([&] { c.initialize(0, three, three, three); }), "zero capacity must be refused");
    CHECK(throws([&] { c.acquire(0, 0, three, three, three, nullptr); }), "acquire before initialize must throw");
    LowBitMatrix b = borrow_lowbit_matrix(reinterpret_cast<uint8_t *>(0x1000), 4, 256, GgmlType::IQ3_S, 440);
    LowBitMatrix m = std::move(b);
    CHECK(m.data == reinterpret_cast<uint8_t *>(0x1000) && !m.owns && b.data == nullptr, "move keeps the borrowed view");
    GpuMatrix g;
    CHECK(throws([&] { launch_q38_router_gemv_f32(g, nullptr, nullptr, nullptr); }), "router without F32 weights must throw");
    LowBitMatrix q = borrow_lowbit_matrix(reinterpret_cast<uint8_t *>(0x1000), 4, 256, GgmlType::Q8_0, 4 * 8 * 34);
    CHECK(throws([&] { launch_iq3_s_gemv_q8_k_f32(q, nullptr, nullptr, nullptr, nullptr); }), "type mismatch must throw");
    CHECK(throws([&] { launch_q8_k_quantize_f32(nullptr, 100, nullptr, nullptr, nullptr, nullptr); }), "Q8_K needs multiples of 256");

    // model file: directory, metadata and tensor bytes through GgufFile
    std::vector<HostLayer> L;
    for (int l = 0; l < 2; ++l) L.push_back(make_layer(500 + l, 256, 32, 8, 2));
    const std::string path = write_model_file(L);
    {
        GgufFile g(path);
        CHECK(g.version() == 3 && g.tensors().size() == 16 && g.data_offset() % 32 == 0, "header: version %u, %zu tensors", g.version(), g.tensors().size());
        CHECK(g.string_meta("general.architecture") == "qwen38" && g.string_meta("absent", "dflt") == "dflt", "string metadata");
        CHECK(g.number_meta("qwen38.expert_count") == 8.0 && g.number_meta("absent", -1.0) == -1.0 && g.has_number_meta("qwen38.expert_weights_scale"), "number metadata");
        CHECK(throws([&] { g.tensor("blk.9.ffn_gate_inp.weight"); }) && g.optional_tensor("blk.0.ffn_gate_up_exps.weight") == nullptr, "absent tensors");
        const Qwen38MoeLayerTensors t = qwen38_moe_tensors(g, 1);
        CHECK(!t.fused_gate_up() && t.gate->dims == std::vector<uint64_t>({256, 32, 8}) && t.gate->type == GgmlType::IQ3_S && t.down->type == GgmlType::Q8_0, "layer tensor set");
        CHECK(t.gate->byte_size() == L[1].gate.size() && std::memcmp(t.gate->data, L[1].gate.data(), L[1].gate.size()) == 0, "gate bytes come back from the mapping");
        CHECK(std::memcmp(t.router->data, L[1].router.data(), L[1].router.size() * 4) == 0, "router floats come back from the mapping");
        CHECK(g.tensor_file_offset(*t.up) == g.data_offset() + t.up->relative_offset && t.up->relative_offset % 32 == 0, "file offsets");
        CHECK(throws([&] { qwen38_moe_tensors(g, 2); }), "a layer the file does not hold must throw");
    }
    CHECK(throws([&] { GgufFile missing(path + ".nope"); }), "opening an absent file must throw");
    unlink(path.c_str());

    // the slot pool's default size (src/qwen38_tuning.hpp:88-116 names 40 GB -> 22 GiB and 80 GB -> 52 GiB)
    unsetenv("WARODECODE_EXPERT_CACHE_MIB");
    CHECK(default_expert_cache_mib(size_t{40} << 30) == 22 * 1024 && default_expert_cache_mib(size_t{80} << 30) == 52 * 1024, "cache size rule");
    CHECK(default_expert_cache_mib(size_t{8} << 30) == 512 && default_expert_cache_mib(size_t{288} << 30) == 64 * 1024, "cache size clamps");
    setenv("WARODECODE_EXPERT_CACHE_MIB", "20000", 1);
    CHECK(default_expert_cache_mib(size_t{80} << 30) == 20000, "cache size override");
    unsetenv("WARODECODE_EXPERT_CACHE_MIB");
    CHECK(default_expert_prefetch_depth(size_t{130} << 30) == 3 && default_expert_prefetch_depth(size_t{80} << 30) == 2 &&
              default_expert_prefetch_depth(size_t{24} << 30) == 1, "read-ahead depth rule");
    Q8_1Buffer q81;
    CHECK(throws([&] { q81.initialize(33); }) && throws([&] { q81.initialize(0); }), "Q8_1 buffer needs a positive multiple of 32");

    // The reference's own files (copied as data) with the answers its tests check or print:
    // tests/gguf_parser_test.cpp:6-8 prints version, tensor count and data offset of tests/min.gguf (3, 1, 160: the
    // header ends at byte 134 and general.alignment is 32); tests/gguf_array_test.cpp:11-27 asserts the arrays of the
    // fixture tests/make_qwen38_fixture.py writes; tests/gguf_type_size_test.cpp:17-25 the block sizes.
    const char *env = std::getenv("WD_GOLDEN_DIR");
    const std::string golden = env ? env : "tests/golden";
    {
        GgufFile g(golden + "/gguf/min.gguf");
        CHECK(g.version() == 3 && g.tensors().size() == 1 && g.data_offset() == 160, "min.gguf: %u %zu %zu", g.version(), g.tensors().size(), g.data_offset());
        CHECK(g.string_meta("general.architecture") == "llama" && g.uint_meta("general.alignment") == 32, "min.gguf metadata");
        const TensorInfo &t = g.tensor("vec");
        const float want[4] = {1.0f, 2.0f, 3.0f, 4.0f};
        CHECK(t.type == GgmlType::F32 && t.dims == std::vector<uint64_t>({4}) && t.byte_size() == 16 && g.tensor_file_offset(t) == 160 &&
                  std::memcmp(t.data, want, 16) == 0, "min.gguf tensor");
    }
    {
        GgufFile g(golden + "/gguf/qwen38-fixture-00001-of-00002.gguf");
        CHECK(g.version() == 3 && g.tensors().empty() && g.data_offset() == 2400, "fixture header: %u %zu %zu", g.version(), g.tensors().size(), g.data_offset());
        const std::vector<int64_t> ratios = g.int_array_meta("qwen4exp.attention.compress_ratios");
        CHECK(ratios.size() == 49 && ratios[3] == 8 && ratios[48] == 0, "compress_ratios");
        const std::vector<uint64_t> ple = g.uint_array_meta("qwen4exp.ple.layers");
        CHECK(ple.size() == 1 && ple[0] == 0, "ple.layers (an int32 array read as unsigned)");
        CHECK(g.uint_array_meta("qwen4exp.ple.layer_multipliers") == std::vector<uint64_t>({3, 5, 7}), "ple.layer_multipliers");
        const std::vector<uint64_t> offsets = g.uint_array_meta("qwen4exp.ple.head_offsets"), sizes = g.uint_array_meta("qwen4exp.ple.head_vocab_sizes");
        CHECK(offsets.size() == 16 && sizes.size() == 16 && offsets.back() == 150 && sizes.back() == 10, "ple head arrays");
        CHECK(g.number_array_meta("qwen4exp.rope.dimension_sections") == std::vector<double>({11, 11, 10, 0}), "rope sections as numbers");
        CHECK(g.number_meta("qwen4exp.expert_weights_scale", 0.0) == 1.25 && g.uint_meta("qwen4exp.hyper_connection.count") == 4, "fixture scalars");
        CHECK(g.has_meta("qwen4exp.ple.layers") && !g.has_meta("qwen4exp.absent"), "has_meta");
        CHECK(throws([&] { g.int_array_meta("qwen4exp.absent"); }) && throws([&] { g.uint_array_meta("qwen4exp.expert_weights_scale"); }), "array accessors refuse absent keys and scalars");
    }
    auto size_of = [](GgmlType type, uint64_t n) {
        TensorInfo ti{"test", {n}, type, 0, nullptr};
        return ti.byte_size();
    };
    CHECK(size_of(GgmlType::F32, 32) == 128 && size_of(GgmlType::F16, 32) == 64 && size_of(GgmlType::BF16, 32) == 64, "float type sizes");
    CHECK(size_of(GgmlType::Q4_0, 32) == 18 && size_of(GgmlType::Q8_0, 32) == 34 && size_of(GgmlType::Q6_K, 256) == 210, "Q4_0 / Q8_0 / Q6_K sizes");
    CHECK(size_of(GgmlType::IQ4_NL, 32) == 18 && size_of(GgmlType::IQ3_S, 256) == 110 && size_of(GgmlType::IQ2_S, 256) == 82, "IQ type sizes");
}

// The reference's three calls, then the read-back a caller does.
static std::vector<float> run_three_calls(int layer, const HostLayer &L, const GpuMatrix &router, GpuExpertCache &cache,
                                          const Qwen38SharedExpertWeights &shared, Qwen38MoeScratch &scratch, const DeviceFloatArray &x,
                                          DeviceFloatArray &out, Stream stream) {
    run_qwen38_routed_moe_separate_f32_x(layer, x.data, router, L.t_gate, L.t_up, L.t_down, cache, scratch, nullptr, 1.0f, stream);
    run_qwen38_shared_expert_f32_x(x.data, shared, scratch, stream);
    q38_finish_moe_f32(scratch, out.data, stream);
    check(wd_stream_sync(stream), "sync");
    std::vector<float> h(L.H);
    out.download(h.data());
    return h;
}

static void gpu_checks() {
    check(wd_init(0), "wd_init");
    void *stream = nullptr;
    check(wd_stream_create(&stream), "stream");
    const int H = 512, F = 128, E = 32, k = 4, layers = 3;
    std::vector<HostLayer> L;
    for (int l = 0; l < layers; ++l) L.push_back(make_layer(1000 + l, H, F, E, k));

    // operators: Q8_K quantiser + IQ3_S GEMV against the oracle
    {
        Rng r(7);
        const std::vector<float> x = rms_normed(r, H);
        DeviceFloatArray dx;
        dx.upload(x.data(), H);
        DeviceArray<int8_t> qs(H);
        DeviceFloatArray sc(H / 256), y(F);
        DeviceArray<int16_t> bs(H / 16);
        launch_q8_k_quantize_f32(dx.data, H, qs.data, sc.data, bs.data, stream);
        TensorInfo one{"gate0", {static_cast<uint64_t>(H), static_cast<uint64_t>(F)}, GgmlType::IQ3_S, 0, L[0].gate.data()};
        LowBitMatrix w = upload_lowbit_matrix(one);
        launch_iq3_s_gemv_q8_k_f32(w, qs.data, sc.data, y.data, stream);
        check(wd_stream_sync(stream), "sync");
        std::vector<int8_t> oq(H);
        std::vector<float> od(H / 256), want(F), got(F);
        std::vector<int16_t> ob(H / 16);
        wdo_quantize_q8_K(x.data(), H, oq.data(), od.data(), ob.data());
        wdo_gemv(WDO_IQ3_S, L[0].gate.data(), F, H, oq.data(), od.data(), want.data(), nullptr);
        y.download(got.data());
        CHECK(same_bits(got.data(), want.data(), F), "launch_iq3_s_gemv_q8_k_f32 differs from the oracle");
    }

    // the output head: Q6_K x Q8_K from the caller's F32 activation, against the oracle
    {
        Rng r(11);
        const int V = 1003;
        const std::vector<float> x = rms_normed(r, H);
        std::vector<uint8_t> head(static_cast<size_t>(V) * (H / 256) * 210);
        for (auto &b : head) b = static_cast<uint8_t>(r.u32());
        for (size_t i = 0; i < head.size() / 210; ++i) {
            const uint16_t d = wdo_f32_to_f16(std::fabs(r.normal()) * 1e-5f);
            std::memcpy(&head[i * 210 + 208], &d, 2);
        }
        TensorInfo info{"output.weight", {static_cast<uint64_t>(H), static_cast<uint64_t>(V)}, GgmlType::Q6_K, 0, head.data()};
        LowBitMatrix w = upload_lowbit_matrix(info);
        CHECK(lowbit_q6_k_head_q8_k_eligible(w), "a Q6_K matrix with 256-multiple columns is eligible");
        DeviceFloatArray dx, y(V);
        dx.upload(x.data(), H);
        launch_q6_k_head_gemv_q8_k_from_f32(w, dx.data, y.data, stream);
        launch_q6_k_head_gemv_q8_k_from_f32(w, dx.data, y.data, stream);  // the kept scratch is reused
        check(wd_stream_sync(stream), "sync");
        std::vector<int8_t> oq(H);
        std::vector<float> od(H / 256), want(V), got(V);
        std::vector<int16_t> ob(H / 16);
        wdo_quantize_q8_K(x.data(), H, oq.data(), od.data(), ob.data());
        wdo_gemv_q6_K(head.data(), V, H, oq.data(), od.data(), ob.data(), want.data(), nullptr);
        y.download(got.data());
        CHECK(same_bits(got.data(), want.data(), V), "launch_q6_k_head_gemv_q8_k_from_f32 differs from the oracle");
        LowBitMatrix q8 = borrow_lowbit_matrix(w.data, V, H, GgmlType::Q8_0, w.bytes);
        CHECK(throws([&] { launch_q6_k_head_gemv_q8_k_from_f32(q8, dx.data, y.data, stream); }), "the head path refuses other types");
        CHECK(throws([&] { launch_q6_k_gemv_q8_k_f32(w, nullptr, nullptr, nullptr, y.data, stream, 48); }), "threads must be a multiple of 32");
    }

    {   // launch_q8_0_gemv_q8_1_f32 through Q8_1Buffer (src/lowbit.cuh:251-362)
        const int R = 96;
        Rng r(4242);
        const std::vector<uint8_t> wq = random_blocks(r, WDO_Q8_0, R, H, 0.02f / 127.0f);
        TensorInfo tw{"w", {static_cast<uint64_t>(H), static_cast<uint64_t>(R)}, GgmlType::Q8_0, 0, wq.data()};
        LowBitMatrix w = upload_lowbit_matrix(tw);
        const std::vector<float> x = rms_normed(r, H);
        DeviceFloatArray dx(H), dy(R);
        dx.upload(x.data(), H);
        Q8_1Buffer buf;
        buf.initialize(H);
        CHECK(throws([&] { buf.initialize(H); }), "double initialisation of the Q8_1 buffer must throw");
        launch_q8_0_gemv_q8_1_f32(w, dx.data, dy.data, buf, stream);
        check(wd_stream_sync(stream), "sync");
        std::vector<float> got(R), want(R);
        dy.download(got.data());
        std::vector<int8_t> q(H);
        std::vector<uint16_t> d(H / 32);
        wdo_quantize_q8_1(x.data(), H, q.data(), d.data());
        wdo_gemv_q8_0_q8_1(wq.data(), R, H, q.data(), d.data(), want.data(), nullptr);
        CHECK(same_bits(got.data(), want.data(), R), "launch_q8_0_gemv_q8_1_f32 differs from the oracle");
        Q8_1Buffer small;
        small.initialize(H / 2);
        CHECK(throws([&] { launch_q8_0_gemv_q8_1_f32(w, dx.data, dy.data, small, stream); }), "a buffer smaller than the row must be refused");
    }

    std::vector<GpuMatrix> routers;
    std::vector<Qwen38SharedExpertWeights> shared(layers);
    for (int l = 0; l < layers; ++l) {
        routers.push_back(upload_matrix(L[l].t_router));
        shared[l].gate_input_f32.upload(L[l].gate_inp.data(), H);
        TensorInfo g{"sg", {static_cast<uint64_t>(H), static_cast<uint64_t>(F)}, GgmlType::Q8_0, 0, L[l].sg.data()};
        TensorInfo u{"su", {static_cast<uint64_t>(H), static_cast<uint64_t>(F)}, GgmlType::Q8_0, 0, L[l].su.data()};
        TensorInfo d{"sd", {static_cast<uint64_t>(F), static_cast<uint64_t>(H)}, GgmlType::Q8_0, 0, L[l].sd.data()};
        shared[l].gate = upload_lowbit_matrix(g), shared[l].up = upload_lowbit_matrix(u), shared[l].down = upload_lowbit_matrix(d);
    }
    Qwen38MoeScratch scratch;
    scratch.initialize(E, k, H, F);
    CHECK(throws([&] { scratch.initialize(E, k, H, F); }), "double initialisation must throw");
    CHECK(throws([&] { q38_finish_moe_f32(scratch, scratch.d_accum(), stream); }), "output aliasing the routed sum must throw");

    ExpertCacheOptions opt;
    opt.layer_count = layers;
    const size_t slot = L[0].t_gate.byte_size() / E * 2 + L[0].t_down.byte_size() / E;

    // (1) room for everything: preloaded, no host round trip; (2) 10 slots for 96 experts: LRU with misses
    for (int mode = 0; mode < 2; ++mode) {
        GpuExpertCache cache;
        const size_t want_slots = mode == 0 ? static_cast<size_t>(layers) * E : 10;
        cache.initialize((want_slots * slot + (1u << 20) - 1) >> 20, L[0].t_gate, L[0].t_up, L[0].t_down, 0, 0, 0, opt);
        CHECK(cache.slot_bytes() == slot, "slot bytes %zu vs %zu", cache.slot_bytes(), slot);
        CHECK(cache.slot_count() >= want_slots, "slot count %zu", cache.slot_count());
        for (int l = 0; l < layers; ++l) cache.register_layer_experts(l, L[l].t_gate, L[l].t_up, L[l].t_down);
        if (mode == 0)
            for (int l = 0; l < layers; ++l) cache.preload_layer(l, stream);
        CHECK(mode == 1 || cache.layer_resident(0), "layer 0 should be resident after the preload");
        Rng r(99 + mode);
        DeviceFloatArray dx(H), dout(H);
        for (int token = 0; token < 4; ++token) {
            for (int l = 0; l < layers; ++l) {
                const std::vector<float> x = rms_normed(r, H);
                dx.upload(x.data(), H);
                const std::vector<float> got = run_three_calls(l, L[l], routers[l], cache, shared[l], scratch, dx, dout, stream);
                std::vector<float> want(H), routed(H);
                std::vector<int> ids(k);
                wdo_dump dump{};
                dump.ids = ids.data(), dump.routed = routed.data();
                wdo_moe_layer(&L[l].o, x.data(), want.data(), &dump, 0);
                CHECK(same_bits(got.data(), want.data(), H), "mode %d token %d layer %d: three-call output differs from the oracle", mode, token, l);
                std::vector<int> gids(k);
                check(wd_memcpy_d2h(gids.data(), scratch.d_ids(), sizeof(int) * k, nullptr), "ids");
                CHECK(gids == ids, "mode %d token %d layer %d: routed ids differ", mode, token, l);
                std::vector<float> acc(H);
                check(wd_memcpy_d2h(acc.data(), scratch.d_accum(), sizeof(float) * H, nullptr), "accum");
                CHECK(same_bits(acc.data(), routed.data(), H), "mode %d token %d layer %d: routed sum differs", mode, token, l);
                if (token == 0) {
                    // the runners by element type (src/qwen38_moe.cuh:3521-3534): half input, half output, the selected
                    // experts' down outputs captured as half - against the oracle on the widened input
                    std::vector<uint16_t> xh(H);
                    std::vector<float> xw(H);
                    for (int i = 0; i < H; ++i) xh[i] = wdo_f32_to_f16_rn(x[i]), xw[i] = wdo_f16_to_f32(xh[i]);
                    DeviceArray<half_bits> dxh(H), dout_h(H);
                    check(wd_memcpy_h2d(dxh.data, xh.data(), sizeof(uint16_t) * H, nullptr), "half input");
                    std::vector<float> want_h(H), routed_h(H), eo(static_cast<size_t>(k) * H);
                    wdo_dump dh{};
                    dh.routed = routed_h.data(), dh.expert_out = eo.data();
                    wdo_moe_layer(&L[l].o, xw.data(), want_h.data(), &dh, 0);
                    run_qwen38_routed_moe_separate<true, half_bits, half_bits>(l, dxh.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache,
                                                                              scratch, dout_h.data, 1.0f, stream, false, scratch.selected_output_trace());
                    check(wd_stream_sync(stream), "sync");
                    std::vector<uint16_t> got_h(H), got_tr(static_cast<size_t>(k) * H);
                    check(wd_memcpy_d2h(got_h.data(), dout_h.data, sizeof(uint16_t) * H, nullptr), "half output");
                    check(wd_memcpy_d2h(got_tr.data(), scratch.selected_output_trace(), sizeof(uint16_t) * got_tr.size(), nullptr), "trace");
                    bool ok_h = true, ok_tr = true;
                    for (int i = 0; i < H; ++i) ok_h = ok_h && got_h[i] == wdo_f32_to_f16_rn(routed_h[i]);
                    for (size_t i = 0; i < got_tr.size(); ++i) ok_tr = ok_tr && got_tr[i] == wdo_f32_to_f16_rn(eo[i]);
                    CHECK(ok_h, "mode %d layer %d: half-in half-out routed sum differs from the rounded oracle", mode, l);
                    CHECK(ok_tr, "mode %d layer %d: selected expert trace differs from the rounded oracle", mode, l);
                    // float output from half input equals the float runner on the widened input
                    DeviceFloatArray dxw(H), o1(H), o2(H);
                    dxw.upload(xw.data(), H);
                    run_qwen38_routed_moe_separate<false, float, half_bits>(l, dxh.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache,
                                                                           scratch, o1.data, 1.0f, stream);
                    run_qwen38_routed_moe_separate<false, float, float>(l, dxw.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, scratch,
                                                                       o2.data, 1.0f, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> a1(H), a2(H);
                    o1.download(a1.data()), o2.download(a2.data());
                    CHECK(same_bits(a1.data(), a2.data(), H) && same_bits(a1.data(), routed_h.data(), H), "mode %d layer %d: half-input runner differs", mode, l);
                    CHECK(throws([&] { run_qwen38_routed_moe_separate<true, float, float>(l, dxw.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down,
                                                                                         cache, scratch, o2.data, 1.0f, stream); }),
                          "a capturing run without a trace buffer must throw");
                }
                if (mode == 1) {
                    // the one-call wrappers with a cache that cannot hold the layer: the ids go through the host instead of
                    // the kernels indexing a slot table with holes in it
                    CHECK(!cache.layer_resident(l), "layer %d cannot be resident in 10 slots", l);
                    run_qwen38_moe_layer_f32_x(l, dx.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, shared[l], scratch, dout.data, 1.0f, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> fused(H);
                    dout.download(fused.data());
                    CHECK(same_bits(fused.data(), want.data(), H), "token %d layer %d: one-call wrapper over the LRU cache differs from the oracle", token, l);
                    CHECK(wd_moe_scratch_status(scratch.handle()) == 0, "token %d layer %d: status word set", token, l);
                    const int hc = 4;
                    Qwen38HcF32DebugScratch hcs;
                    hcs.initialize(H, hc);
                    std::vector<float> res0(static_cast<size_t>(hc) * H), inject(hc);
                    for (auto &v : res0) v = r.normal();
                    for (auto &v : inject) v = 2.0f * r.normal();
                    check(wd_memcpy_h2d(hcs.inject(), inject.data(), sizeof(float) * hc, nullptr), "inject");
                    std::vector<float> want_res = res0;
                    wdo_hc_combine_f32(want_res.data(), want.data(), inject.data(), H, hc, 0);
                    DeviceFloatArray dres;
                    dres.upload(res0.data(), res0.size());
                    run_qwen38_moe_layer_hc_f32_x(l, dx.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, shared[l], scratch, dout.data,
                                                  dres.data, hcs, 1.0f, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> got_res(res0.size());
                    dres.download(got_res.data());
                    CHECK(same_bits(got_res.data(), want_res.data(), got_res.size()), "token %d layer %d: wrapper with combine over the LRU cache differs", token, l);
                }
                if (mode == 0) {
                    run_qwen38_moe_layer_f32_x(l, dx.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, shared[l], scratch, dout.data, 1.0f, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> fused(H);
                    dout.download(fused.data());
                    CHECK(same_bits(fused.data(), want.data(), H), "token %d layer %d: fused call differs from the oracle", token, l);
                    // the layer with the hyper-connection combine folded in, and the combine as calls of its own
                    const int hc = 4;
                    Qwen38HcF32DebugScratch hcs;
                    hcs.initialize(H, hc);
                    std::vector<float> res0(static_cast<size_t>(hc) * H), inject(hc);
                    for (auto &v : res0) v = r.normal();
                    for (auto &v : inject) v = 2.0f * r.normal();
                    check(wd_memcpy_h2d(hcs.inject(), inject.data(), sizeof(float) * hc, nullptr), "inject");
                    std::vector<float> want_res = res0;
                    wdo_hc_combine_f32(want_res.data(), want.data(), inject.data(), H, hc, 0);
                    DeviceFloatArray dres, dres2, dres3;
                    dres.upload(res0.data(), res0.size()), dres2.upload(res0.data(), res0.size()), dres3.upload(res0.data(), res0.size());
                    run_qwen38_moe_layer_hc_f32_x(l, dx.data, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, shared[l], scratch, dout.data,
                                                  dres.data, hcs, 1.0f, stream);
                    run_qwen38_hc_combine_f32_block_f32_inject(dres2.data, dout.data, hcs, stream);
                    run_qwen38_hc_combine_moe_f32_inject(dres3.data, scratch.d_accum(), scratch.down_f32(), scratch.d_shared_gate(), hcs, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> got_res(res0.size());
                    dres.download(got_res.data());
                    CHECK(same_bits(got_res.data(), want_res.data(), got_res.size()), "token %d layer %d: folded combine differs from the oracle", token, l);
                    dres2.download(got_res.data());
                    CHECK(same_bits(got_res.data(), want_res.data(), got_res.size()), "token %d layer %d: combine differs from the oracle", token, l);
                    dres3.download(got_res.data());
                    CHECK(same_bits(got_res.data(), want_res.data(), got_res.size()), "token %d layer %d: combine from the parts differs from the oracle", token, l);
                }
            }
        }
        const wd_expert_cache_stats st = cache.stats();
        if (mode == 0) {
            CHECK(st.evictions == 0 && st.resident == static_cast<uint64_t>(layers) * E, "resident mode evicted (%llu) or lost experts (%llu)",
                  static_cast<unsigned long long>(st.evictions), static_cast<unsigned long long>(st.resident));
        } else {
            CHECK(st.misses > 0 && st.evictions > 0 && st.resident <= cache.slot_count() && cache.slot_count() < static_cast<size_t>(layers) * E, "LRU mode: misses %llu evictions %llu resident %llu",
                  static_cast<unsigned long long>(st.misses), static_cast<unsigned long long>(st.evictions), static_cast<unsigned long long>(st.resident));
            CHECK(st.bytes_copied == st.misses * slot, "bytes copied %llu vs misses x slot", static_cast<unsigned long long>(st.bytes_copied));
            const ExpertDeviceWeights v = cache.acquire(0, 5, L[0].t_gate, L[0].t_up, L[0].t_down, stream);
            check(wd_stream_sync(stream), "sync");
            std::vector<uint8_t> back(v.gate.bytes);
            check(wd_memcpy_d2h(back.data(), v.gate.data, v.gate.bytes, nullptr), "slot read-back");
            CHECK(std::memcmp(back.data(), expert_slice(L[0].t_gate, 5).data, v.gate.bytes) == 0 && !v.gate.owns, "acquired view must hold the expert's gate bytes");
        }
        // a batch of tokens through each layer (resident: on the device throughout; LRU pool of 10 slots: the union of
        // two tokens' experts is acquired at once), every token against its own oracle pass
        {
            const int T = mode == 0 ? 3 : 2;
            std::vector<Qwen38MoeScratch> ts(T);
            std::vector<Qwen38MoeScratch *> tp;
            for (auto &q : ts) q.initialize(E, k, H, F), tp.push_back(&q);
            Rng rt(555 + mode);
            DeviceFloatArray dxs(static_cast<size_t>(T) * H), douts(static_cast<size_t>(T) * H);
            for (int l = 0; l < layers; ++l) {
                std::vector<float> xs(static_cast<size_t>(T) * H);
                for (int t = 0; t < T; ++t) {
                    const std::vector<float> x = rms_normed(rt, H);
                    std::copy(x.begin(), x.end(), xs.begin() + static_cast<size_t>(t) * H);
                }
                dxs.upload(xs.data(), xs.size());
                run_qwen38_moe_tokens_f32_x(l, dxs.data, T, routers[l], L[l].t_gate, L[l].t_up, L[l].t_down, cache, shared[l], tp, douts.data, 1.0f, stream);
                check(wd_stream_sync(stream), "sync");
                std::vector<float> got(xs.size()), want(H);
                douts.download(got.data());
                for (int t = 0; t < T; ++t) {
                    wdo_moe_layer(&L[l].o, xs.data() + static_cast<size_t>(t) * H, want.data(), nullptr, 0);
                    CHECK(same_bits(got.data() + static_cast<size_t>(t) * H, want.data(), H), "mode %d layer %d token %d of the batch differs from the oracle", mode, l, t);
                }
                // the same tokens through the reference's batch object, driven as its caller drives it
                // (src/qwen38_mtp.cuh:702-747): selection of all tokens, the union acquired expert by expert, every pair
                // told its views, one pass, the routed sums out as float and as half
                {
                    Qwen38MoeTokenBatch batch;
                    CHECK(batch.compatible(cache, scratch, L[l].t_gate, L[l].t_up, L[l].t_down, T) == (mode == 0), "mode %d: batch compatibility (8 slots per selection)", mode);
                    CHECK(!batch.compatible(cache, scratch, L[l].t_gate, L[l].t_up, L[l].t_down, kMoeBatchTokenMax + 1) &&
                              !batch.compatible(cache, scratch, L[l].t_down, L[l].t_up, L[l].t_down, T), "batch bound and tensor types");
                    std::vector<const float *> acts;
                    for (int t = 0; t < T; ++t) acts.push_back(dxs.data + static_cast<size_t>(t) * H);
                    batch.open_all(scratch, routers[l], acts, 1.0f, stream, false);
                    std::vector<int> union_expert, union_slot(static_cast<size_t>(T) * k);
                    std::vector<ExpertDeviceWeights> union_weights;
                    for (int p = 0; p < T * k; ++p) {
                        const int expert = scratch.h_ids()[p];
                        int at = -1;
                        for (size_t q = 0; q < union_expert.size(); ++q)
                            if (union_expert[q] == expert) at = static_cast<int>(q);
                        if (at < 0) {
                            at = static_cast<int>(union_expert.size());
                            union_expert.push_back(expert);
                            union_weights.push_back(cache.acquire(l, expert, L[l].t_gate, L[l].t_up, L[l].t_down, stream));
                        }
                        union_slot[static_cast<size_t>(p)] = at;
                    }
                    CHECK(!batch.resolved(), "pairs without views are not resolved");
                    for (int p = 0; p < T * k; ++p) {
                        const ExpertDeviceWeights &w = union_weights[static_cast<size_t>(union_slot[static_cast<size_t>(p)])];
                        batch.set_pair_weights(p, w.gate, w.up, w.down);
                    }
                    CHECK(batch.resolved(true), "mode %d layer %d: the batch should be runnable", mode, l);
                    batch.run(scratch, L[l].t_gate, L[l].t_up, L[l].t_down, stream);
                    DeviceFloatArray bo(static_cast<size_t>(T) * H);
                    DeviceArray<half_bits> bh(static_cast<size_t>(T) * H);
                    batch.write_output(scratch, bo.data, nullptr, stream);
                    batch.write_output(scratch, nullptr, bh.data, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> sums(static_cast<size_t>(T) * H), routed(H);
                    std::vector<uint16_t> halves(sums.size());
                    bo.download(sums.data());
                    check(wd_memcpy_d2h(halves.data(), bh.data, sizeof(uint16_t) * halves.size(), nullptr), "half sums");
                    CHECK(batch.tokens() == T && batch.accumulated(scratch) != nullptr, "batch accessors");
                    for (int t = 0; t < T; ++t) {
                        wdo_dump dd{};
                        std::vector<int> oids(k);
                        dd.routed = routed.data(), dd.ids = oids.data();
                        wdo_moe_layer(&L[l].o, xs.data() + static_cast<size_t>(t) * H, want.data(), &dd, 0);
                        CHECK(std::equal(oids.begin(), oids.end(), scratch.h_ids() + t * k), "mode %d layer %d token %d: batch selection differs", mode, l, t);
                        CHECK(same_bits(sums.data() + static_cast<size_t>(t) * H, routed.data(), H), "mode %d layer %d token %d: batch routed sum differs from the oracle", mode, l, t);
                        bool okh = true;
                        for (int i = 0; i < H; ++i) okh = okh && halves[static_cast<size_t>(t) * H + i] == wdo_f32_to_f16_rn(routed[i]);
                        CHECK(okh, "mode %d layer %d token %d: batch half output differs", mode, l, t);
                    }
                    // a slot recycled under an earlier pair shows as two pairs with one view and two experts
                    if (union_expert.size() >= 2) {
                        const ExpertDeviceWeights &w0 = union_weights[0];
                        int other = -1;
                        for (int p = 0; p < T * k; ++p)
                            if (union_slot[static_cast<size_t>(p)] == 1) other = p;
                        batch.set_pair_weights(other, w0.gate, w0.up, w0.down);
                        CHECK(batch.resolved(false) && !batch.resolved(true), "a recycled slot must fail the slot check");
                    }
                    CHECK(throws([&] { batch.set_pair_weights(kMoeBatchTokenMax * 16, union_weights[0].gate, union_weights[0].up, union_weights[0].down); }), "pair index bound");
                }
            }
        }
    }
    // the same stack driven from a model file: tensors found by name, router / shared expert uploaded from the mapping,
    // the mapping itself as the cache's host source (LRU pool, so experts stream from the file's pages)
    {
        const std::string path = write_model_file(L);
        {
            GgufFile g(path);
            std::vector<Qwen38MoeLayerTensors> T;
            std::vector<GpuMatrix> frouters;
            std::vector<Qwen38SharedExpertWeights> fshared;
            for (int l = 0; l < layers; ++l) {
                T.push_back(qwen38_moe_tensors(g, l));
                frouters.push_back(upload_matrix(*T[l].router));
                fshared.push_back(load_qwen38_shared_expert(g, l, H, F));
            }
            CHECK(throws([&] { load_qwen38_shared_expert(g, 0, H, F + 32); }), "shared expert shape mismatch must throw");
            GpuExpertCache cache;
            cache.initialize((12 * slot + (1u << 20) - 1) >> 20, *T[0].gate, *T[0].up, *T[0].down, 0, 0, 0, opt);
            for (int l = 0; l < layers; ++l) cache.register_layer_experts(l, *T[l].gate, *T[l].up, *T[l].down);
            CHECK(attach_mapped_expert_files(cache, 2) == 1, "the model file's mapping is found through /proc/self/maps");
            attach_expert_file(cache, g, 2);  // naming the file as well changes nothing: misses come through pread and the pinned ring
            Rng r(321);
            DeviceFloatArray dx(H), dout(H);
            for (int token = 0; token < 3; ++token)
                for (int l = 0; l < layers; ++l) {
                    const std::vector<float> x = rms_normed(r, H);
                    dx.upload(x.data(), H);
                    run_qwen38_routed_moe_separate_f32_x(l, dx.data, frouters[l], *T[l].gate, *T[l].up, *T[l].down, cache, scratch, nullptr,
                                                         static_cast<float>(g.number_meta("qwen38.expert_weights_scale", 1.0)), stream);
                    run_qwen38_shared_expert_f32_x(dx.data, fshared[l], scratch, stream);
                    q38_finish_moe_f32(scratch, dout.data, stream);
                    check(wd_stream_sync(stream), "sync");
                    std::vector<float> got(H), want(H);
                    dout.download(got.data());
                    wdo_moe_layer(&L[l].o, x.data(), want.data(), nullptr, 0);
                    CHECK(same_bits(got.data(), want.data(), H), "model file, token %d layer %d: output differs from the oracle", token, l);
                }
            CHECK(cache.stats().misses > 0, "the file-backed pool should have taken misses");
        }
        unlink(path.c_str());
    }
    // fused gate_up tensor (2 * ffn rows per expert) through the fused runner, LRU pool of 10+ slots
    {
        const size_t gb = L[0].t_gate.byte_size() / E;
        std::vector<uint8_t> fused(2 * gb * E);
        for (int e = 0; e < E; ++e) {
            std::memcpy(&fused[2 * gb * e], &L[0].gate[gb * e], gb);
            std::memcpy(&fused[2 * gb * e + gb], &L[0].up[gb * e], gb);
        }
        TensorInfo t_gu{"ffn_gate_up_exps.weight", {static_cast<uint64_t>(H), static_cast<uint64_t>(2 * F), static_cast<uint64_t>(E)}, GgmlType::IQ3_S, 0, fused.data()};
        GpuExpertCache cache;
        cache.initialize((10 * slot + (1u << 20) - 1) >> 20, L[0].t_gate, L[0].t_up, L[0].t_down, 0, 0, 0, opt);
        Rng r(321);
        DeviceFloatArray dx(H), dout(H);
        for (int token = 0; token < 3; ++token) {
            const std::vector<float> x = rms_normed(r, H);
            dx.upload(x.data(), H);
            run_qwen38_routed_moe_fused_f32_x(0, dx.data, routers[0], t_gu, L[0].t_down, cache, scratch, nullptr, 1.0f, stream);
            run_qwen38_shared_expert_f32_x(dx.data, shared[0], scratch, stream);
            q38_finish_moe_f32(scratch, dout.data, stream);
            check(wd_stream_sync(stream), "sync");
            std::vector<float> got(H), want(H);
            dout.download(got.data());
            wdo_moe_layer(&L[0].o, x.data(), want.data(), nullptr, 0);
            CHECK(same_bits(got.data(), want.data(), H), "fused gate_up tensor, token %d: output differs from the oracle", token);
        }
        CHECK(wd_moe_scratch_status(scratch.handle()) == 0, "an in-dispatch wait ran out");
    }
    // the site profiler, bracketed the way the reference's stage code brackets a token (src/qwen38_moe.cuh:296-535):
    // a ten-slot pool, so every layer goes selection -> ids to the host -> acquire -> expert dispatches
    {
        Q38MoeKernelProfiler &prof = Q38MoeKernelProfiler::instance();
        CHECK(!prof.enabled(), "the profiler is off unless WARODECODE_MOE_PROFILE is set");
        check(wd_profile_enable(1), "profiler on");
        check(wd_profile_reset(), "profiler reset");
        GpuExpertCache cache;
        cache.initialize((10 * slot + (1u << 20) - 1) >> 20, L[0].t_gate, L[0].t_up, L[0].t_down, 0, 0, 0, opt);
        for (int l = 0; l < layers; ++l) cache.register_layer_experts(l, L[l].t_gate, L[l].t_up, L[l].t_down);
        Rng r(321);
        DeviceFloatArray dx(H), dout(H);
        const int tokens = 2;
        for (int token = 0; token < tokens; ++token) {
            {
                Q38MoeKernelScope stage(kQ38MoeSiteStageTotal, stream);
                for (int l = 0; l < layers; ++l) {
                    const std::vector<float> x = rms_normed(r, H);
                    dx.upload(x.data(), H);
                    const std::vector<float> got = run_three_calls(l, L[l], routers[l], cache, shared[l], scratch, dx, dout, stream);
                    std::vector<float> want(H);
                    wdo_moe_layer(&L[l].o, x.data(), want.data(), nullptr, 0);
                    CHECK(same_bits(got.data(), want.data(), H), "profiled token %d layer %d: output differs from the oracle", token, l);
                }
            }
            check(wd_device_sync(), "sync");
            prof.flush_token();
        }
        const unsigned long long n = static_cast<unsigned long long>(tokens) * layers;
        const Q38MoeSiteStat stage = prof.site(kQ38MoeSiteStageTotal), routed = prof.site(kQ38MoeSiteRoutedTotal),
                             select = prof.site(kQ38MoeSiteRouter), sync = prof.site(kQ38MoeSiteRouterSync),
                             acquire = prof.site(kQ38MoeSiteAcquire), sh = prof.site(kQ38MoeSiteShared), fin = prof.site(kQ38MoeSiteFinish);
        CHECK(stage.calls == tokens && stage.overflow == 0 && stage.elapsed_fail == 0, "stage brackets: %llu", stage.calls);
        CHECK(routed.calls == n && select.calls == n && sync.calls == n && acquire.calls == n, "per-layer brackets: %llu %llu %llu %llu of %llu",
              routed.calls, select.calls, sync.calls, acquire.calls, n);
        CHECK(sh.calls == n && fin.calls == n, "shared expert and finish brackets: %llu %llu", sh.calls, fin.calls);
        CHECK(stage.total_ms >= 0.98 * routed.total_ms && routed.total_ms >= 0.98 * select.total_ms && select.total_ms > 0.0, "device times nest");
        CHECK(stage.total_host_ms >= routed.total_host_ms && routed.total_host_ms >= select.total_host_ms && select.total_host_ms >= sync.total_host_ms &&
                  sync.total_host_ms > 0.0, "host times nest");
        const std::string text = prof.summary();
        CHECK(text.find("[moe-profile] tokens=2 unit=ms_per_token") == 0 && text.find("moe.router_select") != std::string::npos &&
                  text.find("moe.fused.c") != std::string::npos && text.find("moe.batch.gate_up") == std::string::npos,
              "summary:\n%s", text.c_str());
        CHECK(std::string(q38_moe_site_name(kQ38MoeSiteRouterTopk)) == "moe.router.topk" && kQ38MoeSiteCount == 24, "site names");
        check(wd_profile_enable(0), "profiler off");
        check(wd_profile_reset(), "profiler reset");
    }
    wd_stream_destroy(stream);
}

int main(int argc, char **argv) {
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
    try {
        host_only_checks();
        if (!host_only) gpu_checks();
    } catch (const std::exception &e) {
        std::printf("FAIL: unexpected exception: %s\n", e.what());
        return 2;
    }
    std::printf("%d checks, %d failures\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
