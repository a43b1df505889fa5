// GGUF container reader (versions 2 and 3): memory-maps the file read-only, parses the header, the metadata
// and the tensor directory, and hands out tensor views that point into the mapping - the form in which the
// expert cache and the upload helpers take weights (raw GGUF block bytes, never repacked).
// Same role as the reference's GgufFile / MappedFile (src/gguf.hpp:71-491).  Host code only.
#include "wd_common.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

using namespace wd;

namespace {

struct GgufValue {
    uint32_t type = 0;        // GGUF value type of the scalar, or of the elements when is_array
    bool is_array = false;
    uint64_t u = 0;           // unsigned scalars and bool
    int64_t i = 0;            // signed scalars
    double f = 0.0;           // float scalars
    std::string s;            // string scalar
    uint64_t count = 0;       // array length
    const uint8_t *raw = nullptr;  // array payload inside the mapping (fixed-size element types only)
};

struct GgufTensor {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[4] = {1, 1, 1, 1};
    uint32_t type = 0;
    uint64_t relative_offset = 0;
    uint64_t bytes = 0;  // 0 when the type's size is not known to this library
};

// Bounds-checked little-endian reader over the mapping.
struct Reader {
    const uint8_t *p;
    size_t n, at = 0;
    bool ok = true;
    bool need(size_t k) {
        if (!ok || k > n - at) ok = false;
        return ok;
    }
    template <typename T>
    T get() {
        T v{};
        if (need(sizeof(T))) {
            std::memcpy(&v, p + at, sizeof(T));
            at += sizeof(T);
        }
        return v;
    }
    std::string str() {
        const uint64_t len = get<uint64_t>();
        std::string s;
        if (len <= (1u << 24) && need(static_cast<size_t>(len))) {
            s.assign(reinterpret_cast<const char *>(p + at), static_cast<size_t>(len));
            at += static_cast<size_t>(len);
        } else {
            ok = false;
        }
        return s;
    }
};

size_t scalar_size(uint32_t t) {
    switch (t) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
        default: return 0;  // string (8), array (9), unknown
    }
}

bool read_scalar(Reader &r, uint32_t t, GgufValue &v) {
    v.type = t;
    switch (t) {
        case 0: v.u = r.get<uint8_t>(); break;
        case 1: v.i = r.get<int8_t>(); break;
        case 2: v.u = r.get<uint16_t>(); break;
        case 3: v.i = r.get<int16_t>(); break;
        case 4: v.u = r.get<uint32_t>(); break;
        case 5: v.i = r.get<int32_t>(); break;
        case 6: v.f = r.get<float>(); break;
        case 7: v.u = r.get<uint8_t>() != 0; break;
        case 8: v.s = r.str(); break;
        case 10: v.u = r.get<uint64_t>(); break;
        case 11: v.i = r.get<int64_t>(); break;
        case 12: v.f = r.get<double>(); break;
        default: return false;
    }
    return r.ok;
}

// Bytes of a tensor's data; false when the element count or the byte count does not fit 64 bits (a crafted header
// whose product wraps would otherwise pass the bounds test with a small size).
bool tensor_bytes(const GgufTensor &t, uint64_t *bytes) {
    uint64_t n = 1;
    for (uint32_t d = 0; d < t.n_dims; ++d)
        if (__builtin_mul_overflow(n, t.dims[d], &n)) return false;
    switch (t.type) {
        case 0: return !__builtin_mul_overflow(n, uint64_t{4}, bytes);            // F32
        case 1: case 30: return !__builtin_mul_overflow(n, uint64_t{2}, bytes);   // F16, BF16
        default: break;
    }
    const uint64_t cols = t.n_dims ? t.dims[0] : 0;
    *bytes = 0;
    if (cols == 0 || cols > 0x7fffffffu) return true;
    const uint64_t row = row_bytes(static_cast<int>(t.type), static_cast<int>(cols));
    return !__builtin_mul_overflow(n / cols, row, bytes);
}

}  // namespace

struct wd_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    size_t data_offset = 0;
    std::vector<GgufTensor> tensors;
    std::unordered_map<std::string, size_t> index;
    std::unordered_map<std::string, GgufValue> meta;
};

extern "C" {

int wd_gguf_close(wd_gguf *g) {
    if (!g) return WD_OK;
    if (g->map) ::munmap(const_cast<uint8_t *>(g->map), g->size);
    if (g->fd >= 0) ::close(g->fd);
    delete g;
    return WD_OK;
}

int wd_gguf_open(wd_gguf **out, const char *path) {
    WD_REQUIRE(out != nullptr && path != nullptr, "wd_gguf_open: null argument");
    *out = nullptr;
    wd_gguf *g = new (std::nothrow) wd_gguf;
    WD_REQUIRE(g != nullptr, "wd_gguf_open: out of host memory");
    auto bail = [&](const char *what) {
        const int rc = fail(WD_ERR_ARG, "GGUF %s: %s", path, what);
        wd_gguf_close(g);
        return rc;
    };
    g->fd = ::open(path, O_RDONLY);
    if (g->fd < 0) return bail("cannot open the file");
    struct stat st;
    if (::fstat(g->fd, &st) != 0 || st.st_size < 24) return bail("not a regular file of at least header size");
    g->size = static_cast<size_t>(st.st_size);
    void *m = ::mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) return bail("mmap failed");
    g->map = static_cast<const uint8_t *>(m);

    Reader r{g->map, g->size};
    if (r.get<uint32_t>() != 0x46554747u) return bail("magic is not 'GGUF'");
    g->version = r.get<uint32_t>();
    if (g->version < 2 || g->version > 3) return bail("unsupported version (2 and 3 are read)");
    const uint64_t n_tensors = r.get<uint64_t>(), n_kv = r.get<uint64_t>();
    if (n_tensors > 1000000 || n_kv > 1000000) return bail("implausible header counts");
    for (uint64_t i = 0; i < n_kv && r.ok; ++i) {
        const std::string key = r.str();
        const uint32_t type = r.get<uint32_t>();
        GgufValue v;
        if (type == 9) {
            v.is_array = true;
            v.type = r.get<uint32_t>();
            v.count = r.get<uint64_t>();
            const size_t es = scalar_size(v.type);
            if (es) {
                if (v.count > (r.n - r.at) / es) return bail("metadata array runs past the end of the file");
                v.raw = r.p + r.at;
                r.at += static_cast<size_t>(v.count) * es;
            } else if (v.type == 8) {
                for (uint64_t e = 0; e < v.count && r.ok; ++e) (void)r.str();
            } else {
                return bail("metadata array of an unknown element type");
            }
        } else if (!read_scalar(r, type, v)) {
            return bail("metadata value of an unknown type or past the end of the file");
        }
        g->meta.emplace(key, std::move(v));
    }
    g->tensors.reserve(static_cast<size_t>(n_tensors));
    for (uint64_t i = 0; i < n_tensors && r.ok; ++i) {
        GgufTensor t;
        t.name = r.str();
        t.n_dims = r.get<uint32_t>();
        if (t.n_dims == 0 || t.n_dims > 4) return bail("tensor with an invalid number of dimensions");
        for (uint32_t d = 0; d < t.n_dims; ++d) t.dims[d] = r.get<uint64_t>();
        t.type = r.get<uint32_t>();
        t.relative_offset = r.get<uint64_t>();
        g->index.emplace(t.name, g->tensors.size());
        g->tensors.push_back(std::move(t));
    }
    if (!r.ok) return bail("header runs past the end of the file");
    size_t alignment = 32;
    const auto a = g->meta.find("general.alignment");
    if (a != g->meta.end() && !a->second.is_array) {
        if (a->second.u) alignment = static_cast<size_t>(a->second.u);
        else if (a->second.i > 0) alignment = static_cast<size_t>(a->second.i);
    }
    if (alignment == 0 || (alignment & (alignment - 1)) != 0) return bail("general.alignment is not a power of two");
    g->data_offset = (r.at + alignment - 1) & ~(alignment - 1);
    if (g->data_offset > g->size) return bail("tensor data would start past the end of the file");
    for (GgufTensor &t : g->tensors) {
        if (!tensor_bytes(t, &t.bytes)) {
            const int rc = fail(WD_ERR_ARG, "GGUF %s: the size of tensor %s does not fit 64 bits", path, t.name.c_str());
            wd_gguf_close(g);
            return rc;
        }
        if (t.relative_offset > g->size - g->data_offset || t.bytes > g->size - g->data_offset - t.relative_offset) {
            const int rc = fail(WD_ERR_ARG, "GGUF %s: tensor %s lies outside the file", path, t.name.c_str());
            wd_gguf_close(g);
            return rc;
        }
    }
    *out = g;
    return WD_OK;
}

uint32_t wd_gguf_version(const wd_gguf *g) { return g ? g->version : 0; }
size_t wd_gguf_data_offset(const wd_gguf *g) { return g ? g->data_offset : 0; }
const uint8_t *wd_gguf_map_base(const wd_gguf *g) { return g ? g->map : nullptr; }
size_t wd_gguf_map_bytes(const wd_gguf *g) { return g ? g->size : 0; }
int wd_gguf_fd(const wd_gguf *g) { return g ? g->fd : -1; }
long long wd_gguf_tensor_count(const wd_gguf *g) { return g ? static_cast<long long>(g->tensors.size()) : 0; }

long long wd_gguf_find(const wd_gguf *g, const char *name) {
    if (!g || !name) return -1;
    const auto it = g->index.find(name);
    return it == g->index.end() ? -1 : static_cast<long long>(it->second);
}

int wd_gguf_tensor(const wd_gguf *g, long long i, wd_gguf_tensor_info *out) {
    WD_REQUIRE(g != nullptr && out != nullptr, "wd_gguf_tensor: null argument");
    WD_REQUIRE(i >= 0 && i < static_cast<long long>(g->tensors.size()), "wd_gguf_tensor: index %lld out of range", i);
    const GgufTensor &t = g->tensors[static_cast<size_t>(i)];
    out->name = t.name.c_str();
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; ++d) out->dims[d] = t.dims[d];
    out->type = t.type;
    out->relative_offset = t.relative_offset;
    out->bytes = t.bytes;
    out->data = g->map + g->data_offset + t.relative_offset;
    return WD_OK;
}

int wd_gguf_meta_number(const wd_gguf *g, const char *key, double *out) {
    WD_REQUIRE(g != nullptr && key != nullptr && out != nullptr, "wd_gguf_meta_number: null argument");
    const auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.is_array) return WD_ERR_ARG;
    const GgufValue &v = it->second;
    switch (v.type) {
        case 0: case 2: case 4: case 7: case 10: *out = static_cast<double>(v.u); return WD_OK;
        case 1: case 3: case 5: case 11: *out = static_cast<double>(v.i); return WD_OK;
        case 6: case 12: *out = v.f; return WD_OK;
        default: return WD_ERR_ARG;
    }
}

const char *wd_gguf_meta_string(const wd_gguf *g, const char *key) {
    if (!g || !key) return nullptr;
    const auto it = g->meta.find(key);
    return (it == g->meta.end() || it->second.is_array || it->second.type != 8) ? nullptr : it->second.s.c_str();
}

long long wd_gguf_meta_array(const wd_gguf *g, const char *key, uint32_t *elem_type, const void **data) {
    if (!g || !key) return -1;
    const auto it = g->meta.find(key);
    if (it == g->meta.end() || !it->second.is_array) return -1;
    if (elem_type) *elem_type = it->second.type;
    if (data) *data = it->second.raw;
    return static_cast<long long>(it->second.count);
}

}  // extern "C"
