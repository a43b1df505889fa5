// Host-side plumbing shared by the translation units of libwarpdecode_amd.so:
// error reporting and argument checks.  Not part of the public ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../include/warpdecode_amd.h"

namespace wd {

std::string &last_error_slot();
int fail(int code, const char *fmt, ...);

inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }
// wd_noalloc.hip: looks up, once per device, where that device holds the static scratch array of the layer pass that
// allocates nothing (the current device; wd_init calls it)
int noalloc_setup_current_device();

#define WD_HIP(call)                                                                         \
    do {                                                                                     \
        const hipError_t wd_e_ = (call);                                                     \
        if (wd_e_ != hipSuccess)                                                             \
            return ::wd::fail(WD_ERR_HIP, "%s failed: %s", #call, hipGetErrorString(wd_e_)); \
    } while (0)

#define WD_REQUIRE(cond, ...)                                   \
    do {                                                        \
        if (!(cond)) return ::wd::fail(WD_ERR_ARG, __VA_ARGS__); \
    } while (0)

#define WD_LAUNCH_CHECK() WD_HIP(hipGetLastError())

inline int block_elems(int type) {
    switch (type) {
        case WD_TYPE_IQ3_S:
        case WD_TYPE_IQ2_S:
        case WD_TYPE_Q6_K: return 256;
        case WD_TYPE_Q8_0:
        case WD_TYPE_Q4_0:
        case WD_TYPE_IQ4_NL: return 32;
        case WD_TYPE_F32:
        case WD_TYPE_F16: return 1;
        default: return 0;
    }
}
inline size_t block_bytes(int type) {
    switch (type) {
        case WD_TYPE_IQ3_S: return 110;
        case WD_TYPE_IQ2_S: return 82;
        case WD_TYPE_Q6_K: return 210;
        case WD_TYPE_Q8_0: return 34;
        case WD_TYPE_Q4_0:
        case WD_TYPE_IQ4_NL: return 18;
        case WD_TYPE_F32: return 4;
        case WD_TYPE_F16: return 2;
        default: return 0;
    }
}
inline size_t row_bytes(int type, int cols) {
    const int be = block_elems(type);
    if (be == 0 || cols <= 0 || cols % be != 0) return 0;
    return static_cast<size_t>(cols / be) * block_bytes(type);
}
// int32 chunk sums one row exports for the parity harness
inline int partials_per_row(int type, int cols) {
    switch (type) {
        case WD_TYPE_IQ3_S:
        case WD_TYPE_IQ2_S: return cols / 256 * 8;
        case WD_TYPE_Q8_0:
        case WD_TYPE_IQ4_NL: return cols / 32 * 8;
        case WD_TYPE_Q4_0: return cols / 32;
        default: return 0;
    }
}
inline bool consumes_q8k(int type) { return type == WD_TYPE_IQ3_S || type == WD_TYPE_IQ2_S; }
inline bool consumes_q8_0(int type) {
    return type == WD_TYPE_Q8_0 || type == WD_TYPE_IQ4_NL || type == WD_TYPE_Q4_0;
}

}  // namespace wd
