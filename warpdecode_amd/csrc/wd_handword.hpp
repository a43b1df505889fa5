// The bits a 32-bit value travels with between the workgroups of a resident launch (wd_resident.cuh).  A hand-off word
// that still holds kHandEmpty has not been written; consumers poll the data words themselves.  kHandEmpty is also the
// bit pattern of one particular NaN, which a producer may legitimately compute: it is handed on as the default quiet NaN
// instead, so that its consumer does not wait for it for ever.  Plain C++: the host tests include this file too.
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#define WD_HAND_FN __host__ __device__ inline
#else
#define WD_HAND_FN inline
#endif

namespace wd {

constexpr uint32_t kHandEmpty = 0xffffffffu;
constexpr uint32_t kHandQuietNan = 0x7fc00000u;

WD_HAND_FN uint32_t hand_word_bits(uint32_t bits) { return bits == kHandEmpty ? kHandQuietNan : bits; }
WD_HAND_FN bool hand_arrived(uint32_t word) { return word != kHandEmpty; }

}  // namespace wd
