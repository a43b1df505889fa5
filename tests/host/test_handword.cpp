// Host check of the hand-off word helper of the resident launch (csrc/wd_handword.hpp): the one bit pattern that means
// "not yet written" never leaves a producer, and nothing else is changed.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <initializer_list>

#include "wd_handword.hpp"

static int failures = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                    \
        }                                                                  \
    } while (0)

static float as_float(uint32_t b) {
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

int main() {
    using namespace wd;
    // the pattern itself: a NaN goes in, the default quiet NaN comes out
    CHECK(std::isnan(as_float(kHandEmpty)));
    CHECK(hand_word_bits(kHandEmpty) == kHandQuietNan);
    CHECK(std::isnan(as_float(hand_word_bits(kHandEmpty))));
    CHECK(!hand_arrived(kHandEmpty) && hand_arrived(kHandQuietNan) && hand_arrived(0u));
    // every NaN there is (both signs, all 2^23 - 1 payloads each): unchanged except the one, and never "not yet written"
    unsigned long long nans = 0, changed = 0;
    for (uint32_t sign = 0; sign < 2; ++sign)
        for (uint32_t payload = 1; payload < (1u << 23); ++payload) {
            const uint32_t b = (sign << 31) | 0x7f800000u | payload;
            const uint32_t w = hand_word_bits(b);
            ++nans;
            if (w != b) ++changed;
            if (!hand_arrived(w) || !std::isnan(as_float(w))) ++failures;
        }
    CHECK(nans == 2ull * ((1u << 23) - 1) && changed == 1);
    // everything else, in steps that reach every exponent and both signs: unchanged bit for bit
    unsigned long long others = 0;
    for (uint64_t b = 0; b < (1ull << 32); b += 4099) {
        const uint32_t v = static_cast<uint32_t>(b);
        if (v == kHandEmpty) continue;
        ++others;
        if (hand_word_bits(v) != v || !hand_arrived(hand_word_bits(v))) ++failures;
    }
    for (uint32_t v : {0u, 0x80000000u, 0x7f800000u, 0xff800000u, 0x7fffffffu, 0xfffffffeu, 0x00000001u, 0x3f800000u})
        CHECK(hand_word_bits(v) == v && hand_arrived(v));
    std::printf("%llu NaN patterns and %llu other patterns checked, %d failures\n", nans, others, failures);
    return failures ? 1 : 0;
}
