// Host test of the expert read-ahead ring and of the history that feeds it (warpdecode_amd/csrc/wd_readahead.hpp),
// with the contract of the reference's own test (tests/expert_prefetch_host_test.cpp:1-30): a completed prediction
// hands out exactly the bytes an on-demand read would have put in the slot; a key that was never posted is not handed
// out; the same key is never queued twice; a read that fails never serves a fill and does not wedge the ring; entries
// are recycled only when that is safe; the prediction is the previous token's list of the next `depth` layers, asked
// for once per layer, without the expert being acquired.  No GPU: the ring's buffers are plain memory and the
// "DMA completed" test is a flag the test sets.
#include <fcntl.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "wd_readahead.hpp"

using namespace wd;

static int g_checks = 0, g_fail = 0;
#define CHECK(cond, ...)                                  \
    do {                                                  \
        ++g_checks;                                       \
        if (!(cond)) {                                    \
            ++g_fail;                                     \
            std::fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); \
            std::fprintf(stderr, __VA_ARGS__);            \
            std::fprintf(stderr, "\n");                   \
        }                                                 \
    } while (0)

template <typename F>
static bool wait_for(F value, uint64_t want, int ms) {
    for (int i = 0; i < ms * 10; ++i) {
        if (value() >= want) return true;
        ::usleep(100);
    }
    return value() >= want;
}
static uint64_t key_of(int layer, int expert) { return (static_cast<uint64_t>(static_cast<uint32_t>(layer)) << 32) | static_cast<uint32_t>(expert); }
static bool has(const std::vector<uint64_t> &v, uint64_t k) { return std::find(v.begin(), v.end(), k) != v.end(); }

int main() {
    // a "model file" of 4 MiB of known bytes; a slot is two slices with a gap between them, like gate | up | down
    constexpr size_t kFile = 4u << 20, kOff0 = 1u << 20, kOff1 = 3u << 20, kLen0 = 8192, kLen1 = 8192, kAt1 = 12288, kSlot = kAt1 + kLen1;
    std::vector<uint8_t> disk(kFile);
    uint32_t s = 12345u;
    for (auto &b : disk) s = s * 1664525u + 1013904223u, b = static_cast<uint8_t>(s >> 24);
    char path[] = "/tmp/wd_readahead_XXXXXX";
    const int wfd = ::mkstemp(path);
    CHECK(wfd >= 0 && ::write(wfd, disk.data(), kFile) == static_cast<ssize_t>(kFile), "the test file is written");
    ::close(wfd);
    const int fd = ::open(path, O_RDONLY);
    ::unlink(path);
    CHECK(fd >= 0, "the test file opens");

    {   // ---- the ring
        std::vector<std::vector<uint8_t>> mem(2, std::vector<uint8_t>(kSlot, 0));
        std::vector<uint8_t *> bufs = {mem[0].data(), mem[1].data()};
        bool dma_done[2] = {false, false};
        ReadAheadRing ring;
        CHECK(!ring.enabled(), "a ring without buffers is off");
        CHECK(ring.configure(bufs, [&](int e) { return dma_done[e]; }), "the ring takes its buffers");
        CHECK(ring.enabled() && ring.slots() == 2, "the ring reports its size");
        const uint64_t off[2] = {kOff0, kOff1};
        const size_t at[2] = {0, kAt1}, len[2] = {kLen0, kLen1};
        CHECK(ring.post(11, fd, off, at, len, 2), "a job is published");
        CHECK(!ring.post(11, fd, off, at, len, 2), "the same key is not queued twice");
        CHECK(wait_for([&] { return ring.delivered(); }, 1, 10000), "the reader completes the job");
        CHECK(!ring.post(11, fd, off, at, len, 2), "nor is a key that is ready");
        int entry = -1;
        uint8_t *buf = ring.borrow(11, &entry);
        CHECK(buf != nullptr && entry >= 0, "a completed entry is handed out");
        // what an on-demand fill reads into a slot
        std::vector<uint8_t> demand(kSlot, 0);
        CHECK(::pread(fd, demand.data(), kLen0, kOff0) == static_cast<ssize_t>(kLen0) && ::pread(fd, demand.data() + kAt1, kLen1, kOff1) == static_cast<ssize_t>(kLen1), "on-demand read");
        CHECK(buf && std::memcmp(buf, demand.data(), kSlot) == 0, "the predicted bytes are the on-demand bytes, slice by slice");
        CHECK(buf && std::memcmp(buf, disk.data() + kOff0, kLen0) == 0 && std::memcmp(buf + kAt1, disk.data() + kOff1, kLen1) == 0 && buf[kLen0] == 0 && buf[kAt1 - 1] == 0,
              "slices land at their offsets and the gap is untouched");
        CHECK(ring.borrow(11, nullptr) == nullptr, "a borrowed entry is not handed out twice");
        CHECK(ring.borrow(12, nullptr) == nullptr, "a key that was never queued is not handed out");
        CHECK(ring.used() == 1, "the used counter follows the hand-out");
        CHECK(ring.state_of(entry) == ReadAheadRing::kBorrowed, "the entry is borrowed until its DMA is queued");
        // a read past the end of the file
        const uint64_t bad[1] = {kFile + 4096};
        CHECK(ring.post(13, fd, bad, at, len, 1), "a job past EOF is published");
        CHECK(wait_for([&] { return ring.failed(); }, 1, 10000), "the reader reports the failure");
        CHECK(ring.borrow(13, nullptr) == nullptr, "a failed read never serves a fill");
        // recycling: the borrowed entry may not be reused before its DMA is queued and done; the failed one may
        CHECK(ring.post(14, fd, off, at, len, 2), "the failed entry is recycled for the next job");
        CHECK(wait_for([&] { return ring.delivered(); }, 2, 10000), "the ring is not wedged by a failure");
        CHECK(ring.post(15, fd, off, at, len, 2), "a ready prediction nobody used is the next to go");
        CHECK(wait_for([&] { return ring.delivered(); }, 3, 10000), "and is read again");
        CHECK(ring.borrow(14, nullptr) == nullptr, "the recycled prediction is gone");
        int e15 = -1;
        CHECK(ring.borrow(15, &e15) != nullptr && e15 != entry, "the new one is served from the other entry");
        CHECK(!ring.post(16, fd, off, at, len, 2) && ring.dropped() == 1, "two borrowed entries: nothing to recycle, the job is dropped");
        ring.finish_borrow(11);
        CHECK(ring.state_of(entry) == ReadAheadRing::kInFlight, "finish_borrow marks the DMA as queued");
        CHECK(!ring.post(16, fd, off, at, len, 2), "an entry whose DMA has not completed is not recycled");
        dma_done[entry] = true;
        CHECK(ring.post(16, fd, off, at, len, 2), "after the DMA it is");
        CHECK(wait_for([&] { return ring.delivered(); }, 4, 10000) && !ring.busy(), "the last job completes");
        CHECK(ring.posted() == 5, "posted counts accepted jobs (%llu)", static_cast<unsigned long long>(ring.posted()));
        ring.release();
        CHECK(!ring.enabled(), "release() drops the ring");
    }
    {   // ---- the history
        ReadAheadHistory h;
        CHECK(h.note_access(0, key_of(0, 1)).empty(), "depth 0: no prediction");
        h.set_depth(1);
        // token 1: layer 0 takes experts 1 2 3, layer 1 takes 5 6
        for (int e : {1, 2, 3}) CHECK(h.note_access(0, key_of(0, e)).empty(), "the first token has no history to predict from");
        for (int e : {5, 6}) CHECK(h.note_access(1, key_of(1, e)).empty(), "still the first token");
        // token 2, layer 0, first acquire (expert 9)
        std::vector<uint64_t> c = h.note_access(0, key_of(0, 9));
        CHECK(c.size() == 3 && has(c, key_of(0, 1)) && has(c, key_of(0, 2)) && has(c, key_of(0, 3)), "the prediction is the previous token's list of this layer");
        CHECK(!has(c, key_of(0, 9)), "the expert being acquired is never a candidate");
        CHECK(!has(c, key_of(1, 5)), "a depth of 1 does not read into the next layer");
        CHECK(h.note_access(0, key_of(0, 2)).empty(), "the prediction is evaluated once per layer");
        c = h.note_access(1, key_of(1, 5));
        CHECK(c.size() == 1 && c[0] == key_of(1, 6), "layer 1: its own list without the expert being acquired");
        // token 3 with depth 2: layer 0's first acquire reaches into layer 1 of token 2
        h.set_depth(2);
        c = h.note_access(0, key_of(0, 4));
        CHECK(c.size() == 3 && has(c, key_of(0, 9)) && has(c, key_of(0, 2)) && has(c, key_of(1, 5)), "depth 2 covers this layer and the next (token 2 took 9 2 | 5)");
    }
    ::close(fd);
    std::printf("%d checks, %d failures\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
