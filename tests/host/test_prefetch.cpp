// Host test of the expert prefetcher and of the planner that feeds it (warpdecode_amd/csrc/wd_prefetch.hpp), with the
// contract of the reference's own test (tests/expert_prefetch_host_test.cpp:1-30): a completed prediction hands out
// exactly the bytes an on-demand read would have put in the slot; an expert that was never requested is not handed out;
// the same expert is never read twice at once; a read that fails never serves a fill and does not wedge the prefetcher;
// shelves are reused only when that is safe; the prediction is the previous token's list of the next `depth` layers,
// asked for once per layer, without the expert being acquired.  No GPU: the shelves are plain memory and the
// "copy completed" test is a flag the test sets.
#include <fcntl.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "wd_prefetch.hpp"

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
    char path[] = "/tmp/wd_prefetch_XXXXXX";
    const int wfd = ::mkstemp(path);
    CHECK(wfd >= 0 && ::write(wfd, disk.data(), kFile) == static_cast<ssize_t>(kFile), "the test file is written");
    ::close(wfd);
    const int fd = ::open(path, O_RDONLY);
    ::unlink(path);
    CHECK(fd >= 0, "the test file opens");

    {   // ---- the prefetcher
        std::vector<std::vector<uint8_t>> mem(2, std::vector<uint8_t>(kSlot, 0));
        std::vector<uint8_t *> bufs = {mem[0].data(), mem[1].data()};
        bool copy_done[2] = {false, false};
        ExpertPrefetcher pf;
        CHECK(!pf.running(), "a prefetcher without shelves is off");
        CHECK(pf.start(bufs, [&](int s) { return copy_done[s]; }), "the prefetcher takes its shelves");
        CHECK(pf.running() && pf.shelves() == 2, "it reports its size");
        const PrefetchRun two[2] = {{kOff0, 0, kLen0}, {kOff1, kAt1, kLen1}};
        CHECK(pf.request(11, fd, two, 2), "an order is accepted");
        CHECK(!pf.request(11, fd, two, 2), "the same expert is not read twice at once");
        CHECK(wait_for([&] { return pf.delivered(); }, 1, 10000), "the reader completes the order");
        CHECK(!pf.request(11, fd, two, 2), "nor is an expert that is on a shelf");
        const int shelf = pf.claim(11);
        CHECK(shelf >= 0, "a completed prediction is handed out");
        const uint8_t *buf = shelf >= 0 ? pf.data(shelf) : nullptr;
        // what an on-demand fill reads into a slot
        std::vector<uint8_t> demand(kSlot, 0);
        CHECK(::pread(fd, demand.data(), kLen0, kOff0) == static_cast<ssize_t>(kLen0) && ::pread(fd, demand.data() + kAt1, kLen1, kOff1) == static_cast<ssize_t>(kLen1), "on-demand read");
        CHECK(buf && std::memcmp(buf, demand.data(), kSlot) == 0, "the predicted bytes are the on-demand bytes, run by run");
        CHECK(buf && std::memcmp(buf, disk.data() + kOff0, kLen0) == 0 && std::memcmp(buf + kAt1, disk.data() + kOff1, kLen1) == 0 && buf[kLen0] == 0 && buf[kAt1 - 1] == 0,
              "runs land at their offsets and the gap is untouched");
        CHECK(pf.claim(11) < 0, "a claimed shelf is not handed out twice");
        CHECK(pf.claim(12) < 0, "an expert that was never requested is not handed out");
        CHECK(pf.claimed() == 1, "the counter follows the hand-out");
        // a read past the end of the file
        const PrefetchRun bad[1] = {{kFile + 4096, 0, kLen0}};
        CHECK(pf.request(13, fd, bad, 1), "an order past EOF is accepted");
        CHECK(wait_for([&] { return pf.failed(); }, 1, 10000), "the reader reports the failure");
        CHECK(pf.claim(13) < 0, "a failed read never serves a fill");
        // reuse: the claimed shelf may not be taken before its copy is queued and done; the failed one is free at once
        CHECK(pf.request(14, fd, two, 2), "the shelf of the failed read takes the next order");
        CHECK(wait_for([&] { return pf.delivered(); }, 2, 10000), "the prefetcher is not wedged by a failure");
        CHECK(pf.request(15, fd, two, 2) && pf.unused() == 1, "a shelved prediction nobody claimed is the next to go");
        CHECK(wait_for([&] { return pf.delivered(); }, 3, 10000), "and its shelf is read again");
        CHECK(pf.claim(14) < 0, "the overwritten prediction is gone");
        const int s15 = pf.claim(15);
        CHECK(s15 >= 0 && s15 != shelf, "the new one is served from the other shelf");
        CHECK(!pf.request(16, fd, two, 2) && pf.dropped() == 1, "two claimed shelves: nothing to reuse, the order is dropped");
        pf.copy_queued(shelf);
        CHECK(!pf.request(16, fd, two, 2) && pf.dropped() == 2, "a shelf whose copy has not completed is not reused");
        copy_done[shelf] = true;
        CHECK(pf.request(16, fd, two, 2), "after the copy it is");
        CHECK(wait_for([&] { return pf.delivered(); }, 4, 10000) && !pf.busy(), "the last order completes");
        const int s16 = pf.claim(16);
        CHECK(s16 == shelf && std::memcmp(pf.data(s16), demand.data(), kSlot) == 0, "the reused shelf holds the new expert's bytes");
        CHECK(pf.requested() == 5, "requested counts accepted orders (%llu)", static_cast<unsigned long long>(pf.requested()));
        // many orders against a slow consumer: every accepted order ends as delivered, nothing is lost or doubled
        pf.copy_queued(s15), pf.copy_queued(s16);
        copy_done[0] = copy_done[1] = true;
        uint64_t accepted = 0;
        for (uint64_t k = 100; k < 140; ++k) accepted += pf.request(k, fd, two, 2) ? 1 : 0;
        CHECK(accepted >= 2, "orders are accepted while shelves can be reused (%llu)", static_cast<unsigned long long>(accepted));
        CHECK(wait_for([&] { return pf.delivered(); }, 4 + accepted, 10000) && !pf.busy() && pf.delivered() == 4 + accepted,
              "every accepted order is delivered exactly once");
        pf.stop();
        CHECK(!pf.running(), "stop() drops the shelves");
    }
    {   // ---- the planner
        PrefetchPlanner h;
        CHECK(h.on_acquire(0, key_of(0, 1)).empty(), "depth 0: no prediction");
        h.set_depth(1);
        // token 1: layer 0 takes experts 1 2 3, layer 1 takes 5 6
        for (int e : {1, 2, 3}) CHECK(h.on_acquire(0, key_of(0, e)).empty(), "the first token has no history to predict from");
        for (int e : {5, 6}) CHECK(h.on_acquire(1, key_of(1, e)).empty(), "still the first token");
        // token 2, layer 0, first acquire (expert 9)
        std::vector<uint64_t> c = h.on_acquire(0, key_of(0, 9));
        CHECK(c.size() == 3 && has(c, key_of(0, 1)) && has(c, key_of(0, 2)) && has(c, key_of(0, 3)), "the prediction is the previous token's list of this layer");
        CHECK(!has(c, key_of(0, 9)), "the expert being acquired is never a candidate");
        CHECK(!has(c, key_of(1, 5)), "a depth of 1 does not read into the next layer");
        CHECK(h.on_acquire(0, key_of(0, 2)).empty(), "the prediction is evaluated once per layer");
        c = h.on_acquire(1, key_of(1, 5));
        CHECK(c.size() == 1 && c[0] == key_of(1, 6), "layer 1: its own list without the expert being acquired");
        // token 3 with depth 2: layer 0's first acquire reaches into layer 1 of token 2
        h.set_depth(2);
        c = h.on_acquire(0, key_of(0, 4));
        CHECK(c.size() == 3 && has(c, key_of(0, 9)) && has(c, key_of(0, 2)) && has(c, key_of(1, 5)), "depth 2 covers this layer and the next (token 2 took 9 2 | 5)");
    }
    ::close(fd);
    std::printf("%d checks, %d failures\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
