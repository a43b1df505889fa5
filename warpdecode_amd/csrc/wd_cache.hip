// Expert-slot cache: an LRU pool of fixed-size slots in HBM fed from pinned host memory.
//
// Semantics follow the reference cache (src/expert_cache.cuh:2156-2536): key (layer << 32 | expert),
// a hit refreshes last_use, a miss takes the lowest-numbered empty slot or else the slot with the
// smallest last_use (inside the layer's partition when partitioning is on), the old key is dropped,
// the slot is filled with gate | up | down at fixed offsets.  What differs is the machinery:
//   * victim choice is O(1) (an intrusive list ordered by last_use and an ordered free list give
//     the same victim as the reference's linear scan);
//   * the kernels never see host pointers: every layer has a device table expert -> slot that the
//     grouped GEMVs index with the routed ids, updated by a small kernel ordered on the caller's
//     stream, so no pointer table is uploaded per layer;
//   * fills run on a private copy stream: the copy stream waits for the work already queued on the caller's
//     stream (which may still read the victim slot) and the caller's stream waits for the fills, so no host
//     thread ever blocks.  When a layer's host tensors are pinned (the GPU can read them) and 16-byte aligned,
//     all misses of an acquire call are filled by ONE copy kernel that reads host memory directly (three
//     segments per miss, many workgroups per segment): a miss is three sub-megabyte pieces, and per-copy set-up
//     of the DMA path, not the link, was what bounded the fill rate.  Otherwise (pageable memory such as a file
//     mapping, odd alignment) the three pieces go through hipMemcpyAsync;
//   * a file mapping attached to the cache (wd_expert_cache_attach_file) turns fills from pointers inside it into
//     pread() of the expert's three slices into one entry of a pinned ring, shared out over a few worker threads
//     (a single core does not reach the page cache's bandwidth), followed by ONE DMA of the whole slot from the
//     ring entry; an entry is reused when the event recorded behind its DMA has completed.  Same role as the
//     reference's ExpertFileMap / ExpertPreadPool / pinned ring (src/expert_cache.cuh:204-508, :858-1583); the file
//     is named by the caller or found through /proc/self/maps (wd_expert_cache_attach_mappings).
#include "wd_common.h"
#include "wd_profile.hpp"
#include "wd_prefetch.hpp"

#include <fcntl.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstring>
#include <functional>
#include <list>
#include <mutex>
#include <new>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

using namespace wd;

namespace {

struct SlotUpdate {
    int32_t index;  // position in the concatenated [layer][expert] table
    int32_t value;  // slot number or -1
};

// Copy kernel of the fill path: segment blockIdx.y is copied by gridDim.x workgroups in 16-byte words.
constexpr int kMaxFillSegments = 3 * (64 / 2);  // three per miss, at most kMaxUpdates / 2 misses per call
struct FillSegments {
    const uint8_t *src[kMaxFillSegments];  // pinned host memory, read over the host link
    uint8_t *dst[kMaxFillSegments];
    uint32_t words[kMaxFillSegments];      // 16-byte words
};
#ifndef WD_FILL_WGS
#define WD_FILL_WGS 20     // workgroups of a fill launch, whatever the number of segments
#endif
#ifndef WD_FILL_UNROLL
#define WD_FILL_UNROLL 8   // 16-byte words a thread moves per round, all requested before the first is stored
#endif
// A few one-wave workgroups walk all the segments together.  The link, not the number of workgroups, bounds the rate
// (160 KB in flight keep it at 50 GB/s and more), and every workgroup lives as long as the launch, so what matters is
// how little the launch disturbs the layer kernels that run beside it.  Measured on the mode B workload (tokens per
// second at a hit rate of 0.93): one workgroup of 256 threads per piece of every segment 400 (hundreds of workgroups
// that each wait on the link for most of a millisecond: the layer kernels could not place theirs); 8 x 256 threads for
// the whole launch 570 (k_layer_ab 22.6 instead of 16 us: the compute units that host a fill workgroup serve their
// layer workgroups late, and the grid waits for those); 32 x 64 threads 589, 24 x 64 642, 20 x 64 670, 16 x 64 582
// (the link is no longer kept busy).  The loop below keeps a round's words in a private array that the compiler
// places in scratch memory (the stores are conditional): the words go link -> registers -> scratch -> registers ->
// slot, one store at a time.  Forms that keep them in registers (unconditional stores of a plain vector type; 20 x 64
// x 8, 20 x 64 x 4, 40 x 64 x 4, 40 x 64 x 2, 64 x 64 x 2) all measured 530..590 against 669 on the same box: a copy
// that runs through its stores faster takes more from the layer kernels than it gains on the link.
#ifndef WD_FILL_THREADS
#define WD_FILL_THREADS 64
#endif
// What a fill launch tells a one-launch stack that runs beside it (wd_resident.cuh, fill_need / fill_done): when the
// launch's last workgroup is through, done[l] = seq for every layer l in `layers` (bit l).
struct FillMarks {
    uint32_t *done;               // null: nothing to tell
    unsigned *arrivals;           // workgroups of this launch that are through (back to 0 when the last one is)
    unsigned long long layers;
    uint32_t seq;
};
// When the launch's last workgroup is through: the layers are counted off.
WD_DEV void fill_marks(const FillMarks &m) {
    if (!m.done) return;
    __threadfence();  // the stores of the copy are where every compute unit of the device reads them
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned last = gridDim.x - 1;
        if (atomicInc(m.arrivals, last) == last) {  // (wraps to 0 for the next launch)
            __threadfence();
            for (unsigned long long rest = m.layers; rest; rest &= rest - 1)
                __hip_atomic_store(m.done + (__ffsll(rest) - 1), m.seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}
__global__ __launch_bounds__(WD_FILL_THREADS) void k_fill_slots(FillSegments f, int n_seg) {
    const uint32_t stride = gridDim.x * WD_FILL_THREADS;
    for (int seg = 0; seg < n_seg; ++seg) {
        const uint4 *src = reinterpret_cast<const uint4 *>(f.src[seg]);
        uint4 *dst = reinterpret_cast<uint4 *>(f.dst[seg]);
        const uint32_t n = f.words[seg];
        // every round: WD_FILL_UNROLL requests per thread in flight (lanes past the end repeat the last word and store nothing)
        for (uint32_t base = blockIdx.x * WD_FILL_THREADS + threadIdx.x; base < n; base += WD_FILL_UNROLL * stride) {
            uint4 v[WD_FILL_UNROLL];
#pragma unroll
            for (int u = 0; u < WD_FILL_UNROLL; ++u) {
                const uint32_t i = base + u * stride;
                v[u] = src[i < n ? i : n - 1];
            }
#pragma unroll
            for (int u = 0; u < WD_FILL_UNROLL; ++u) {
                const uint32_t i = base + u * stride;
                if (i < n) dst[i] = v[u];
            }
        }
    }
}
// The same copy for a launch that has to find room beside a one-launch stack, whose workgroups stay on every compute unit
// until the stack is through: a workgroup of this kernel takes no LDS, no scratch memory and few registers (a round's
// three words in named registers, every store unconditional: no private array).  Beside the stack's six waves a SIMD has
// 32 vector registers left, and of the scalar registers what the stack kernel's own cap leaves (see k_stack_resident):
// a kernel that needs more of either is not started before the stack has ended, which the stack, waiting for it, never does.
// 54 workgroups: as many bytes in flight as the 20 of the other form have.  Mode B, tokens per second: 32 workgroups 706,
// 54 743, 96 656, 160 561 (the more waves sit beside the stack's, the later its slowest workgroup).
constexpr int kFillBesideWgs = 54, kFillBesideUnroll = 3;
__global__ __launch_bounds__(WD_FILL_THREADS) void k_fill_slots_beside(FillSegments f, int n_seg, FillMarks m) {
    const uint32_t stride = gridDim.x * WD_FILL_THREADS;
    for (int seg = 0; seg < n_seg; ++seg) {
        const uint4 *src = reinterpret_cast<const uint4 *>(f.src[seg]);
        uint4 *dst = reinterpret_cast<uint4 *>(f.dst[seg]);
        const uint32_t n = f.words[seg];
        uint32_t base = blockIdx.x * WD_FILL_THREADS + threadIdx.x;
        for (; base + 2 * stride < n; base += 3 * stride) {
            const uint4 a = src[base], b = src[base + stride], c = src[base + 2 * stride];
            dst[base] = a, dst[base + stride] = b, dst[base + 2 * stride] = c;
        }
        for (; base < n; base += stride) dst[base] = src[base];
    }
    fill_marks(m);
}

// One thread, in order: a batch may name the same table entry twice (evicted, then filled again).
__global__ void k_apply_slot_updates(int32_t *table, const SlotUpdate *updates, int n) {
    if (blockIdx.x == 0 && threadIdx.x == 0)
        for (int i = 0; i < n; ++i) table[updates[i].index] = updates[i].value;
}

__global__ void k_fill_i32(int32_t *dst, int32_t v, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = v;
}

struct Slot {
    uint64_t key = 0;
    uint64_t last_use = 0;
    bool valid = false;
    std::list<size_t>::iterator lru;  // position in its partition's list (valid slots only)
};

struct Partition {
    size_t begin = 0, end = 0;
    std::list<size_t> lru;       // front = least recently used
    std::vector<size_t> free;    // empty slots, descending so that back() is the lowest index
};

// Counterfactual caches fed with the same (layer, expert) access trace as the real pool; they hold keys only
// and never touch device memory (reference: ShadowLru / ShadowFreq, src/expert_cache.cuh:1592-1668).
struct Shadow {
    int policy = 0;  // 0 = LRU, 1 = LFU with the least recently inserted among the least frequent leaving
    size_t capacity = 1;
    uint64_t hits = 0, accesses = 0;
    std::list<uint64_t> order;  // LRU: front = most recent
    std::unordered_map<uint64_t, std::list<uint64_t>::iterator> where;
    struct Entry {
        uint64_t key, freq;
    };
    std::vector<Entry> entries;                    // LFU residents
    std::unordered_map<uint64_t, size_t> resident; // LFU: key -> entry
    std::unordered_map<uint64_t, uint64_t> seen;   // LFU: lifetime count of every key

    void access(uint64_t key) {
        ++accesses;
        if (policy == 0) {
            auto it = where.find(key);
            if (it != where.end()) {
                ++hits;
                order.splice(order.begin(), order, it->second);
                return;
            }
            order.push_front(key);
            where[key] = order.begin();
            if (order.size() > capacity) {
                where.erase(order.back());
                order.pop_back();
            }
            return;
        }
        const uint64_t n = ++seen[key];
        auto it = resident.find(key);
        if (it != resident.end()) {
            ++entries[it->second].freq;
            ++hits;
            return;
        }
        if (entries.size() < capacity) {
            resident[key] = entries.size();
            entries.push_back({key, n});
            return;
        }
        size_t victim = 0;
        for (size_t i = 1; i < entries.size(); ++i)
            if (entries[i].freq < entries[victim].freq) victim = i;
        resident.erase(entries[victim].key);
        entries[victim] = {key, n};
        resident[key] = victim;
    }
};

constexpr int kUpdateRing = 32;
constexpr int kMaxUpdates = 64;  // 2 per missed expert, k <= 16... one acquire call never needs more

}  // namespace

namespace {

// Fork-join pool for pread(): the caller publishes a list of (fd, offset, length, destination) pieces, takes its
// share and returns when every piece has landed.  threads == 1 keeps everything inline.
struct PreadPiece {
    int fd;
    uint64_t off;
    size_t len;
    uint8_t *dst;
};
class PreadPool {
public:
    explicit PreadPool(int threads) {
        for (int i = 1; i < threads; ++i) workers_.emplace_back([this] { loop(); });
    }
    ~PreadPool() {
        {
            std::lock_guard<std::mutex> g(m_);
            stop_ = true;
        }
        cv_.notify_all();
        for (std::thread &t : workers_) t.join();
    }
    // false when a read came up short or failed
    bool run(const PreadPiece *pieces, int n) {
        {
            std::lock_guard<std::mutex> g(m_);
            pieces_ = pieces, n_ = n, next_ = 0, pending_ = n, failed_ = false;
            ++generation_;
        }
        cv_.notify_all();
        work();
        std::unique_lock<std::mutex> g(m_);
        done_.wait(g, [this] { return pending_ == 0; });
        pieces_ = nullptr, n_ = 0;
        return !failed_;
    }

private:
    static bool read_all(const PreadPiece &p) {
        size_t got = 0;
        while (got < p.len) {
            const ssize_t r = ::pread(p.fd, p.dst + got, p.len - got, static_cast<off_t>(p.off + got));
            if (r <= 0) return false;
            got += static_cast<size_t>(r);
        }
        return true;
    }
    void work() {
        for (;;) {
            PreadPiece p;
            {
                std::lock_guard<std::mutex> g(m_);
                if (next_ >= n_) return;
                p = pieces_[next_++];
            }
            const bool ok = read_all(p);
            std::lock_guard<std::mutex> g(m_);
            if (!ok) failed_ = true;
            if (--pending_ == 0) done_.notify_all();
        }
    }
    void loop() {
        uint64_t seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> g(m_);
                cv_.wait(g, [&] { return stop_ || generation_ != seen; });
                if (stop_) return;
                seen = generation_;
            }
            work();
        }
    }
    std::vector<std::thread> workers_;
    std::mutex m_;
    std::condition_variable cv_, done_;
    const PreadPiece *pieces_ = nullptr;
    int n_ = 0, next_ = 0, pending_ = 0;
    uint64_t generation_ = 0;
    bool stop_ = false, failed_ = false;
};

struct FileSource {
    const uint8_t *base = nullptr;  // start of the caller's read-only mapping of the file
    size_t size = 0;
    int fd = -1;                    // our own descriptor of the same file
    uint64_t file_off = 0;          // offset in the file of the byte at `base`
};

// The file mapping that holds `ptr`, from /proc/self/maps ("start-end perms offset dev inode path"); consecutive lines
// of one file whose addresses and offsets continue each other count as one mapping.  Same role as the reference's
// ExpertFileMap (src/expert_cache.cuh:204-330).
bool find_file_mapping(const void *ptr, wd_file_mapping *out) {
    FILE *maps = std::fopen("/proc/self/maps", "r");
    if (!maps) return false;
    const uint64_t want = reinterpret_cast<uintptr_t>(ptr);
    char line[4352];
    uint64_t run_start = 0, run_end = 0, run_off = 0;
    std::string run_path;
    bool found = false;
    auto flush = [&]() {
        if (!run_path.empty() && want >= run_start && want < run_end) {
            out->start = run_start, out->end = run_end, out->file_offset = run_off;
            std::snprintf(out->path, sizeof(out->path), "%s", run_path.c_str());
            found = run_path.size() < sizeof(out->path);
        }
    };
    while (!found && std::fgets(line, sizeof(line), maps)) {
        unsigned long long a = 0, b = 0, off = 0, inode = 0;
        char perms[8] = {0}, dev[16] = {0};
        int at = 0;
        if (std::sscanf(line, "%llx-%llx %7s %llx %15s %llu %n", &a, &b, perms, &off, dev, &inode, &at) < 6) continue;
        std::string path(line + at);
        while (!path.empty() && (path.back() == '\n' || path.back() == ' ')) path.pop_back();
        const bool file = inode != 0 && !path.empty() && path[0] == '/' && perms[0] == 'r';
        if (file && path == run_path && a == run_end && off == run_off + (run_end - run_start)) {
            run_end = b;  // the same file goes on
            continue;
        }
        flush();
        if (file)
            run_start = a, run_end = b, run_off = off, run_path = path;
        else
            run_path.clear();
    }
    if (!found) flush();
    std::fclose(maps);
    return found;
}

constexpr int kStageRing = 16;  // pinned ring entries of one slot each
constexpr int kTimingSlots = 32;
struct TimingSlot {
    hipEvent_t wait_a = nullptr, wait_b = nullptr, begin = nullptr, end = nullptr;  // all recorded on the copy stream
    bool used = false, has_wait = false, has_dma = false;
};
constexpr int kRowsRing = 4, kRowsLayers = 64, kRowsK = 16, kRowsEntry = kRowsLayers * (kRowsK + 1);

}  // namespace

struct wd_expert_cache {
    uint8_t *pool = nullptr;
    size_t n_slots = 0, slot_bytes = 0, gate_bytes = 0, up_bytes = 0, down_bytes = 0;
    int n_layers = 0, n_experts = 0;
    bool partitioned = false;
    std::vector<Slot> slots;
    std::vector<Partition> parts;
    std::unordered_map<uint64_t, size_t> index;
    uint64_t clock = 0;
    uint64_t prev_floor = 0;     // clock value before the previous acquire call
    bool fills_pending = false;  // a deferred acquire's fills have not been waited for yet
    std::vector<hipEvent_t> ev_layer;      // token-ahead acquires: the fills of layer l are complete
    std::vector<int> layer_event;          //   ... when ev_layer[layer_event[l]] has passed (fills are launched by groups of layers)
    int last_waited = -1;                  // the event the caller's stream was last made to wait for in this token
    // read-ahead of predicted experts from the model file (wd_prefetch.hpp); the reader thread touches ra_mem only
    wd::ExpertPrefetcher ra;
    wd::PrefetchPlanner ra_plan;
    uint8_t *ra_mem = nullptr;             // pinned, one slot per shelf
    std::vector<hipEvent_t> ra_done;       // per shelf: the DMA that last read it
    uint64_t ra_fills = 0, ra_candidates = 0, ra_resident_skips = 0;
    hipEvent_t ev_token[2] = {nullptr, nullptr};  // recorded on the caller's stream when a token-ahead acquire begins, alternately
    int token_parity = 0;
    bool have_prev_token = false;
    uint64_t prev_token_floor = 0;         // the clock when the previous token-ahead acquire began
    std::vector<uint8_t> layer_pending;    // ev_layer[l] has been recorded and not yet waited for
    std::vector<const uint8_t *> h_gate, h_up, h_down;
    std::vector<size_t> s_gate, s_up, s_down;  // bytes from one expert to the next in the host tensors
    std::vector<uint8_t> gpu_readable;          // per layer: pinned and 16-byte aligned, the copy kernel can read it
    bool use_copy_kernel = true;
    uint64_t kernel_fills = 0, dma_fills = 0;   // misses filled by the copy kernel / by hipMemcpyAsync
    std::vector<FileSource> files;              // attached mappings: fills from pointers inside them go through pread
    std::vector<int8_t> layer_file;             // per layer: index into files, or -1
    uint8_t *stage = nullptr;                   // pinned ring [kStageRing][slot_bytes]
    hipEvent_t stage_done[kStageRing] = {};
    bool stage_used[kStageRing] = {};
    int stage_next = 0;
    PreadPool *pread_pool = nullptr;
    uint64_t pread_fills = 0;
    double pread_ms = 0.0;
    int32_t *d_table = nullptr;  // [n_layers][n_experts]
    hipStream_t copy_stream = nullptr;
    hipEvent_t ev_retire = nullptr, ev_done = nullptr;
    SlotUpdate *h_updates = nullptr;  // pinned ring [kUpdateRing][kMaxUpdates]
    SlotUpdate *d_updates = nullptr;  // device ring of the same shape
    hipEvent_t ring_free[kUpdateRing] = {};
    bool ring_used[kUpdateRing] = {};
    int ring_next = 0;
    // One-launch stacks (wd_moe_stack_cached_f32): per token, the slot of every expert of the routing trace and per layer
    // the number its fills carry, uploaded ahead of the launch; the fills count layers off in d_fill_done.
    int32_t *h_rows = nullptr, *d_rows = nullptr;   // pinned / device ring [kRowsRing][kRowsLayers * (kRowsK + 1)]
    hipEvent_t rows_free[kRowsRing] = {};
    bool rows_used[kRowsRing] = {};
    int rows_next = 0;
    uint32_t *d_fill_done = nullptr;                // device [kRowsLayers] numbers, then the fill launches' arrival counter
    uint32_t fill_seq = 0;                          // the number of the last token whose fills count layers off
    uint32_t mark_seq = 0;                          // not 0: the token-ahead acquire in progress counts layers off with it
    std::vector<uint32_t> layer_need;               // per layer: the number to wait for in this token, 0 = nothing on its way
    uint64_t resident_tokens = 0;                   // tokens that went through the one-launch stack
    // Timings of the monitor (reference: src/expert_cache.cuh:1395-1416, 1833-1847).  Device side, only when switched on
    // (wd_expert_cache_set_timing): per acquire with misses (per group of layers in a token-ahead acquire), how long the
    // copy stream waited for the slots' last readers and how long the fills then took.  Host side, always: the time between
    // two acquire calls, by whether the layer changed.
    TimingSlot timing[kTimingSlots];
    bool timing_on = false;
    int timing_next = 0, timing_cur = -1;           // timing_cur: the slot of the fills being queued, -1 none
    double dma_ms = 0.0, dma_max_ms = 0.0, stall_ms = 0.0, stall_max_ms = 0.0;
    uint64_t dma_calls = 0, stall_calls = 0, timing_skipped = 0;
    std::chrono::steady_clock::time_point last_acquire_exit{};
    int last_gap_layer = -1;
    double intra_gap_ms = 0.0, layer_gap_ms = 0.0;
    uint64_t tokens_seen = 0;
    wd_expert_cache_stats stats{};
    // monitor (reference: ExpertCacheMonitor, src/expert_cache.cuh:1670-2105)
    std::vector<Shadow> shadows;
    std::vector<uint64_t> layer_access, layer_misses;
    std::unordered_set<uint64_t> distinct;
    std::vector<std::vector<int32_t>> prev_ids;   // per layer: the ids of the previous acquire call
    uint64_t prev_ready = 0, prev_hit = 0, acquire_calls = 0;
    double acquire_ms = 0.0;
};

namespace {
// Can the copy kernel read this layer's host tensors?  They must be pinned (known to the runtime as host memory) and
// every expert slice must start and end on 16-byte boundaries.
void classify_layer(wd_expert_cache *c, int layer) {
    if (c->gpu_readable.size() < static_cast<size_t>(c->n_layers)) c->gpu_readable.assign(c->n_layers, 0);
    bool ok = c->gate_bytes % 16 == 0 && c->up_bytes % 16 == 0 && c->down_bytes % 16 == 0 && c->slot_bytes % 16 == 0 &&
              c->s_gate[layer] % 16 == 0 && c->s_up[layer] % 16 == 0 && c->s_down[layer] % 16 == 0;
    const uint8_t *ptrs[3] = {c->h_gate[layer], c->h_up[layer], c->h_down[layer]};
    for (const uint8_t *p : ptrs) {
        if (!ok) break;
        hipPointerAttribute_t attr{};
        if (reinterpret_cast<uintptr_t>(p) % 16 != 0 || hipPointerGetAttributes(&attr, p) != hipSuccess ||
            attr.type != hipMemoryTypeHost) {
            (void)hipGetLastError();  // a pointer the runtime does not know is an error there, not here
            ok = false;
        }
    }
    c->gpu_readable[layer] = ok ? 1 : 0;
    // all three tensors inside one attached mapping: misses are read from the file
    if (c->layer_file.size() < static_cast<size_t>(c->n_layers)) c->layer_file.assign(c->n_layers, -1);
    c->layer_file[layer] = -1;
    const size_t span[3] = {c->s_gate[layer] * (c->n_experts - 1) + c->gate_bytes, c->s_up[layer] * (c->n_experts - 1) + c->up_bytes,
                            c->s_down[layer] * (c->n_experts - 1) + c->down_bytes};
    for (size_t f = 0; f < c->files.size() && !ok; ++f) {
        bool inside = true;
        for (int q = 0; q < 3; ++q)
            inside = inside && ptrs[q] >= c->files[f].base && ptrs[q] + span[q] <= c->files[f].base + c->files[f].size;
        if (inside) {
            c->layer_file[layer] = static_cast<int8_t>(f);
            break;
        }
    }
}
}  // namespace

extern "C" {

int wd_expert_cache_create(wd_expert_cache **out, size_t capacity_bytes, size_t gate_bytes, size_t up_bytes,
                           size_t down_bytes, int n_layers, int n_experts, int layer_partition) {
    WD_REQUIRE(out != nullptr, "expert cache: null output pointer");
    WD_REQUIRE(capacity_bytes > 0, "expert cache capacity is zero");
    WD_REQUIRE(gate_bytes > 0 && up_bytes > 0 && down_bytes > 0, "expert cache slot is empty");
    WD_REQUIRE(n_layers > 0 && n_experts > 0, "expert cache: invalid layer/expert counts");
    // every tensor of a slot starts 16-byte aligned so that rows keep the alignment they have in a GGUF file
    WD_REQUIRE(gate_bytes % 16 == 0 && up_bytes % 16 == 0 && down_bytes % 16 == 0,
               "expert cache: tensor slices must be multiples of 16 bytes");
    const size_t slot_bytes = gate_bytes + up_bytes + down_bytes;
    const size_t n_slots = capacity_bytes / slot_bytes;
    WD_REQUIRE(n_slots > 0, "expert cache capacity is smaller than one expert slot");
    wd_expert_cache *c = new (std::nothrow) wd_expert_cache;
    WD_REQUIRE(c != nullptr, "expert cache: out of host memory");
    c->n_slots = n_slots, c->slot_bytes = slot_bytes;
    c->gate_bytes = gate_bytes, c->up_bytes = up_bytes, c->down_bytes = down_bytes;
    c->n_layers = n_layers, c->n_experts = n_experts;
    c->partitioned = layer_partition != 0 && static_cast<size_t>(n_layers) <= n_slots;
    c->slots.resize(n_slots);
    const int n_parts = c->partitioned ? n_layers : 1;
    c->parts.resize(n_parts);
    for (int p = 0; p < n_parts; ++p) {
        // same split as the reference: n / layers slots each, the first n % layers partitions one more
        const size_t per = n_slots / n_parts, rem = n_slots % n_parts;
        Partition &P = c->parts[p];
        P.begin = p * per + std::min<size_t>(p, rem);
        P.end = P.begin + per + (static_cast<size_t>(p) < rem ? 1 : 0);
        for (size_t s = P.end; s > P.begin; --s) P.free.push_back(s - 1);
    }
    c->h_gate.assign(n_layers, nullptr);
    c->h_up.assign(n_layers, nullptr);
    c->h_down.assign(n_layers, nullptr);
    c->s_gate.assign(n_layers, gate_bytes), c->s_up.assign(n_layers, up_bytes), c->s_down.assign(n_layers, down_bytes);
    auto bail = [&](const char *what, hipError_t e) {
        const int rc = fail(WD_ERR_HIP, "expert cache: %s failed: %s", what, hipGetErrorString(e));
        wd_expert_cache_destroy(c);
        return rc;
    };
    hipError_t e;
    if ((e = hipMalloc(reinterpret_cast<void **>(&c->pool), n_slots * slot_bytes)) != hipSuccess) return bail("hipMalloc pool", e);
    const size_t table_n = static_cast<size_t>(n_layers) * n_experts;
    if ((e = hipMalloc(reinterpret_cast<void **>(&c->d_table), table_n * sizeof(int32_t))) != hipSuccess)
        return bail("hipMalloc slot table", e);
    k_fill_i32<<<dim3(static_cast<unsigned>((table_n + 255) / 256)), dim3(256)>>>(c->d_table, -1, table_n);
    if ((e = hipDeviceSynchronize()) != hipSuccess) return bail("slot table fill", e);
    if ((e = hipStreamCreateWithFlags(&c->copy_stream, hipStreamNonBlocking)) != hipSuccess) return bail("copy stream", e);
    if ((e = hipEventCreateWithFlags(&c->ev_retire, hipEventDisableTiming)) != hipSuccess) return bail("event", e);
    if ((e = hipEventCreateWithFlags(&c->ev_done, hipEventDisableTiming)) != hipSuccess) return bail("event", e);
    if ((e = hipHostMalloc(reinterpret_cast<void **>(&c->h_updates), sizeof(SlotUpdate) * kUpdateRing * kMaxUpdates,
                           hipHostMallocDefault)) != hipSuccess)
        return bail("pinned update ring", e);
    if ((e = hipMalloc(reinterpret_cast<void **>(&c->d_updates), sizeof(SlotUpdate) * kUpdateRing * kMaxUpdates)) != hipSuccess)
        return bail("device update ring", e);
    for (int i = 0; i < kUpdateRing; ++i)
        if ((e = hipEventCreateWithFlags(&c->ring_free[i], hipEventDisableTiming)) != hipSuccess) return bail("ring event", e);
    c->stats.slots = n_slots;
    c->stats.slot_bytes = slot_bytes;
    *out = c;
    return WD_OK;
}

int wd_expert_cache_destroy(wd_expert_cache *c) {
    if (!c) return WD_OK;
    if (c->copy_stream) (void)hipStreamSynchronize(c->copy_stream);
    c->ra.stop();  // (joins the reader before its buffers go)
    if (c->ra_mem) (void)hipHostFree(c->ra_mem);
    for (hipEvent_t ev : c->ra_done)
        if (ev) (void)hipEventDestroy(ev);
    (void)hipFree(c->pool);
    (void)hipFree(c->d_table);
    (void)hipFree(c->d_updates);
    if (c->h_updates) (void)hipHostFree(c->h_updates);
    for (TimingSlot &t : c->timing)
        for (hipEvent_t ev : {t.wait_a, t.wait_b, t.begin, t.end})
            if (ev) (void)hipEventDestroy(ev);
    (void)hipFree(c->d_rows);
    (void)hipFree(c->d_fill_done);
    if (c->h_rows) (void)hipHostFree(c->h_rows);
    for (hipEvent_t ev : c->rows_free)
        if (ev) (void)hipEventDestroy(ev);
    if (c->ev_retire) (void)hipEventDestroy(c->ev_retire);
    for (hipEvent_t ev : c->ev_token)
        if (ev) (void)hipEventDestroy(ev);
    if (c->ev_done) (void)hipEventDestroy(c->ev_done);
    for (hipEvent_t ev : c->ev_layer)
        if (ev) (void)hipEventDestroy(ev);
    for (int i = 0; i < kUpdateRing; ++i)
        if (c->ring_free[i]) (void)hipEventDestroy(c->ring_free[i]);
    if (c->copy_stream) (void)hipStreamDestroy(c->copy_stream);
    delete c->pread_pool;
    if (c->stage) (void)hipHostFree(c->stage);
    for (int i = 0; i < kStageRing; ++i)
        if (c->stage_done[i]) (void)hipEventDestroy(c->stage_done[i]);
    for (FileSource &f : c->files)
        if (f.fd >= 0) ::close(f.fd);
    delete c;
    return WD_OK;
}

static int attach_file_at(wd_expert_cache *c, const uint8_t *map_base, size_t map_bytes, int fd, uint64_t file_off, int threads);

int wd_expert_cache_attach_file(wd_expert_cache *c, const uint8_t *map_base, size_t map_bytes, int fd, int threads) {
    return attach_file_at(c, map_base, map_bytes, fd, 0, threads);
}

int wd_file_mapping_of(const void *ptr, wd_file_mapping *out) {
    WD_REQUIRE(ptr != nullptr && out != nullptr, "file mapping lookup: null pointer");
    std::memset(out, 0, sizeof(*out));
    if (!find_file_mapping(ptr, out)) return fail(WD_ERR_ARG, "no readable file mapping holds %p", ptr);
    return WD_OK;
}

int wd_expert_cache_attach_mappings(wd_expert_cache *c, int threads, int *n_attached) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    int attached = 0;
    for (int l = 0; l < c->n_layers; ++l) {
        if (!c->h_gate[l]) continue;
        const uint8_t *ptrs[3] = {c->h_gate[l], c->h_up[l], c->h_down[l]};
        for (const uint8_t *p : ptrs) {
            bool known = false;
            for (const FileSource &f : c->files) known = known || (p >= f.base && p < f.base + f.size);
            if (known) continue;
            wd_file_mapping m;
            if (!find_file_mapping(p, &m)) continue;  // anonymous or pinned memory: the other fill paths take it
            const int fd = ::open(m.path, O_RDONLY | O_CLOEXEC);
            if (fd < 0) continue;
            const int rc = attach_file_at(c, reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(m.start)),
                                          static_cast<size_t>(m.end - m.start), fd, m.file_offset, threads);
            ::close(fd);  // the cache keeps a duplicate
            if (rc != WD_OK) return rc;
            ++attached;
        }
    }
    if (n_attached) *n_attached = attached;
    return WD_OK;
}

static int attach_file_at(wd_expert_cache *c, const uint8_t *map_base, size_t map_bytes, int fd, uint64_t file_off, int threads) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    WD_REQUIRE(map_base != nullptr && map_bytes > 0 && fd >= 0, "expert cache: invalid file mapping");
    WD_REQUIRE(threads >= 1 && threads <= 64, "expert cache: 1..64 pread threads (got %d)", threads);
    WD_REQUIRE(c->files.size() < 100, "expert cache: too many attached files");
    const int own = ::dup(fd);
    WD_REQUIRE(own >= 0, "expert cache: cannot duplicate the file descriptor");
    if (!c->stage) {
        hipError_t e = hipHostMalloc(reinterpret_cast<void **>(&c->stage), static_cast<size_t>(kStageRing) * c->slot_bytes,
                                     hipHostMallocDefault);
        if (e != hipSuccess) {
            ::close(own);
            return fail(WD_ERR_HIP, "expert cache: pinned staging ring failed: %s", hipGetErrorString(e));
        }
        for (int i = 0; i < kStageRing; ++i) WD_HIP(hipEventCreateWithFlags(&c->stage_done[i], hipEventDisableTiming));
    }
    if (!c->pread_pool) c->pread_pool = new PreadPool(threads);
    FileSource f;
    f.base = map_base, f.size = map_bytes, f.fd = own, f.file_off = file_off;
    c->files.push_back(f);
    for (int l = 0; l < c->n_layers; ++l)  // layers registered before the file was attached
        if (c->h_gate[l]) classify_layer(c, l);
    return WD_OK;
}

int wd_expert_cache_register_layer(wd_expert_cache *c, int layer, const uint8_t *h_gate, const uint8_t *h_up,
                                   const uint8_t *h_down) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    WD_REQUIRE(layer >= 0 && layer < c->n_layers, "expert cache: layer %d out of range", layer);
    WD_REQUIRE(h_gate && h_up && h_down, "expert cache: null host tensor");
    c->h_gate[layer] = h_gate, c->h_up[layer] = h_up, c->h_down[layer] = h_down;
    c->s_gate[layer] = c->gate_bytes, c->s_up[layer] = c->up_bytes, c->s_down[layer] = c->down_bytes;
    classify_layer(c, layer);
    return WD_OK;
}

int wd_expert_cache_register_layer_strided(wd_expert_cache *c, int layer, const uint8_t *h_gate, const uint8_t *h_up,
                                           const uint8_t *h_down, size_t gate_stride, size_t up_stride,
                                           size_t down_stride) {
    if (const int rc = wd_expert_cache_register_layer(c, layer, h_gate, h_up, h_down)) return rc;
    WD_REQUIRE(gate_stride >= c->gate_bytes && up_stride >= c->up_bytes && down_stride >= c->down_bytes,
               "expert cache: an expert stride is smaller than the expert");
    c->s_gate[layer] = gate_stride, c->s_up[layer] = up_stride, c->s_down[layer] = down_stride;
    classify_layer(c, layer);
    return WD_OK;
}

int wd_expert_cache_set_read_ahead(wd_expert_cache *c, int depth, int slots) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    WD_REQUIRE(depth >= 0 && depth <= 8 && slots >= 0 && slots <= 1024, "expert cache read-ahead: depth 0..8, slots 0..1024 (got %d, %d)", depth, slots);
    if (c->copy_stream) WD_HIP(hipStreamSynchronize(c->copy_stream));  // no DMA reads the old ring any more
    c->ra.stop();
    if (c->ra_mem) (void)hipHostFree(c->ra_mem);
    c->ra_mem = nullptr;
    for (hipEvent_t ev : c->ra_done)
        if (ev) (void)hipEventDestroy(ev);
    c->ra_done.clear();
    c->ra_plan = wd::PrefetchPlanner();
    c->ra_plan.set_depth(depth);
    if (depth == 0) return WD_OK;
    const int n = slots > 0 ? slots : depth * 16;  // (the reference's default, src/expert_cache.cuh:995)
    WD_HIP(hipHostMalloc(reinterpret_cast<void **>(&c->ra_mem), static_cast<size_t>(n) * c->slot_bytes, hipHostMallocDefault));
    std::vector<uint8_t *> bufs;
    c->ra_done.assign(n, nullptr);
    for (int i = 0; i < n; ++i) {
        bufs.push_back(c->ra_mem + static_cast<size_t>(i) * c->slot_bytes);
        WD_HIP(hipEventCreateWithFlags(&c->ra_done[i], hipEventDisableTiming));
    }
    c->ra.start(bufs, [c](int shelf) { return hipEventQuery(c->ra_done[static_cast<size_t>(shelf)]) == hipSuccess; });
    return WD_OK;
}

int wd_expert_cache_set_copy_kernel(wd_expert_cache *c, int enabled) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    c->use_copy_kernel = enabled != 0;
    return WD_OK;
}

}  // extern "C"

namespace {

// `defer_wait`: the fills are queued behind the work already on `stream`, but `stream` is not made to wait
// for them; the caller does that later with wait_fills(), after it has queued work that does not depend on
// the new experts (the previous layer).  A victim must then be older than the previous acquire call too.
// `ahead` (token-ahead acquires, see acquire_token_ahead): victims must be older than ahead->floor, the fills'
// completion is recorded in the layer's own event, and the wait for the slots' last readers is done once per token.
struct AheadState {
    uint64_t floor;
    bool retired;
    hipEvent_t before = nullptr;  // not null: the fills may start once this event of the caller's stream has passed
    std::vector<SlotUpdate> updates;
    // Copy-kernel fills are collected over a group of layers and launched together: a launch that moves one expert
    // reaches 31 GB/s over the host link, one that moves eight 46 GB/s (the fixed cost of a launch is about 20 us).
    FillSegments fills;
    int n_fill = 0;
    uint32_t max_words = 0;
    std::vector<int> group;  // layers whose fills are queued but not yet covered by an event
};

int launch_fill_segments(wd_expert_cache *c, FillSegments &fills, int &n_fill, uint32_t &max_words, unsigned long long mark_layers = 0ull);


// ---- device-side timings of the fills (only with c->timing_on) ----------------------------------------------------
// Intervals whose events have passed are added up and their slots given back.
void timing_harvest(wd_expert_cache *c) {
    for (TimingSlot &t : c->timing) {
        if (!t.used) continue;
        if (hipEventQuery(t.end) != hipSuccess) {
            (void)hipGetLastError();
            continue;
        }
        float ms = 0.0f;
        if (t.has_dma && hipEventElapsedTime(&ms, t.begin, t.end) == hipSuccess) {
            c->dma_ms += ms, ++c->dma_calls;
            if (ms > c->dma_max_ms) c->dma_max_ms = ms;
        }
        if (t.has_wait && hipEventElapsedTime(&ms, t.wait_a, t.wait_b) == hipSuccess) {
            c->stall_ms += ms, ++c->stall_calls;
            if (ms > c->stall_max_ms) c->stall_max_ms = ms;
        }
        (void)hipGetLastError();
        t.used = t.has_wait = t.has_dma = false;
    }
}
// The slot the fills being queued are timed in (opened on demand); null when timing is off or every slot is in flight.
TimingSlot *timing_slot(wd_expert_cache *c) {
    if (!c->timing_on) return nullptr;
    if (c->timing_cur >= 0) return &c->timing[c->timing_cur];
    for (int pass = 0; pass < 2; ++pass) {
        for (int i = 0; i < kTimingSlots; ++i) {
            const int idx = (c->timing_next + i) % kTimingSlots;
            if (!c->timing[idx].used) {
                c->timing_cur = idx, c->timing_next = (idx + 1) % kTimingSlots;
                c->timing[idx].has_wait = c->timing[idx].has_dma = false;
                return &c->timing[idx];
            }
        }
        timing_harvest(c);
    }
    ++c->timing_skipped;
    return nullptr;
}
// Around the copy stream's wait for the slots' last readers.
void timing_wait_begin(wd_expert_cache *c) {
    if (TimingSlot *t = timing_slot(c)) (void)hipEventRecord(t->wait_a, c->copy_stream);
}
void timing_wait_end(wd_expert_cache *c) {
    if (c->timing_cur >= 0) {
        TimingSlot &t = c->timing[c->timing_cur];
        (void)hipEventRecord(t.wait_b, c->copy_stream);
        t.has_wait = true;
    }
}
// Before the first copy or copy kernel of the fills being queued.
void timing_dma_begin(wd_expert_cache *c) {
    TimingSlot *t = timing_slot(c);
    if (t && !t->has_dma) {
        (void)hipEventRecord(t->begin, c->copy_stream);
        t->has_dma = true;
    }
}
// After their last one.
void timing_close(wd_expert_cache *c) {
    if (c->timing_cur < 0) return;
    TimingSlot &t = c->timing[c->timing_cur];
    if (!t.has_dma) (void)hipEventRecord(t.begin, c->copy_stream);  // (a wait without fills of its own: an empty interval closes the slot)
    (void)hipEventRecord(t.end, c->copy_stream);
    t.used = true;
    c->timing_cur = -1;
}

// Uploads a batch of slot-table changes and applies them in order on the caller's stream.
int flush_slot_updates(wd_expert_cache *c, const SlotUpdate *updates, int n_updates, hipStream_t st) {
    for (int done = 0; done < n_updates; done += kMaxUpdates) {
        const int n = n_updates - done < kMaxUpdates ? n_updates - done : kMaxUpdates;
        const int r = c->ring_next;
        c->ring_next = (r + 1) % kUpdateRing;
        if (c->ring_used[r]) WD_HIP(hipEventSynchronize(c->ring_free[r]));  // the entry's last use has been consumed
        SlotUpdate *h = c->h_updates + static_cast<size_t>(r) * kMaxUpdates;
        SlotUpdate *d = c->d_updates + static_cast<size_t>(r) * kMaxUpdates;
        for (int i = 0; i < n; ++i) h[i] = updates[done + i];
        WD_HIP(hipMemcpyAsync(d, h, sizeof(SlotUpdate) * n, hipMemcpyHostToDevice, st));
        k_apply_slot_updates<<<dim3(1), dim3(64), 0, st>>>(c->d_table, d, n);
        WD_LAUNCH_CHECK();
        WD_HIP(hipEventRecord(c->ring_free[r], st));  // both copies of ring entry r are free after this point
        c->ring_used[r] = true;
    }
    return WD_OK;
}
int acquire_impl(wd_expert_cache *c, int layer, const int32_t *h_ids, int k, uint8_t *hit_out, void *stream,
                 bool defer_wait, AheadState *ahead = nullptr) {
    WD_REQUIRE(c != nullptr && c->pool != nullptr, "expert cache is not initialized");
    WD_REQUIRE(layer >= 0 && layer < c->n_layers, "expert cache: layer %d out of range", layer);
    WD_REQUIRE(h_ids != nullptr && k > 0 && 2 * k <= kMaxUpdates, "expert cache: invalid id list (k=%d)", k);
    WD_REQUIRE(c->h_gate[layer] != nullptr, "expert cache: layer %d has no registered host tensors", layer);
    Partition &P = c->parts[c->partitioned ? layer : 0];
    WD_REQUIRE(P.end - P.begin >= static_cast<size_t>(k), "expert cache: %zu slots cannot hold %d experts at once",
               P.end - P.begin, k);
    // every id is checked before anything changes: a bad one must not leave half of the call applied
    for (int j = 0; j < k; ++j)
        WD_REQUIRE(h_ids[j] >= 0 && h_ids[j] < c->n_experts, "expert index out of range: %d", h_ids[j]);
    hipStream_t st = as_stream(stream);
    SiteScope site(WD_SITE_ACQUIRE, st);
    const auto t_begin = std::chrono::steady_clock::now();
    if (c->last_gap_layer >= 0) {  // the host's time since the previous acquire returned, by whether the layer changed
        const double gap = std::chrono::duration<double, std::milli>(t_begin - c->last_acquire_exit).count();
        (layer == c->last_gap_layer ? c->intra_gap_ms : c->layer_gap_ms) += gap;
    }
    if (c->last_gap_layer < 0 || layer < c->last_gap_layer) ++c->tokens_seen;  // (a lower layer than the one before begins a token)
    c->last_gap_layer = layer;
    struct Timer {
        wd_expert_cache *c;
        std::chrono::steady_clock::time_point t0;
        ~Timer() {
            const auto now = std::chrono::steady_clock::now();
            c->acquire_ms += std::chrono::duration<double, std::milli>(now - t0).count();
            ++c->acquire_calls;
            c->last_acquire_exit = now;
        }
    } timer{c, t_begin};
    if (c->layer_access.size() < static_cast<size_t>(c->n_layers)) {
        c->layer_access.assign(c->n_layers, 0);
        c->layer_misses.assign(c->n_layers, 0);
        c->prev_ids.assign(c->n_layers, {});
    }
    {   // reuse of the previous call's experts of this layer (the previous token in a decode loop)
        std::vector<int32_t> &prev = c->prev_ids[layer];
        if (!prev.empty()) {
            for (int j = 0; j < k; ++j) {
                ++c->prev_ready;
                for (int32_t p : prev)
                    if (p == h_ids[j]) {
                        ++c->prev_hit;
                        break;
                    }
            }
        }
        prev.assign(h_ids, h_ids + k);
    }
    const uint64_t epoch_floor = c->clock;  // slots touched by this call carry last_use > epoch_floor
    const uint64_t victim_floor = ahead ? ahead->floor : (defer_wait ? c->prev_floor : epoch_floor);
    c->prev_floor = epoch_floor;
    SlotUpdate updates[kMaxUpdates];
    int n_updates = 0;
    bool waited = false;
    const bool by_kernel = c->use_copy_kernel && static_cast<size_t>(layer) < c->gpu_readable.size() && c->gpu_readable[layer];
    const bool by_file = !by_kernel && static_cast<size_t>(layer) < c->layer_file.size() && c->layer_file[layer] >= 0 &&
                         !(static_cast<size_t>(layer) < c->gpu_readable.size() && c->gpu_readable[layer]);
    FillSegments own_fills;
    int own_n_fill = 0;
    uint32_t own_max_words = 0;
    FillSegments &fills = ahead ? ahead->fills : own_fills;
    int &n_fill = ahead ? ahead->n_fill : own_n_fill;
    uint32_t &max_words = ahead ? ahead->max_words : own_max_words;

    // A failure inside the loop (no slot may be recycled, a short read from the file) ends the loop, not the call: the
    // fills and slot-table changes of the experts acquired before it are still issued below, so that the host's index
    // and the device's table describe the same pool when the error is returned.
    int rc_late = WD_OK;
    for (int j = 0; j < k; ++j) {
        const int e = h_ids[j];
        const uint64_t key = (static_cast<uint64_t>(static_cast<uint32_t>(layer)) << 32) | static_cast<uint32_t>(e);
        ++c->clock;
        ++c->stats.accesses;
        ++c->layer_access[layer];
        c->distinct.insert(key);
        for (Shadow &sh : c->shadows) sh.access(key);
        if (c->ra.running() && !ahead) {
            // what the previous token took in this layer (and the next ones): read it from the file while the layers compute
            for (uint64_t cand : c->ra_plan.on_acquire(layer, key)) {
                ++c->ra_candidates;
                if (c->index.find(cand) != c->index.end()) {
                    ++c->ra_resident_skips;
                    continue;
                }
                const size_t cl = static_cast<size_t>(cand >> 32), ce = static_cast<size_t>(cand & 0xffffffffu);
                if (cl >= c->layer_file.size() || c->layer_file[cl] < 0 || (cl < c->gpu_readable.size() && c->gpu_readable[cl]) ||
                    !c->h_gate[cl] || ce >= static_cast<size_t>(c->n_experts))
                    continue;
                const FileSource &fs = c->files[c->layer_file[cl]];
                const uint8_t *src[3] = {c->h_gate[cl] + ce * c->s_gate[cl], c->h_up[cl] + ce * c->s_up[cl], c->h_down[cl] + ce * c->s_down[cl]};
                const wd::PrefetchRun runs[3] = {{fs.file_off + static_cast<uint64_t>(src[0] - fs.base), 0, c->gate_bytes},
                                                 {fs.file_off + static_cast<uint64_t>(src[1] - fs.base), c->gate_bytes, c->up_bytes},
                                                 {fs.file_off + static_cast<uint64_t>(src[2] - fs.base), c->gate_bytes + c->up_bytes, c->down_bytes}};
                c->ra.request(cand, fs.fd, runs, 3);
            }
        }
        auto it = c->index.find(key);
        if (it != c->index.end()) {
            Slot &s = c->slots[it->second];
            s.last_use = c->clock;
            Partition &Q = c->parts[c->partitioned ? static_cast<int>(s.key >> 32) : 0];
            Q.lru.splice(Q.lru.end(), Q.lru, s.lru);  // most recently used goes to the back
            ++c->stats.hits;
            if (hit_out) hit_out[j] = 1;
            continue;
        }
        ++c->stats.misses;
        ++c->layer_misses[layer];
        if (hit_out) hit_out[j] = 0;
        size_t slot;
        if (!P.free.empty()) {
            slot = P.free.back();
            P.free.pop_back();
        } else {
            slot = P.lru.front();
            Slot &victim = c->slots[slot];
            if (victim.last_use > victim_floor) {
                rc_late = fail(WD_ERR_STATE, "expert cache: all slots are held by the experts being acquired");
                break;
            }
            P.lru.pop_front();
            c->index.erase(victim.key);
            updates[n_updates++] = {static_cast<int32_t>((victim.key >> 32) * c->n_experts + (victim.key & 0xffffffffu)), -1};
            ++c->stats.evictions;
        }
        Slot &s = c->slots[slot];
        s.key = key, s.last_use = c->clock, s.valid = true;
        P.lru.push_back(slot);
        s.lru = std::prev(P.lru.end());
        c->index[key] = slot;
        updates[n_updates++] = {static_cast<int32_t>(layer * c->n_experts + e), static_cast<int32_t>(slot)};

        if (!waited) {
            // kernels already queued on the caller's stream may still read the victim slot
            if (!ahead || !ahead->retired) {
                timing_wait_begin(c);
                if (ahead && ahead->before) {
                    WD_HIP(hipStreamWaitEvent(c->copy_stream, ahead->before, 0));
                } else {
                    WD_HIP(hipEventRecord(c->ev_retire, st));
                    WD_HIP(hipStreamWaitEvent(c->copy_stream, c->ev_retire, 0));
                }
                timing_wait_end(c);
                if (ahead) ahead->retired = true;
            }
            waited = true;
        }
        uint8_t *dst = c->pool + slot * c->slot_bytes;
        const uint8_t *src3[3] = {c->h_gate[layer] + static_cast<size_t>(e) * c->s_gate[layer],
                                  c->h_up[layer] + static_cast<size_t>(e) * c->s_up[layer],
                                  c->h_down[layer] + static_cast<size_t>(e) * c->s_down[layer]};
        uint8_t *dst3[3] = {dst, dst + c->gate_bytes, dst + c->gate_bytes + c->up_bytes};
        const size_t len3[3] = {c->gate_bytes, c->up_bytes, c->down_bytes};
        const bool one_piece = src3[0] + len3[0] == src3[1] && src3[1] + len3[1] == src3[2];
        const int shelf = by_file ? c->ra.claim(key) : -1;
        if (shelf >= 0) {
            // a prediction that came true: the slot's bytes are in pinned memory already, laid out like the slot
            timing_dma_begin(c);
            const hipError_t e1 = hipMemcpyAsync(dst, c->ra.data(shelf), c->slot_bytes, hipMemcpyHostToDevice, c->copy_stream);
            const hipError_t e2 = hipEventRecord(c->ra_done[static_cast<size_t>(shelf)], c->copy_stream);
            c->ra.copy_queued(shelf);  // (also after an error: the event then speaks of whatever was queued before)
            WD_HIP(e1);
            WD_HIP(e2);
            ++c->ra_fills;
        } else if (by_file) {
            // the three slices land in one ring entry in slot order, then the slot is filled with one DMA
            const FileSource &fs = c->files[c->layer_file[layer]];
            const int r = c->stage_next;
            c->stage_next = (r + 1) % kStageRing;
            if (c->stage_used[r]) WD_HIP(hipEventSynchronize(c->stage_done[r]));  // its last DMA has read it
            uint8_t *entry = c->stage + static_cast<size_t>(r) * c->slot_bytes;
            const auto t0 = std::chrono::steady_clock::now();
            PreadPiece pieces[3 * 8];
            int n_pieces = 0;
            size_t at = 0;
            for (int q = 0; q < 3; ++q) {  // pieces of about 256 KiB so that the workers share one expert
                const uint64_t file_off = fs.file_off + static_cast<uint64_t>(src3[q] - fs.base);
                const size_t parts = len3[q] >= (512u << 10) ? 4 : (len3[q] >= (256u << 10) ? 2 : 1);
                for (size_t pi = 0; pi < parts; ++pi) {
                    const size_t lo = len3[q] * pi / parts, hi = len3[q] * (pi + 1) / parts;
                    pieces[n_pieces++] = {fs.fd, file_off + lo, hi - lo, entry + at + lo};
                }
                at += len3[q];
            }
            if (!c->pread_pool->run(pieces, n_pieces)) {
                // this expert never reached its slot: take it out of the index again (the victim stays evicted)
                c->index.erase(key);
                P.lru.pop_back();
                s.valid = false;
                P.free.insert(std::upper_bound(P.free.begin(), P.free.end(), slot, std::greater<size_t>()), slot);
                --n_updates;
                rc_late = fail(WD_ERR_STATE, "expert cache: pread of layer %d expert %d failed or came up short", layer, e);
                break;
            }
            c->pread_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            timing_dma_begin(c);
            WD_HIP(hipMemcpyAsync(dst, entry, c->slot_bytes, hipMemcpyHostToDevice, c->copy_stream));
            WD_HIP(hipEventRecord(c->stage_done[r], c->copy_stream));
            c->stage_used[r] = true;
            ++c->pread_fills;
        } else if (by_kernel) {
            if (n_fill + 3 > kMaxFillSegments)  // (token-ahead groups only: one call alone never has that many)
                if (const int rc = launch_fill_segments(c, fills, n_fill, max_words)) return rc;
            // an expert whose three pieces lie back to back on the host (a copy packed per expert) is one segment
            const int n_seg = one_piece ? 1 : 3;
            for (int q = 0; q < n_seg; ++q) {
                fills.src[n_fill] = src3[q], fills.dst[n_fill] = dst3[q];
                fills.words[n_fill] = static_cast<uint32_t>((one_piece ? c->slot_bytes : len3[q]) / 16);
                max_words = fills.words[n_fill] > max_words ? fills.words[n_fill] : max_words;
                ++n_fill;
            }
            ++c->kernel_fills;
        } else {
            timing_dma_begin(c);
            if (one_piece) {
                WD_HIP(hipMemcpyAsync(dst, src3[0], c->slot_bytes, hipMemcpyHostToDevice, c->copy_stream));
            } else {
                for (int q = 0; q < 3; ++q)
                    WD_HIP(hipMemcpyAsync(dst3[q], src3[q], len3[q], hipMemcpyHostToDevice, c->copy_stream));
            }
            ++c->dma_fills;
        }
        c->stats.bytes_copied += c->slot_bytes;
    }
    c->stats.resident = c->index.size();
    if (!ahead)
        if (const int rc = launch_fill_segments(c, fills, n_fill, max_words)) return rc;

    if (n_updates > 0) {
        if (ahead) {  // applied once for the whole token, before its first layer
            ahead->updates.insert(ahead->updates.end(), updates, updates + n_updates);
        } else if (const int rc = flush_slot_updates(c, updates, n_updates, st)) {
            return rc;
        }
    }
    if (waited) {
        if (ahead) {
            ahead->group.push_back(layer);  // the event that covers the layer is recorded when its group is closed
        } else {
            timing_close(c);
            WD_HIP(hipEventRecord(c->ev_done, c->copy_stream));
            if (defer_wait)
                c->fills_pending = true;
            else
                WD_HIP(hipStreamWaitEvent(st, c->ev_done, 0));
        }
    }
    return rc_late;
}

int launch_fill_segments(wd_expert_cache *c, FillSegments &fills, int &n_fill, uint32_t &max_words, unsigned long long mark_layers) {
    if (n_fill > 0 || mark_layers != 0ull) {
        SiteScope site(WD_SITE_CACHE_FILL, c->copy_stream);
        // enough workgroups per segment to keep the host link busy, few enough to leave the decode its compute units
        timing_dma_begin(c);
        const bool beside = c->mark_seq != 0u;  // the token goes through a one-launch stack: every fill has to find room beside it
        const uint32_t round_words = WD_FILL_THREADS * (beside ? kFillBesideUnroll : WD_FILL_UNROLL), most = beside ? kFillBesideWgs : WD_FILL_WGS;
        const uint32_t per_seg = (max_words + round_words - 1) / round_words;
        const dim3 grid(per_seg < most ? (per_seg ? per_seg : 1) : most);
        if (beside) {
            const FillMarks marks{mark_layers ? c->d_fill_done : nullptr, reinterpret_cast<unsigned *>(c->d_fill_done + kRowsLayers), mark_layers, c->mark_seq};
            k_fill_slots_beside<<<grid, dim3(WD_FILL_THREADS), 0, c->copy_stream>>>(fills, n_fill, marks);
        } else {
            k_fill_slots<<<grid, dim3(WD_FILL_THREADS), 0, c->copy_stream>>>(fills, n_fill);
        }
        WD_LAUNCH_CHECK();
    }
    n_fill = 0, max_words = 0;
    return WD_OK;
}
// Launches what the group has collected and records the event its layers wait for.
int close_ahead_group(wd_expert_cache *c, AheadState &ahead) {
    unsigned long long mark_layers = 0ull;
    if (c->mark_seq != 0u)
        for (int l : ahead.group)
            if (l < kRowsLayers) mark_layers |= 1ull << l, c->layer_need[static_cast<size_t>(l)] = c->mark_seq;
    if (const int rc = launch_fill_segments(c, ahead.fills, ahead.n_fill, ahead.max_words, mark_layers)) return rc;
    if (!ahead.group.empty()) {
        const int last = ahead.group.back();
        timing_close(c);
        WD_HIP(hipEventRecord(c->ev_layer[last], c->copy_stream));
        for (int l : ahead.group) c->layer_pending[l] = 1, c->layer_event[l] = last;
        ahead.group.clear();
    }
    return WD_OK;
}

#ifndef WD_AHEAD_GROUP
#define WD_AHEAD_GROUP 8  // layers per group of fills at most (the first groups are 1, 1, 2, 4 layers: the first layers wait least)
#endif
// Acquires the experts of every layer of one token before any of the token's layers is launched, so that the host
// link streams the token's misses back to back while the layers compute; wait_layer_fills(l) then makes the stream
// wait for layer l's fills only.  Needs a pool that holds a whole token: the slots a token touches are not evicted
// by its own later layers (victims must be older than the token).  h_ids: [n_layers][k].
int acquire_token_ahead(wd_expert_cache *c, int n_layers, const int32_t *h_ids, int k, void *stream) {
    if (c->ev_layer.size() < static_cast<size_t>(c->n_layers)) {
        c->ev_layer.resize(c->n_layers, nullptr);
        c->layer_pending.assign(c->n_layers, 0);
        c->layer_event.assign(c->n_layers, 0);
        for (hipEvent_t &ev : c->ev_layer)
            if (!ev) WD_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    }
    AheadState ahead;
    ahead.floor = c->clock, ahead.retired = false;
    c->last_waited = -1;
    // A pool that holds three tokens' experts always has a victim that the previous token did not touch either: such a
    // slot was last read by work queued before the previous token, so this token's fills need not wait for the previous
    // token's layers - they wait for the event recorded when the previous token was queued, and cross the host link
    // while its layers compute.
    if (!c->ev_token[0])
        for (hipEvent_t &ev : c->ev_token) WD_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    const Partition &P0 = c->parts[0];
    const bool relaxed = !c->partitioned && c->have_prev_token && P0.end - P0.begin >= 3 * static_cast<size_t>(n_layers) * k;
    WD_HIP(hipEventRecord(c->ev_token[c->token_parity], as_stream(stream)));  // everything queued before this token
    if (relaxed) {
        ahead.floor = c->prev_token_floor;
        ahead.before = c->ev_token[c->token_parity ^ 1];
    }
    c->prev_token_floor = c->clock, c->have_prev_token = true, c->token_parity ^= 1;
    int rc_late = WD_OK, group_end = 1, group_len = 1;
    for (int l = 0; l < n_layers && rc_late == WD_OK; ++l) {
        rc_late = acquire_impl(c, l, h_ids + static_cast<size_t>(l) * k, k, nullptr, stream, true, &ahead);
        if (l + 1 == group_end || l + 1 == n_layers || rc_late != WD_OK) {
            if (const int rc = close_ahead_group(c, ahead)) return rc;
            group_len = l + 1 < 2 ? 1 : (2 * group_len < WD_AHEAD_GROUP ? 2 * group_len : WD_AHEAD_GROUP);
            group_end = l + 1 + group_len;
        }
    }
    // also after a failure: the table must describe what the layers before it did to the pool
    const int rc = flush_slot_updates(c, ahead.updates.data(), static_cast<int>(ahead.updates.size()), as_stream(stream));
    return rc_late != WD_OK ? rc_late : rc;
}

int wait_layer_fills(wd_expert_cache *c, int layer, hipStream_t st) {
    if (static_cast<size_t>(layer) < c->layer_pending.size() && c->layer_pending[layer]) {
        // the layers of a group wait for one event: the stream is told once (the call costs the host about 20 us)
        if (c->layer_event[layer] != c->last_waited) WD_HIP(hipStreamWaitEvent(st, c->ev_layer[c->layer_event[layer]], 0));
        c->last_waited = c->layer_event[layer];
        c->layer_pending[layer] = 0;
    }
    return WD_OK;
}

// What a one-launch stack needs beside the pool (allocated at the first such token).
int rows_prepare(wd_expert_cache *c) {
    if (c->d_fill_done) return WD_OK;
    WD_HIP(hipHostMalloc(reinterpret_cast<void **>(&c->h_rows), sizeof(int32_t) * kRowsRing * kRowsEntry, hipHostMallocDefault));
    WD_HIP(hipMalloc(reinterpret_cast<void **>(&c->d_rows), sizeof(int32_t) * kRowsRing * kRowsEntry));
    for (hipEvent_t &ev : c->rows_free) WD_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    uint32_t *done = nullptr;
    WD_HIP(hipMalloc(reinterpret_cast<void **>(&done), sizeof(uint32_t) * (kRowsLayers + 64)));
    WD_HIP(hipMemset(done, 0, sizeof(uint32_t) * (kRowsLayers + 64)));
    c->d_fill_done = done;
    c->layer_need.assign(kRowsLayers, 0u);
    return WD_OK;
}

// Begins a token whose fills count layers off: the number they carry (never 0).
uint32_t rows_begin_token(wd_expert_cache *c) {
    if (++c->fill_seq == 0u) ++c->fill_seq;
    std::fill(c->layer_need.begin(), c->layer_need.end(), 0u);
    return c->fill_seq;
}

// After the token's acquire: the slot of every (layer, expert) of h_ids [n_layers][k] and every layer's number, on their
// way to the device behind the work already on `st`.  rows: [n_layers][k] slot numbers; need: [n_layers].
int rows_upload(wd_expert_cache *c, int n_layers, const int32_t *h_ids, int k, hipStream_t st, const int32_t **rows, const uint32_t **need) {
    const int r = c->rows_next;
    c->rows_next = (r + 1) % kRowsRing;
    if (c->rows_used[r]) WD_HIP(hipEventSynchronize(c->rows_free[r]));  // the copy that last read this entry is through
    int32_t *h = c->h_rows + static_cast<size_t>(r) * kRowsEntry, *d = c->d_rows + static_cast<size_t>(r) * kRowsEntry;
    for (int l = 0; l < n_layers; ++l) {
        for (int j = 0; j < k; ++j) {
            const auto it = c->index.find((static_cast<uint64_t>(static_cast<uint32_t>(l)) << 32) | static_cast<uint32_t>(h_ids[l * k + j]));
            WD_REQUIRE(it != c->index.end(), "expert cache: layer %d expert %d has no slot after its acquire", l, h_ids[l * k + j]);
            h[l * k + j] = static_cast<int32_t>(it->second);
        }
        h[n_layers * k + l] = static_cast<int32_t>(c->layer_need[static_cast<size_t>(l)]);
    }
    WD_HIP(hipMemcpyAsync(d, h, sizeof(int32_t) * static_cast<size_t>(n_layers) * (k + 1), hipMemcpyHostToDevice, st));
    WD_HIP(hipEventRecord(c->rows_free[r], st));
    c->rows_used[r] = true;
    *rows = d, *need = reinterpret_cast<const uint32_t *>(d + n_layers * k);
    return WD_OK;
}

int wait_fills(wd_expert_cache *c, hipStream_t st) {
    if (c->fills_pending) {
        WD_HIP(hipStreamWaitEvent(st, c->ev_done, 0));
        c->fills_pending = false;
    }
    return WD_OK;
}

}  // namespace

extern "C" {

int wd_expert_cache_acquire(wd_expert_cache *c, int layer, const int32_t *h_ids, int k, uint8_t *hit_out,
                            void *stream) {
    if (c && c->fills_pending) {
        if (const int rc = wait_fills(c, as_stream(stream))) return rc;
    }
    return acquire_impl(c, layer, h_ids, k, hit_out, stream, false);
}

const int32_t *wd_expert_cache_slot_table(wd_expert_cache *c, int layer) {
    if (!c || layer < 0 || layer >= c->n_layers) return nullptr;
    return c->d_table + static_cast<size_t>(layer) * c->n_experts;
}

const uint8_t *wd_expert_cache_pool(wd_expert_cache *c) { return c ? c->pool : nullptr; }

long long wd_expert_cache_slot_of(wd_expert_cache *c, int layer, int expert) {
    if (!c || layer < 0 || expert < 0) return -1;
    const auto it = c->index.find((static_cast<uint64_t>(layer) << 32) | static_cast<uint32_t>(expert));
    return it == c->index.end() ? -1 : static_cast<long long>(it->second);
}

int wd_expert_cache_add_shadow(wd_expert_cache *c, int policy, size_t slots) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    WD_REQUIRE(policy == 0 || policy == 1, "expert cache shadow: policy must be 0 (LRU) or 1 (LFU)");
    WD_REQUIRE(c->stats.accesses == 0, "expert cache shadow: add shadows before the first acquire");
    Shadow sh;
    sh.policy = policy;
    sh.capacity = slots ? slots : 1;
    c->shadows.push_back(std::move(sh));
    return WD_OK;
}

int wd_expert_cache_set_timing(wd_expert_cache *c, int enabled) {
    WD_REQUIRE(c != nullptr, "expert cache is not initialized");
    if (enabled && !c->timing[0].end) {
        for (TimingSlot &t : c->timing)
            for (hipEvent_t *ev : {&t.wait_a, &t.wait_b, &t.begin, &t.end}) WD_HIP(hipEventCreate(ev));
    }
    if (!enabled && c->timing_cur >= 0) timing_close(c);
    c->timing_on = enabled != 0;
    return WD_OK;
}

// JSON object with the counters; returns the length needed (without the terminator), writes at most cap bytes.
size_t wd_expert_cache_dump_json(wd_expert_cache *c, char *buf, size_t cap) {
    if (!c) return 0;
    auto arr = [](const std::vector<uint64_t> &v) {
        std::string s = "[";
        for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + std::to_string(v[i]);
        return s + "]";
    };
    char num[64];
    auto fixed = [&](double v, int digits) {
        std::snprintf(num, sizeof(num), "%.*f", digits, v);
        return std::string(num);
    };
    const wd_expert_cache_stats &st = c->stats;
    timing_harvest(c);
    const double tokens = c->tokens_seen ? static_cast<double>(c->tokens_seen) : 1.0;
    std::string s = "{";
    s += "\"mode\":\"" + std::string(c->partitioned ? "layer-partitioned" : "shared") + "\"";
    s += ",\"slots\":" + std::to_string(c->n_slots) + ",\"slot_bytes\":" + std::to_string(c->slot_bytes);
    s += ",\"accesses\":" + std::to_string(st.accesses) + ",\"hits\":" + std::to_string(st.hits);
    s += ",\"misses\":" + std::to_string(st.misses);
    s += ",\"hit_rate\":" + fixed(st.accesses ? static_cast<double>(st.hits) / st.accesses : 0.0, 4);
    s += ",\"evictions\":" + std::to_string(st.evictions) + ",\"bytes_copied\":" + std::to_string(st.bytes_copied);
    s += ",\"gib_copied\":" + fixed(st.bytes_copied / (1024.0 * 1024.0 * 1024.0), 3);
    s += ",\"resident\":" + std::to_string(c->index.size()) + ",\"distinct_pairs\":" + std::to_string(c->distinct.size());
    s += ",\"acquire_calls\":" + std::to_string(c->acquire_calls) + ",\"acquire_ms\":" + fixed(c->acquire_ms, 1);
    s += ",\"fills_by_copy_kernel\":" + std::to_string(c->kernel_fills) + ",\"fills_by_memcpy\":" + std::to_string(c->dma_fills);
    s += ",\"fills_by_pread\":" + std::to_string(c->pread_fills) + ",\"pread_ms\":" + fixed(c->pread_ms, 1);
    s += ",\"read_ahead\":{\"depth\":" + std::to_string(c->ra_plan.depth()) + ",\"slots\":" + std::to_string(c->ra.shelves()) +
         ",\"candidates\":" + std::to_string(c->ra_candidates) + ",\"already_resident\":" + std::to_string(c->ra_resident_skips) +
         ",\"posted\":" + std::to_string(c->ra.requested()) + ",\"dropped\":" + std::to_string(c->ra.dropped()) +
         ",\"delivered\":" + std::to_string(c->ra.delivered()) + ",\"failed\":" + std::to_string(c->ra.failed()) +
         ",\"fills\":" + std::to_string(c->ra_fills) + "}";
    s += ",\"io_timing\":" + std::string(c->timing_on ? "true" : "false");
    s += ",\"io_dma_ms\":" + fixed(c->dma_ms, 1) + ",\"io_dma_max_ms\":" + fixed(c->dma_max_ms, 3) + ",\"io_dma_calls\":" + std::to_string(c->dma_calls);
    s += ",\"io_dma_stall_ms\":" + fixed(c->stall_ms, 1) + ",\"io_dma_stall_max_ms\":" + fixed(c->stall_max_ms, 3) +
         ",\"io_dma_stall_calls\":" + std::to_string(c->stall_calls) + ",\"io_timing_skipped\":" + std::to_string(c->timing_skipped);
    s += ",\"intra_gap_ms\":" + fixed(c->intra_gap_ms, 1) + ",\"layer_gap_ms\":" + fixed(c->layer_gap_ms, 1);
    s += ",\"intra_gap_per_token\":" + fixed(c->intra_gap_ms / tokens, 2) + ",\"layer_gap_per_token\":" + fixed(c->layer_gap_ms / tokens, 2);
    s += ",\"acquire_per_token\":" + fixed(c->acquire_ms / tokens, 2) + ",\"tokens\":" + std::to_string(c->tokens_seen);
    s += ",\"tokens_in_one_launch\":" + std::to_string(c->resident_tokens);
    s += ",\"prev_token_ready\":" + std::to_string(c->prev_ready);
    s += ",\"prev_token_reuse\":" + fixed(c->prev_ready ? static_cast<double>(c->prev_hit) / c->prev_ready : 0.0, 4);
    s += ",\"layer_access\":" + arr(c->layer_access) + ",\"layer_misses\":" + arr(c->layer_misses);
    s += ",\"shadows\":[";
    for (size_t i = 0; i < c->shadows.size(); ++i) {
        const Shadow &sh = c->shadows[i];
        s += std::string(i ? "," : "") + "{\"policy\":\"" + (sh.policy ? "lfu" : "lru") + "\",\"slots\":" + std::to_string(sh.capacity) +
             ",\"hits\":" + std::to_string(sh.hits) + ",\"hit_rate\":" +
             fixed(sh.accesses ? static_cast<double>(sh.hits) / sh.accesses : 0.0, 4) + "}";
    }
    s += "]}";
    if (buf && cap) {
        const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return s.size();
}

int wd_expert_cache_get_stats(wd_expert_cache *c, wd_expert_cache_stats *out) {
    WD_REQUIRE(c != nullptr && out != nullptr, "expert cache stats: null pointer");
    *out = c->stats;
    out->resident = c->index.size();
    return WD_OK;
}

}  // extern "C"
