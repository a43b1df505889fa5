// Read-ahead of experts that a later acquire is expected to want: a ring of buffers laid out like a cache slot, filled
// from the model file by a reader thread while the layers before compute, so that the acquire that does want the expert
// finds its bytes in pinned memory and queues the DMA without reading the file itself.
// Same role and rules as the reference's ExpertReadAhead and the history that feeds it (src/expert_cache.cuh:547-824,
// :1094-1127).  Host code only, no GPU call: the owner supplies the buffers (pinned memory in the cache, plain memory in
// the host test) and tells the ring when the DMA that last read an entry has completed.
//
// Entry states: Free -> Queued (posted, the reader has not got to it) -> Ready (bytes in the buffer) or Failed (a read
// came up short) -> Borrowed (an acquire is queueing its DMA from the buffer) -> InFlight (the DMA is queued and the
// owner's completion test describes this transfer) -> Free again once that test passes.  Only an entry in InFlight,
// Ready or Failed is ever recycled: before InFlight the completion test would still speak of the previous use, and
// recycling would let the reader overwrite bytes the DMA engine is about to read.
#pragma once

#include <unistd.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace wd {

constexpr int kReadAheadSlices = 8;

class ReadAheadRing {
public:
    enum State : int { kFree = 0, kQueued = 1, kReady = 2, kFailed = 3, kBorrowed = 4, kInFlight = 5 };

    ReadAheadRing() = default;
    ReadAheadRing(const ReadAheadRing &) = delete;
    ReadAheadRing &operator=(const ReadAheadRing &) = delete;
    ~ReadAheadRing() { release(); }

    // buffers: one per entry, each able to hold a slot.  dma_done(entry): true when the DMA that was queued from the
    // entry's buffer by its last borrower has completed (called for entries in InFlight only).
    bool configure(const std::vector<uint8_t *> &buffers, std::function<bool(int)> dma_done) {
        release();
        if (buffers.empty()) return false;
        entries_ = std::vector<Entry>(buffers.size());
        for (size_t i = 0; i < buffers.size(); ++i) entries_[i].buf = buffers[i];
        dma_done_ = std::move(dma_done);
        running_.store(true, std::memory_order_release);
        reader_ = std::thread([this] { reader_loop(); });
        return true;
    }
    void release() {
        if (reader_.joinable()) {
            running_.store(false, std::memory_order_release);
            cv_.notify_all();
            reader_.join();
        }
        entries_.clear();
    }
    bool enabled() const { return !entries_.empty(); }
    size_t slots() const { return entries_.size(); }

    // One read-ahead job: `count` slices, slice i = `bytes[i]` bytes at `file_off[i]` of `fd`, to land at `offset[i]` of
    // the entry's buffer.  False when the key is already queued or ready, or when no entry can be recycled (the caller
    // then simply does not read ahead).
    bool post(uint64_t key, int fd, const uint64_t *file_off, const size_t *offset, const size_t *bytes, int count) {
        if (!enabled() || count < 1 || count > kReadAheadSlices) return false;
        for (const Entry &e : entries_) {
            const int st = e.state.load(std::memory_order_acquire);
            if ((st == kQueued || st == kReady) && e.key == key) return false;
        }
        Entry *target = nullptr;
        for (Entry &e : entries_)  // 1) a free entry
            if (e.state.load(std::memory_order_acquire) == kFree) {
                target = &e;
                break;
            }
        if (!target)  // 2) the oldest prediction that was never used (or whose read failed)
            for (Entry &e : entries_) {
                const int st = e.state.load(std::memory_order_acquire);
                if ((st == kReady || st == kFailed) && (!target || e.seq < target->seq)) target = &e;
            }
        if (!target) {  // 3) the oldest borrowed entry whose DMA has completed
            for (size_t i = 0; i < entries_.size(); ++i) {
                Entry &e = entries_[i];
                if (e.state.load(std::memory_order_acquire) != kInFlight) continue;
                if (dma_done_ && dma_done_(static_cast<int>(i)) && (!target || e.seq < target->seq)) target = &e;
            }
        }
        if (!target) {
            ++dropped_;
            return false;
        }
        target->key = key, target->seq = ++posted_seq_, target->fd = fd, target->count = count;
        for (int i = 0; i < count; ++i) target->offset[i] = offset[i], target->bytes[i] = bytes[i], target->file_off[i] = file_off[i];
        target->state.store(kQueued, std::memory_order_release);
        {
            std::lock_guard<std::mutex> lock(mutex_);
            ++queued_;
        }
        cv_.notify_all();
        ++posted_;
        return true;
    }

    // The completed entry for `key`: its buffer (and its index, for the owner's completion test), or null when there is
    // no completed prediction.  The caller queues its DMA from the buffer and then calls finish_borrow.
    uint8_t *borrow(uint64_t key, int *entry_out) {
        for (size_t i = 0; i < entries_.size(); ++i) {
            Entry &e = entries_[i];
            if (e.state.load(std::memory_order_acquire) != kReady || e.key != key) continue;
            e.state.store(kBorrowed, std::memory_order_release);
            if (entry_out) *entry_out = static_cast<int>(i);
            ++used_;
            return e.buf;
        }
        return nullptr;
    }
    void finish_borrow(uint64_t key) {
        for (Entry &e : entries_)
            if (e.key == key && e.state.load(std::memory_order_acquire) == kBorrowed) {
                e.state.store(kInFlight, std::memory_order_release);
                return;
            }
    }

    bool busy() const { return queued_.load(std::memory_order_relaxed) != 0; }
    int state_of(int entry) const { return entries_[static_cast<size_t>(entry)].state.load(std::memory_order_acquire); }
    uint64_t posted() const { return posted_; }
    uint64_t dropped() const { return dropped_; }
    uint64_t used() const { return used_; }
    uint64_t delivered() const { return delivered_.load(std::memory_order_relaxed); }
    uint64_t failed() const { return failed_.load(std::memory_order_relaxed); }

private:
    struct Entry {
        Entry() = default;
        Entry(const Entry &o) : buf(o.buf), state(o.state.load(std::memory_order_relaxed)) {}  // (only while the ring is being sized)
        Entry &operator=(const Entry &o) {
            buf = o.buf;
            state.store(o.state.load(std::memory_order_relaxed), std::memory_order_relaxed);
            return *this;
        }
        uint8_t *buf = nullptr;
        std::atomic<int> state{kFree};
        uint64_t key = 0, seq = 0;
        int fd = -1, count = 0;  // carried by the entry: the reader shares no state with the poster
        size_t offset[kReadAheadSlices] = {}, bytes[kReadAheadSlices] = {};
        uint64_t file_off[kReadAheadSlices] = {};
    };

    void reader_loop() {
        while (running_.load(std::memory_order_acquire)) {
            Entry *job = nullptr;
            for (Entry &e : entries_)
                if (e.state.load(std::memory_order_acquire) == kQueued && (!job || e.seq < job->seq)) job = &e;
            if (!job) {
                std::unique_lock<std::mutex> lock(mutex_);
                cv_.wait_for(lock, std::chrono::microseconds(200));
                continue;
            }
            const bool ok = read_entry(*job);
            if (ok)
                ++delivered_;
            else
                ++failed_;
            job->state.store(ok ? kReady : kFailed, std::memory_order_release);
            std::lock_guard<std::mutex> lock(mutex_);
            if (queued_.load(std::memory_order_relaxed) > 0) --queued_;
        }
    }
    static bool read_entry(const Entry &e) {
        if (e.fd < 0) return false;
        for (int i = 0; i < e.count; ++i) {
            size_t done = 0;
            while (done < e.bytes[i]) {
                const ssize_t n = ::pread(e.fd, e.buf + e.offset[i] + done, e.bytes[i] - done, static_cast<off_t>(e.file_off[i] + done));
                if (n <= 0) return false;
                done += static_cast<size_t>(n);
            }
        }
        return true;
    }

    std::vector<Entry> entries_;
    std::function<bool(int)> dma_done_;
    std::thread reader_;
    std::atomic<bool> running_{false};
    std::mutex mutex_;
    std::condition_variable cv_;
    std::atomic<uint64_t> queued_{0}, delivered_{0}, failed_{0};
    uint64_t posted_seq_ = 0, posted_ = 0, dropped_ = 0, used_ = 0;
};

// What to read ahead: the previous token's expert lists of the next `depth` layers (the layer being acquired counts as
// the first), asked for once per layer and token - at the layer's first acquire, when the previous token's list for it
// is complete - and never containing the expert that is being acquired right now.  A layer index that goes down marks
// a new token.  (src/expert_cache.cuh:1094-1127)
class ReadAheadHistory {
public:
    void set_depth(int depth) { depth_ = depth < 0 ? 0 : depth; }
    int depth() const { return depth_; }
    // The list is owned by this object and overwritten by the next call.
    const std::vector<uint64_t> &note_access(int layer, uint64_t key) {
        candidates_.clear();
        if (depth_ <= 0) return candidates_;
        const size_t li = static_cast<size_t>(layer < 0 ? 0 : layer);
        if (last_layer_ >= 0 && layer < last_layer_) {
            prev_.swap(cur_);
            for (std::vector<uint64_t> &v : cur_) v.clear();
            valid_ = true;
        }
        if (cur_.size() <= li) cur_.resize(li + 1);
        const bool first_of_layer = cur_[li].empty();
        if (first_of_layer && valid_ && prev_.size() > li) {
            size_t last = li + static_cast<size_t>(depth_);
            if (last > prev_.size()) last = prev_.size();
            for (size_t l = li; l < last; ++l)
                for (uint64_t k : prev_[l])
                    if (k != key) candidates_.push_back(k);
        }
        cur_[li].push_back(key);
        last_layer_ = layer;
        return candidates_;
    }

private:
    int depth_ = 0, last_layer_ = -1;
    bool valid_ = false;
    std::vector<std::vector<uint64_t>> cur_, prev_;
    std::vector<uint64_t> candidates_;
};

}  // namespace wd
