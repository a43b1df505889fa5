// Expert prefetch from the model file: while the layers in front compute, a reader thread fills pinned "shelves" (each
// laid out like a cache slot) with experts that a later acquire will probably ask for, so that the acquire finds the
// bytes in pinned memory and only has to queue the copy to the device.  Same role as the reference's ExpertReadAhead
// with the history that feeds it (src/expert_cache.cuh:547-824, :1094-1127) and the contract of its host test
// (tests/expert_prefetch_host_test.cpp): a shelf is never reused while a copy may still read it, a read that fails
// gives its shelf back and never serves a fill, the same expert is never read twice at once, predictions are the
// previous token's experts.  Host code only: the owner supplies the shelves (pinned memory in the cache, plain memory
// in the host test) and a test that says whether the copy last queued from a shelf has completed.
//
// Division of labour.  All bookkeeping belongs to ONE thread, the owner (the thread that acquires experts): which
// expert sits on which shelf, what may be reused, the counters.  It is plain data without atomics.  The reader thread
// knows nothing of it: it takes read orders (a value type that carries everything the read needs) from a queue, reads,
// and puts a receipt into a second queue; both queues sit behind one mutex and the reader sleeps on a condition
// variable while there is nothing to read.  The owner collects receipts at the start of each of its calls.
//
// A shelf, as the owner sees it: idle -> reading (an order is out) -> shelved (the receipt says the bytes are there)
// -> claimed (an acquire is queueing its copy from it) -> copying (the copy is queued; `copy_done` speaks of it)
// -> idle.  A receipt that reports a failed read returns the shelf to idle at once.  Shelves are reused in this order
// of preference: an idle one; the oldest shelved prediction nobody claimed; the oldest copying shelf whose copy has
// completed.  A reading or claimed shelf is never taken: the reader, or a copy not yet queued, still uses its memory.
#pragma once

#include <unistd.h>

#include <algorithm>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

namespace wd {

constexpr int kPrefetchRuns = 8;  // contiguous runs of one order (gate | up | down of an expert are three)

struct PrefetchRun {
    uint64_t file_off;  // where the run starts in the file
    size_t at;          // where it lands on the shelf
    size_t bytes;
};

class ExpertPrefetcher {
public:
    ExpertPrefetcher() = default;
    ExpertPrefetcher(const ExpertPrefetcher &) = delete;
    ExpertPrefetcher &operator=(const ExpertPrefetcher &) = delete;
    ~ExpertPrefetcher() { stop(); }

    // shelves: one buffer per shelf, each able to hold a slot.  copy_done(shelf): whether the copy that was queued from
    // the shelf when it was last claimed has completed (asked for copying shelves only, on the owner's thread).
    bool start(const std::vector<uint8_t *> &shelves, std::function<bool(int)> copy_done) {
        stop();
        if (shelves.empty()) return false;
        mem_ = shelves;
        copy_done_ = std::move(copy_done);
        const int n = static_cast<int>(mem_.size());
        where_.assign(mem_.size(), Where::kIdle);
        serial_of_.assign(mem_.size(), 0);
        key_of_.assign(mem_.size(), 0);
        for (int s = n - 1; s >= 0; --s) idle_.push_back(s);  // shelf 0 is taken first
        stopping_ = false;
        reader_ = std::thread([this] { read_orders(); });
        return true;
    }
    // Ends the reader (after the read it is in) and forgets every shelf.  The caller makes sure that no copy reads a shelf.
    void stop() {
        if (reader_.joinable()) {
            {
                std::lock_guard<std::mutex> lock(mutex_);
                stopping_ = true;
            }
            wake_.notify_all();
            reader_.join();
        }
        orders_.clear(), receipts_.clear();
        mem_.clear(), where_.clear(), serial_of_.clear(), key_of_.clear();
        idle_.clear(), waiting_.clear(), copying_.clear(), on_shelf_.clear();
        reading_ = 0;
    }
    bool running() const { return !mem_.empty(); }
    size_t shelves() const { return mem_.size(); }

    // Asks for expert `key` to be read: `n` runs of file `fd`.  False when the expert is already being read or shelved,
    // or when no shelf may be reused right now (the caller then goes without a prediction).
    bool request(uint64_t key, int fd, const PrefetchRun *runs, int n) {
        if (!running() || n < 1 || n > kPrefetchRuns) return false;
        collect();
        if (on_shelf_.count(key)) return false;
        const int s = shelf_to_reuse();
        if (s < 0) {
            ++dropped_;
            return false;
        }
        where_[s] = Where::kReading, key_of_[s] = key, serial_of_[s] = ++serial_;
        on_shelf_[key] = s;
        waiting_.push_back(s);
        ++reading_, ++requested_;
        Order o;
        o.shelf = s, o.serial = serial_, o.dst = mem_[s], o.fd = fd, o.n = n;
        std::copy(runs, runs + n, o.runs);
        {
            std::lock_guard<std::mutex> lock(mutex_);
            orders_.push_back(o);
        }
        wake_.notify_one();
        return true;
    }

    // The shelf that holds expert `key`, completely read, or -1.  The caller queues its copy from data(shelf) and then
    // calls copy_queued(shelf); until then the shelf is out of every list and cannot be reused.
    int claim(uint64_t key) {
        if (!running()) return -1;
        collect();
        const auto it = on_shelf_.find(key);
        if (it == on_shelf_.end() || where_[it->second] != Where::kShelved) return -1;
        const int s = it->second;
        on_shelf_.erase(it);
        waiting_.erase(std::find(waiting_.begin(), waiting_.end(), s));
        where_[s] = Where::kClaimed;
        ++claimed_;
        return s;
    }
    uint8_t *data(int shelf) const { return mem_[static_cast<size_t>(shelf)]; }
    void copy_queued(int shelf) {
        if (shelf < 0 || static_cast<size_t>(shelf) >= where_.size() || where_[shelf] != Where::kClaimed) return;
        where_[shelf] = Where::kCopying;
        copying_.push_back(shelf);
    }

    // (each of these first collects the reader's receipts)
    bool busy() {
        collect();
        return reading_ != 0;
    }
    uint64_t delivered() {
        collect();
        return delivered_;
    }
    uint64_t failed() {
        collect();
        return failed_;
    }
    uint64_t requested() const { return requested_; }
    uint64_t dropped() const { return dropped_; }
    uint64_t claimed() const { return claimed_; }
    uint64_t unused() const { return unused_; }  // shelved predictions that were overwritten unclaimed

private:
    enum class Where : uint8_t { kIdle, kReading, kShelved, kClaimed, kCopying };
    struct Order {  // everything a read needs, by value
        int shelf = -1, fd = -1, n = 0;
        uint64_t serial = 0;
        uint8_t *dst = nullptr;
        PrefetchRun runs[kPrefetchRuns] = {};
    };
    struct Receipt {
        int shelf;
        uint64_t serial;
        bool ok;
    };

    // ---- reader thread
    void read_orders() {
        std::unique_lock<std::mutex> lock(mutex_);
        for (;;) {
            wake_.wait(lock, [this] { return stopping_ || !orders_.empty(); });
            if (stopping_) return;
            const Order o = orders_.front();
            orders_.pop_front();
            lock.unlock();
            const bool ok = read_runs(o);
            lock.lock();
            receipts_.push_back({o.shelf, o.serial, ok});
        }
    }
    static bool read_runs(const Order &o) {
        if (o.fd < 0) return false;
        for (int i = 0; i < o.n; ++i) {
            const PrefetchRun &r = o.runs[i];
            for (size_t got = 0; got < r.bytes;) {
                const ssize_t n = ::pread(o.fd, o.dst + r.at + got, r.bytes - got, static_cast<off_t>(r.file_off + got));
                if (n <= 0) return false;  // end of file or an error: the order fails as a whole
                got += static_cast<size_t>(n);
            }
        }
        return true;
    }

    // ---- owner thread
    void collect() {
        std::deque<Receipt> got;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            got.swap(receipts_);
        }
        for (const Receipt &r : got) {
            const size_t s = static_cast<size_t>(r.shelf);
            if (s >= where_.size() || where_[s] != Where::kReading || serial_of_[s] != r.serial) continue;  // (a stale receipt)
            --reading_;
            if (r.ok) {
                where_[s] = Where::kShelved;
                ++delivered_;
            } else {
                ++failed_;
                on_shelf_.erase(key_of_[s]);
                waiting_.erase(std::find(waiting_.begin(), waiting_.end(), r.shelf));
                where_[s] = Where::kIdle;
                idle_.push_back(r.shelf);
            }
        }
    }
    int shelf_to_reuse() {
        if (!idle_.empty()) {
            const int s = idle_.back();
            idle_.pop_back();
            return s;
        }
        for (auto it = waiting_.begin(); it != waiting_.end(); ++it) {  // oldest request first
            if (where_[*it] != Where::kShelved) continue;
            const int s = *it;
            waiting_.erase(it);
            on_shelf_.erase(key_of_[s]);
            ++unused_;
            return s;
        }
        for (auto it = copying_.begin(); it != copying_.end(); ++it) {  // oldest copy first
            if (copy_done_ && !copy_done_(*it)) continue;
            const int s = *it;
            copying_.erase(it);
            return s;
        }
        return -1;
    }

    // owner's data
    std::vector<uint8_t *> mem_;
    std::function<bool(int)> copy_done_;
    std::vector<Where> where_;
    std::vector<uint64_t> serial_of_, key_of_;
    std::vector<int> idle_;
    std::deque<int> waiting_;                      // shelves reading or shelved, in the order they were requested
    std::deque<int> copying_;                      // shelves whose copy is queued, in that order
    std::unordered_map<uint64_t, int> on_shelf_;   // expert -> shelf, for reading and shelved shelves
    uint64_t serial_ = 0, reading_ = 0;
    uint64_t requested_ = 0, dropped_ = 0, claimed_ = 0, unused_ = 0, delivered_ = 0, failed_ = 0;
    // shared with the reader, behind mutex_
    std::mutex mutex_;
    std::condition_variable wake_;
    std::deque<Order> orders_;
    std::deque<Receipt> receipts_;
    bool stopping_ = false;
    std::thread reader_;
};

// What to ask the prefetcher for.  The acquires of a token arrive layer by layer; a layer number that goes down says
// that a new token has begun.  The experts a token used are kept in a flat table [layer][kPlanWidth]; at a layer's
// first acquire of a token the plan is what the token before used in this layer and the `depth - 1` layers after it,
// without the expert that is being acquired at this moment (src/expert_cache.cuh:1094-1127).
constexpr int kPlanWidth = 16;  // experts kept per layer and token (top-k is at most 16)

class PrefetchPlanner {
public:
    void set_depth(int depth) { depth_ = std::max(depth, 0); }
    int depth() const { return depth_; }

    // Records the acquire of `key` in `layer`; returns the experts to request now (valid until the next call).
    const std::vector<uint64_t> &on_acquire(int layer, uint64_t key) {
        plan_.clear();
        if (depth_ == 0) return plan_;
        const size_t l = static_cast<size_t>(std::max(layer, 0));
        if (layer < newest_layer_) {  // a new token: its table becomes the one to predict from
            now_ ^= 1;
            std::fill(count_[now_].begin(), count_[now_].end(), 0);
            have_previous_ = true;
        }
        newest_layer_ = layer;
        grow(l + 1);
        if (count_[now_][l] == 0 && have_previous_) {
            const int before = now_ ^ 1;
            const size_t end = std::min(l + static_cast<size_t>(depth_), count_[before].size());
            for (size_t q = l; q < end; ++q)
                for (int i = 0; i < std::min(count_[before][q], kPlanWidth); ++i) {
                    const uint64_t k = used_[before][q * kPlanWidth + static_cast<size_t>(i)];
                    if (k != key) plan_.push_back(k);
                }
        }
        int &n = count_[now_][l];
        if (n < kPlanWidth) used_[now_][l * kPlanWidth + static_cast<size_t>(n)] = key;
        ++n;  // (counts past the width still say "not the first acquire of the layer")
        return plan_;
    }

private:
    void grow(size_t layers) {
        for (int t = 0; t < 2; ++t)
            if (count_[t].size() < layers) {
                count_[t].resize(layers, 0);
                used_[t].resize(layers * kPlanWidth, 0);
            }
    }
    int depth_ = 0, newest_layer_ = -1, now_ = 0;
    bool have_previous_ = false;
    std::vector<int> count_[2];
    std::vector<uint64_t> used_[2];
    std::vector<uint64_t> plan_;
};

}  // namespace wd
