// Site profiler of the MoE path: event brackets around the library's own dispatches and around regions a caller
// names, accumulated per decode token into device time, host time and their gap.  Same purpose and report as the
// reference's Q38MoeKernelProfiler / Q38MoeKernelScope (src/qwen38_moe.cuh:296-535); the sites that exist in both
// keep the reference's numbers and names, the dispatches that only exist here (the merged launch, the down+combine
// launch, the one-launch stack, the multi-token pass, the cache fills) follow them.
//
// Off (the default) every hook is one relaxed load and a branch.  On, a bracket records a HIP event on the caller's
// stream at either end - never on a stream that is being captured, where an event would become a graph node and its
// time could not be read: such brackets count as dropped.
#pragma once

#include <atomic>
#include <chrono>
#include <mutex>
#include <string>
#include <vector>

#include "wd_common.h"

namespace wd {

// names by site number; the first WD_PROFILE_FIRST_OWN_SITE are the reference's (q38_moe_site_name)
inline const char *profile_site_name(int site) {
    static const char *const names[WD_PROFILE_SITE_COUNT] = {
        "moe.stage_total",     "moe.routed_total",    "moe.router_select",  "moe.router.act_quant", "moe.router.gemv",
        "moe.router.topk",     "moe.router.d2h",      "moe.router.sync",    "moe.accum_zero",       "moe.rx_quant",
        "moe.acquire",         "moe.ptr_h2d",         "moe.batch_total",    "moe.batch.gate_up",    "moe.batch.silu",
        "moe.batch.q8_quant",  "moe.batch.down",      "moe.batch.accum",    "moe.batch.capture",    "moe.loop_total",
        "moe.finish",          "moe.shared",          "moe.shared.gate",    "moe.mirror",
        // dispatches of this library
        "moe.fused.ab",        "moe.fused.a",         "moe.fused.b",        "moe.fused.c",          "moe.stack_total",
        "moe.stack.resident",  "moe.cache.fill",      "moe.tokens_total",   "moe.tokens.a",         "moe.tokens.b",
        "moe.tokens.c",        "moe.hc_combine"};
    return site >= 0 && site < WD_PROFILE_SITE_COUNT ? names[site] : "unknown";
}

class SiteProfiler {
public:
    // a token has at most 64 layers here and a site fires at most once per layer (twice for the cache's fills with a
    // token acquired ahead): 160 brackets per site and token, the rest is reported as dropped
    static constexpr int kCap = 160;

    static SiteProfiler &instance() {
        static SiteProfiler p;
        return p;
    }
    bool enabled() const { return enabled_.load(std::memory_order_relaxed); }

    int enable(bool on) {
        std::lock_guard<std::mutex> g(mu_);
        if (on && start_.empty()) {
            start_.assign(static_cast<size_t>(WD_PROFILE_SITE_COUNT) * kCap, nullptr);
            stop_.assign(start_.size(), nullptr);
            for (size_t i = 0; i < start_.size(); ++i) {
                if (hipEventCreate(&start_[i]) != hipSuccess || hipEventCreate(&stop_[i]) != hipSuccess) {
                    release_events();
                    return fail(WD_ERR_HIP, "profiler: hipEventCreate failed after %zu events", 2 * i);
                }
            }
        }
        if (on != enabled())
            for (Live &l : live_) l.depth = 0, l.armed = false;  // a bracket cut in two by the switch is forgotten
        enabled_.store(on, std::memory_order_relaxed);
        return WD_OK;
    }

    void begin(int site, hipStream_t st) {
        if (!enabled() || site < 0 || site >= WD_PROFILE_SITE_COUNT) return;
        std::lock_guard<std::mutex> g(mu_);
        Live &l = live_[site];
        if (l.depth++ != 0) return;  // a nested bracket of the same site stays one interval
        l.host_begin = std::chrono::steady_clock::now();
        l.armed = false;
        if (l.written >= kCap || capturing(st) || !record(start_[index(site, l.written)], st)) {
            ++l.dropped;
            return;
        }
        l.armed = true;
    }

    void end(int site, hipStream_t st) {
        if (!enabled() || site < 0 || site >= WD_PROFILE_SITE_COUNT) return;
        std::lock_guard<std::mutex> g(mu_);
        Live &l = live_[site];
        if (l.depth <= 0 || --l.depth != 0) return;
        l.host_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - l.host_begin).count();
        if (!l.armed) return;  // counted as dropped when it began
        l.armed = false;
        if (capturing(st) || !record(stop_[index(site, l.written)], st)) {
            ++l.dropped;
            return;
        }
        ++l.written;
    }

    // once per token, after the caller has synchronised the streams it bracketed: every event has completed then
    int flush_token() {
        if (!enabled()) return WD_OK;
        std::lock_guard<std::mutex> g(mu_);
        for (int s = 0; s < WD_PROFILE_SITE_COUNT; ++s) {
            Live &l = live_[s];
            wd_profile_site_stat &t = stats_[s];
            for (int i = 0; i < l.written; ++i) {
                float ms = 0.0f;
                if (hipEventElapsedTime(&ms, start_[index(s, i)], stop_[index(s, i)]) == hipSuccess) {
                    t.device_ms += ms;
                    ++t.calls;
                } else {
                    ++t.unreadable;
                }
            }
            (void)hipGetLastError();  // an unreadable pair must not surface in the caller's next launch check
            t.recorded += static_cast<unsigned long long>(l.written);
            t.host_ms += l.host_ms;
            t.dropped += static_cast<unsigned long long>(l.dropped);
            l = Live{};
        }
        ++tokens_;
        return WD_OK;
    }

    void reset() {
        std::lock_guard<std::mutex> g(mu_);
        for (int s = 0; s < WD_PROFILE_SITE_COUNT; ++s) live_[s] = Live{}, stats_[s] = wd_profile_site_stat{};
        tokens_ = 0;
    }

    unsigned long long tokens() const { return tokens_; }
    wd_profile_site_stat stat(int site) {
        std::lock_guard<std::mutex> g(mu_);
        return stats_[site];
    }

    // one line per site that saw anything, per token: device ms, host ms, host - device, brackets per token, and the
    // three counts that tell "never ran", "never closed / no room" and "events not readable" apart
    std::string report() {
        std::lock_guard<std::mutex> g(mu_);
        char line[256];
        std::snprintf(line, sizeof(line), "[moe-profile] tokens=%llu unit=ms_per_token\n", tokens_);
        std::string out = line;
        const double div = tokens_ ? static_cast<double>(tokens_) : 1.0;
        for (int s = 0; s < WD_PROFILE_SITE_COUNT; ++s) {
            const wd_profile_site_stat &t = stats_[s];
            if (t.recorded == 0 && t.dropped == 0 && t.unreadable == 0 && t.host_ms == 0.0) continue;
            std::snprintf(line, sizeof(line),
                          "[moe-profile] %-20s dev=%9.4f host=%9.4f gap=%9.4f calls/token=%.2f recorded=%llu dropped=%llu evfail=%llu\n",
                          profile_site_name(s), t.device_ms / div, t.host_ms / div, (t.host_ms - t.device_ms) / div,
                          static_cast<double>(t.calls) / div, t.recorded, t.dropped, t.unreadable);
            out += line;
        }
        return out;
    }

private:
    struct Live {
        int depth = 0, written = 0, dropped = 0;
        bool armed = false;
        double host_ms = 0.0;
        std::chrono::steady_clock::time_point host_begin{};
    };
    SiteProfiler() = default;
    ~SiteProfiler() = default;  // the events live as long as the process: the runtime may be gone when statics die
    SiteProfiler(const SiteProfiler &) = delete;
    SiteProfiler &operator=(const SiteProfiler &) = delete;

    static size_t index(int site, int slot) { return static_cast<size_t>(site) * kCap + static_cast<size_t>(slot); }
    static bool capturing(hipStream_t st) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
            (void)hipGetLastError();  // (the legacy stream while another stream captures): not the caller's next launch's error
            return true;
        }
        return cs != hipStreamCaptureStatusNone;
    }
    static bool record(hipEvent_t ev, hipStream_t st) {
        if (hipEventRecord(ev, st) == hipSuccess) return true;
        (void)hipGetLastError();
        return false;
    }
    void release_events() {
        for (hipEvent_t e : start_)
            if (e) (void)hipEventDestroy(e);
        for (hipEvent_t e : stop_)
            if (e) (void)hipEventDestroy(e);
        start_.clear(), stop_.clear();
    }

    std::atomic<bool> enabled_{false};
    std::mutex mu_;
    std::vector<hipEvent_t> start_, stop_;
    Live live_[WD_PROFILE_SITE_COUNT];
    wd_profile_site_stat stats_[WD_PROFILE_SITE_COUNT] = {};
    unsigned long long tokens_ = 0;
};

// bracket of one region, closed when the scope ends (also on an early return)
class SiteScope {
public:
    SiteScope(int site, hipStream_t st) : site_(site), st_(st), on_(SiteProfiler::instance().enabled()) {
        if (on_) SiteProfiler::instance().begin(site_, st_);
    }
    ~SiteScope() {
        if (on_) SiteProfiler::instance().end(site_, st_);
    }
    SiteScope(const SiteScope &) = delete;
    SiteScope &operator=(const SiteScope &) = delete;

private:
    int site_;
    hipStream_t st_;
    bool on_;
};

}  // namespace wd
