// A whole stack of MoE layers in ONE launch: 512 resident workgroups walk the layers together.
//
// The per-layer dispatches (wd_fused.cuh) pay two launches per layer and fetch every weight only after the value it is
// multiplied with exists.  Here the workgroups stay on their compute units for the whole decode step, so
//   * no launch lies between two dependent stages - values are handed from workgroup to workgroup through small
//     buffers in global memory whose words say themselves whether they have been written (see below);
//   * weights that do not depend on a value still being computed are already on the compute unit when that value
//     arrives: the router row and the shared expert's rows of layer l + 1 are fetched during layer l, and the routed
//     down rows are requested together with the routed gate/up rows, as soon as the expert ids are known.
//
// Geometry (the C2 layer shape): hidden 2048, expert ffn 512, at most 512 experts, top-k <= 10, IQ3_S or IQ2_S gate/up,
// Q8_0 down, Q8_0 shared expert.  Workgroup r (0..511) has 12 waves:
//   waves 0..9   routed rung j = wave: row r of gate and up of expert ids[j], then rows 4r..4r+3 of its down tensor
//   wave 10      the shared expert: row r of its gate/up, rows 4r..4r+3 of its down tensor
//   wave 11      router row r
// and wave 0 folds the eleven results of rows 4r..4r+3 in the reference order and publishes these four values of the
// next layer's input.  Workgroup 0 also selects the experts (its waves are idle until the ids exist anyway).
// The float operations and their order are those of the per-layer kernels: results are bit-identical.
//
// Hand-off buffers.  Every layer of a launch has its own copy of each buffer, so no word is written twice during a
// launch.  A word holds kResEmpty (0xffffffff) until its producer stores the value; consumers poll the data words
// themselves with device-scope loads, so no flag, counter or ordering between stores is needed.  What a workgroup
// hands on in a layer: its logit, in a 16-byte record that only workgroup 0 polls (64 lines for the 512 logits); its
// eleven activations (48 bytes) and its four values of the next input (16 bytes), pushed into eight contiguous
// copies, one per group of workgroups, each of which polls its own.  A line that many compute units write piece
// by piece while the whole grid polls it changes hands once per write: thirty-two writers per line made a hand-off
// take 17 us, hence pieces of 16 bytes or more.  (An f32 result with
// that very bit pattern - a NaN that no arithmetic here produces by itself - would be taken for "not yet" and end in
// a timeout.)  There are two sets of these buffers: a launch works in one and resets the other as it goes (the router
// waves, which have time to spare), so nothing has to be cleaned up when a launch ends.  Waits are bounded: a wait that runs out sets status[0], after which
// every wait in the grid ends at once and later launches return immediately until the scratch is reset.
#pragma once

#include "wd_fused.cuh"

namespace wd {

#ifndef WD_RES_SLEEP4
#define WD_RES_SLEEP4 2
#endif
#ifndef WD_RES_XDELAY
#define WD_RES_XDELAY 24
#endif
#ifndef WD_RES_SLEEP16
#define WD_RES_SLEEP16 2
#endif
constexpr int kResMaxLayers = 64;
constexpr int kResWgs = 512, kResWaves = 12, kResThreads = kResWaves * 64;
constexpr int kResH = 2048, kResF = 512, kResMaxK = 10, kResSharedSlot = 10, kResActSlots = 11;
constexpr uint32_t kResEmpty = 0xffffffffu;
constexpr int kResIdCopies = 16;   // replicas of the published ids (pollers spread over lines)
constexpr int kResXtRow = 68;      // floats per row of the transposed input in LDS (64 + bank spread)
constexpr int kResGateSlot = 15;   // word of the weights record that holds the shared expert's sigmoid gate

struct ResidentLayer {
    const float *router;      // f32 [E][2048]
    const float *sh_inp;      // f32 [2048] or null (no shared expert)
    const uint8_t *sh_gate, *sh_up, *sh_down;
    const uint8_t *gate, *up, *down;
    size_t gate_stride, up_stride, down_stride;
    float w_scale;
    int pad_;
};

// The last layer's values, as the per-layer path leaves them in the scratch.
struct ResidentViews {
    float *logits, *weights, *accum, *down_f32, *shared_gate;
    int32_t *ids;
};

// Byte offsets inside the hand-off block.
constexpr unsigned kHandRec = 0;          // [layers][512] records of kRecBytes, one per (layer, workgroup): word 0 the router
// (Measured on one box: records of 128 / 64 / 32 / 16 bytes 0.869 / 0.861 / 0.856 / 0.851 ms per token - workgroup 0 polls
// 64 lines instead of 512; the gate logit moved into the line of the router weights, which every workgroup polls, costs
// 1.2 % again, and records of 8 bytes are no better than 16.)
constexpr unsigned kRecBytes = 16;        //   logit of row r, word 1 the shared expert's gate logit (workgroup 1 only)
static_assert(kRecBytes % 16 == 0 && kRecBytes <= 128, "records are reset in 16-byte pieces by eight lanes");
// What every workgroup needs from every other - four values of the next input, eleven activations - is written by its
// producer into kResCopies copies, one per group of workgroups (r % kResCopies; on this device the workgroups of a group
// share an L2), laid out contiguously: the consumers of a group fetch their copy with coalesced requests, and a line is
// polled from one L2 only.
constexpr int kResCopies = 8;
#ifndef WD_RES_XSTRIDE
#define WD_RES_XSTRIDE 16
#endif
constexpr unsigned kXcStride = WD_RES_XSTRIDE;  // bytes from one workgroup's four values of a layer input to the next one's
constexpr unsigned kXcBytes = kXcStride * kResWgs;                                     // one copy
constexpr unsigned kHandXc = kHandRec + kRecBytes * kResMaxLayers * kResWgs;           // [layers][copies][512] pieces of four f32: layer inputs
constexpr unsigned kAcRec = 48;                                                        // bytes of a workgroup's activations: slots 0..10, a zero
constexpr unsigned kAcBytes = kAcRec * kResWgs;                                        // 24 KB per copy
constexpr unsigned kHandAc = kHandXc + kXcBytes * kResMaxLayers * kResCopies;        // f32 [layers][copies][512][12] activations
constexpr unsigned kHandIdh = kHandAc + kAcBytes * kResMaxLayers * kResCopies;         // u32 [layers][copies][16] selected ids
constexpr unsigned kHandWh = kHandIdh + 4u * kResMaxLayers * kResIdCopies * 16;  // u32 [layers][16] router weights, [15] the shared gate
constexpr unsigned kHandSet = kHandWh + 4u * kResMaxLayers * 16;             // bytes of one set of hand-off buffers
// The block holds two such sets and the number of launches finished.  Launch e works in set e % 2 and, layer by layer and
// off its critical path, puts set (e + 1) % 2 back to "not yet written": no launch has to clean up behind itself.
constexpr unsigned kHandEpoch = 2u * kHandSet;
constexpr unsigned kHandBytes = kHandEpoch + 256u;
static_assert(kHandXc % 128 == 0 && kHandAc % 128 == 0 && kHandIdh % 128 == 0 && kHandWh % 16 == 0 && kHandSet % 128 == 0, "hand-off block alignment");
WD_DEV unsigned rec_off(int l, int wg) { return kHandRec + static_cast<unsigned>(l * kResWgs + wg) * kRecBytes; }
WD_DEV unsigned xc_off(int l, int copy) { return kHandXc + static_cast<unsigned>(l * kResCopies + copy) * kXcBytes; }
WD_DEV unsigned ac_off(int l, int copy) { return kHandAc + static_cast<unsigned>(l * kResCopies + copy) * kAcBytes; }

struct ResidentArgs {
    const ResidentLayer *layers;  // device array [n_layers]
    int n_layers, E, k;
    int shared;                   // every layer has a shared expert (1) or none has (0)
    size_t gate_stride, up_stride, down_stride;  // bytes per expert, the same in every layer
    float *x;                     // [2048] in: input of the first layer; out: input of the layer after the last
    float *out;                   // [2048] output of the last layer
    float residual_scale;
    const int32_t *ids_trace;     // null, or [n_layers][k]: ids that replace the selected ones (the weights stay the router's)
    const struct ResidentViews *views;  // device: where the last layer's values go
    uint8_t *hand;   // the hand-off block (kHand* offsets below)
    unsigned *status;
    unsigned spin_limit;
    unsigned long long *trace;  // null, or [12][16] time stamps (100 MHz) of workgroup trace_wg in layer trace_layer
    int trace_wg, trace_layer;
    int debug;  // experiments: 1 no gate/up decode, 2 no weight loads, 4 no wait for the activations, 8 no down dots.
                // (The tests of these bits stay in the kernel on purpose: as branches around the weight requests and the
                // dot products they keep the compiler from moving these against each other - the down rows' request in
                // particular must follow the gate/up rows' arrival -, and the kernel measured 5 % slower without them.)
};

// ---- device-scope access to the hand-off buffers ------------------------------------------------------------
typedef unsigned wd_u4v __attribute__((ext_vector_type(4)));
constexpr int kAuxDevice = 16;  // sc1: the access is coherent across the device's L2 caches
constexpr int kAuxPoll = static_cast<int>(0x80000010u);  // the same, volatile: two polls of one address are two requests
WD_DEV __amdgpu_buffer_rsrc_t hand_rsrc(const void *p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, static_cast<int>(bytes), 0x00020000);
}
WD_DEV uint4 hand_load16(__amdgpu_buffer_rsrc_t rs, unsigned off) {
    const wd_u4v v = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<int>(off), 0, kAuxPoll);
    return make_uint4(v.x, v.y, v.z, v.w);
}
WD_DEV uint32_t hand_load4(__amdgpu_buffer_rsrc_t rs, unsigned off) {
    return __builtin_amdgcn_raw_buffer_load_b32(rs, static_cast<int>(off), 0, kAuxPoll);
}
WD_DEV void hand_store16(__amdgpu_buffer_rsrc_t rs, unsigned off, uint4 v) {
    const wd_u4v w = {v.x, v.y, v.z, v.w};
    __builtin_amdgcn_raw_buffer_store_b128(w, rs, static_cast<int>(off), 0, kAuxDevice);
}
WD_DEV void hand_store4(__amdgpu_buffer_rsrc_t rs, unsigned off, uint32_t v) {
    __builtin_amdgcn_raw_buffer_store_b32(v, rs, static_cast<int>(off), 0, kAuxDevice);
}

// ---- bounded waits ------------------------------------------------------------------------------------------------
// `dead`: a wait ran out somewhere in the grid; every further wait then returns at once (with whatever it holds).
// One unsuccessful poll more; true when the wait has to end.
WD_DEV bool res_give_up(const ResidentArgs &a, unsigned &spins, bool &dead) {
    ++spins;
    if (spins >= a.spin_limit) {
        __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        dead = true;
    } else if ((spins & 63u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
        dead = true;
    }
    return dead;
}
WD_DEV bool res_full(const uint4 &v) { return v.x != kResEmpty && v.y != kResEmpty && v.z != kResEmpty && v.w != kResEmpty; }

// N 16-byte pieces per lane (lanes with on == false take no part): returns when every word of every piece has been
// written.  Only pieces that are still incomplete are requested again.
// WD_RES_PIPE16 / WD_RES_PIPE4 > 1: that many polls are kept in flight.  A poll that has to travel to memory and back
// before the next one is issued notices a value up to one round trip late; several polls under way notice it within the
// interval at which they were issued.
#ifndef WD_RES_DOWN_AT
#define WD_RES_DOWN_AT 0  // the down rows are requested 0: when the gate/up rows have arrived, 1: after the decode, 2: after the exchange
#endif
#ifndef WD_RES_PIPE16
#define WD_RES_PIPE16 1
#endif
#ifndef WD_RES_PIPE4
#define WD_RES_PIPE4 1
#endif
#ifndef WD_RES_PIPE16_MAXN
#define WD_RES_PIPE16_MAXN 1
#endif
template <int N, int D>
WD_DEV void hand_wait16_piped(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, const unsigned (&off)[N], const bool (&on)[N], uint4 (&v)[N], bool &dead) {
    static_assert(D == 2, "two polls in flight");
    bool need[N];
    uint4 p0[N], p1[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        need[i] = on[i];
        v[i] = p0[i] = p1[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (dead) return;
    auto issue = [&](uint4 (&p)[N]) {
#pragma unroll
        for (int i = 0; i < N; ++i)
            if (need[i]) p[i] = hand_load16(rs, off[i]);
    };
    auto arrived = [&](const uint4 (&p)[N]) {  // true when nothing is missing any more (or the wait is given up)
        bool any = false;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            if (need[i]) {
                v[i] = p[i];
                need[i] = !res_full(v[i]);
            }
            any = any || need[i];
        }
        return __builtin_amdgcn_ballot_w64(any) == 0ull;
    };
    issue(p0);
    __builtin_amdgcn_s_sleep(WD_RES_SLEEP16);
    issue(p1);
    unsigned spins = 0;
    for (;;) {
        if (arrived(p0) || res_give_up(a, spins, dead)) return;
        issue(p0);
        __builtin_amdgcn_s_sleep(WD_RES_SLEEP16);
        if (arrived(p1) || res_give_up(a, spins, dead)) return;
        issue(p1);
        __builtin_amdgcn_s_sleep(WD_RES_SLEEP16);
    }
}
template <int D>
WD_DEV uint32_t hand_wait4_piped(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, unsigned off, bool on, bool &dead) {
    uint32_t v = 0u;
    if (dead) return v;
    bool need = on;
    uint32_t s[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        s[d] = 0u;
        if (need) s[d] = hand_load4(rs, off);
        if (d + 1 < D) __builtin_amdgcn_s_sleep(WD_RES_SLEEP4);
    }
    unsigned spins = 0;
    bool done = false;
    while (!done) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (!done) {
                if (need) {
                    v = s[d];
                    need = v == kResEmpty;
                }
                done = __builtin_amdgcn_ballot_w64(need) == 0ull || res_give_up(a, spins, dead);
                if (!done) {
                    if (need) s[d] = hand_load4(rs, off);
                    __builtin_amdgcn_s_sleep(WD_RES_SLEEP4);
                }
            }
        }
    }
    return v;
}
template <int N>
WD_DEV void hand_wait16(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, const unsigned (&off)[N], const bool (&on)[N], uint4 (&v)[N], bool &dead) {
    if constexpr (WD_RES_PIPE16 > 1 && N <= WD_RES_PIPE16_MAXN) {
        hand_wait16_piped<N, WD_RES_PIPE16>(a, rs, off, on, v, dead);
        return;
    }
    bool need[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        need[i] = on[i];
        v[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (dead) return;
    unsigned spins = 0;
    for (;;) {
        bool any = false;
#pragma unroll
        for (int i = 0; i < N; ++i)
            if (need[i]) v[i] = hand_load16(rs, off[i]);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            need[i] = need[i] && !res_full(v[i]);
            any = any || need[i];
        }
        if (__builtin_amdgcn_ballot_w64(any) == 0ull) return;
        if (res_give_up(a, spins, dead)) return;
        __builtin_amdgcn_s_sleep(WD_RES_SLEEP16);
    }
}
template <int N>
WD_DEV void hand_wait16(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, const unsigned (&off)[N], bool on, uint4 (&v)[N], bool &dead) {
    bool each[N];
#pragma unroll
    for (int i = 0; i < N; ++i) each[i] = on;
    hand_wait16<N>(a, rs, off, each, v, dead);
}
// One word per lane.
WD_DEV uint32_t hand_wait4(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, unsigned off, bool on, bool &dead) {
    if constexpr (WD_RES_PIPE4 > 1) return hand_wait4_piped<WD_RES_PIPE4>(a, rs, off, on, dead);
    uint32_t v = 0u;
    if (dead) return v;
    bool need = on;
    unsigned spins = 0;
    for (;;) {
        if (need) v = hand_load4(rs, off);
        need = need && v == kResEmpty;
        if (__builtin_amdgcn_ballot_w64(need) == 0ull) return v;
        if (res_give_up(a, spins, dead)) return v;
        __builtin_amdgcn_s_sleep(WD_RES_SLEEP4);
    }
}

// ---- router row of 2048 columns, weights fetched ahead --------------------------------------------------------
// Accumulator t of ggml's 4 x 8 scheme lives in lanes t and t + 32 (router_rows_wave): lane t runs the multiply-adds
// of columns t, t + 32, ... below 1024 and hands the value to lane t + 32, which continues with the upper half.
WD_DEV void res_router_fetch(const float *__restrict__ row, float (&wv)[32], int lane) {
    const float *p = uniform_ptr(row) + ((lane >= 32) ? 1024 : 0) + (lane & 31);
#pragma unroll
    for (int u = 0; u < 32; ++u) wv[u] = p[32 * u];
}
// The row's dot product with the input (LDS, transposed: xt[t][v] = x[32 v + t], rows of kResXtRow floats); valid in lane 32.
WD_DEV float res_router_dot(const float (&wv)[32], const float *xt, int lane) {
    const int t = lane & 31;
    const bool upper = lane >= 32;
    const float4 *xp = reinterpret_cast<const float4 *>(xt + t * kResXtRow + (upper ? 32 : 0));
    float4 xv[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) xv[q] = xp[q];
    auto run_half = [&](float start) {
        float v = start;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            v = __builtin_fmaf(wv[4 * q + 0], xv[q].x, v);
            v = __builtin_fmaf(wv[4 * q + 1], xv[q].y, v);
            v = __builtin_fmaf(wv[4 * q + 2], xv[q].z, v);
            v = __builtin_fmaf(wv[4 * q + 3], xv[q].w, v);
        }
        return v;
    };
    float s = 0.0f;
    if (!upper) s = run_half(0.0f);
    const wd_uint2v fwd = __builtin_amdgcn_permlane32_swap(f_bits(s), f_bits(s), false, false);
    if (upper) s = run_half(bits_f(fwd.x));
    // the 32 accumulators are final in the upper half: ggml's closing tree
    float o = __shfl_down(s, 16, 32);
    if (t < 16) s = s + o;
    o = __shfl_down(s, 8, 32);
    if (t < 8) s = s + o;
    o = __shfl_down(s, 4, 32);
    if (t < 4) s = s + o;
    o = __shfl_down(s, 1, 32);
    if (t == 0 || t == 2) s = s + o;
    o = __shfl_down(s, 2, 32);
    return s + o;
}

// ---- LDS layout -----------------------------------------------------------------------------------------------
constexpr int kResLdsXs = 0;                                  // f32 [32][68] layer input, xt[t][v] = x[32 v + t]: the 64 values that
                                                              //   accumulator t of a router row meets are contiguous
constexpr int kResLdsXq = kResLdsXs + 4 * 32 * kResXtRow;     // int8 [2048] its Q8_K quants
constexpr int kResLdsXd = kResLdsXq + kResH;                  // f32 [8] Q8_K scales
constexpr int kResLdsX0q = kResLdsXd + 32;                    // int8 [2048] its Q8_0 quants
constexpr int kResLdsX0d = kResLdsX0q + kResH;                // f16 [64] Q8_0 scales
constexpr int kResLdsTables = kResLdsX0d + 128;               // IqTables
constexpr int kResLdsWave = kResLdsTables + static_cast<int>(sizeof(IqTables));  // per slot 0..10: tile/stage, then aq, ad
constexpr int kResTileBytes = static_cast<int>(sizeof(Q8TileNB<16>));
constexpr int kResWaveBytes = kResTileBytes + kResF + 64;
constexpr int kResLdsY = kResLdsWave + kResActSlots * kResWaveBytes;  // f32 [11][4] down results
constexpr int kResLdsSel = kResLdsY + 4 * 4 * kResActSlots;           // selection scratch, then ids [16], weights [16]
constexpr int kResLdsRoles = kResLdsSel + kTopkLdsBytes1 + 128;       // int [12] SIMD of every wave
constexpr int kResLdsActv = kResLdsRoles + 64;                        // f32 [12] this workgroup's activations (word 11 zero)
constexpr int kResLdsBytes = kResLdsActv + 64;
constexpr int kResLdsLand = kResLdsWave;  // f32 [11][512] all activations of the layer, while no slot area is in use
static_assert(kResLdsXq % 16 == 0 && kResLdsTables % 16 == 0 && kResLdsWave % 16 == 0 && kResWaveBytes % 16 == 0 && kResLdsSel % 16 == 0, "LDS alignment");
static_assert(sizeof(Q8RowTile) <= sizeof(Q8TileNB<16>) && 2 * kIqStageBytes <= kResTileBytes, "a slot's area serves every stage");
static_assert(kResLdsBytes <= 65536, "LDS of the resident stack kernel");
static_assert(4 * kResActSlots * 512 <= kResActSlots * kResWaveBytes, "the activations land in the slot areas");

// Values the optimiser must take as new in every layer: without them it computes hundreds of per-lane addresses once,
// ahead of the layer loop, and keeps them in registers (which then spill) instead of recomputing a handful per layer.
WD_DEV int fresh_v(int v) {
    asm volatile("" : "+v"(v));
    return v;
}
WD_DEV int fresh_s(int v) {  // v is the same in every lane
    v = __builtin_amdgcn_readfirstlane(v);
    asm volatile("" : "+s"(v));
    return v;
}

// What a wave is and where it works.  slot: 0..9 routed rung, 10 the shared expert; -1 for the router wave.
struct ResCtx {
    uint8_t *lds;
    int r, lane, wave, slot;
    __amdgpu_buffer_rsrc_t hb;  // the hand-off block
    WD_DEV float *xt() const { return reinterpret_cast<float *>(lds + kResLdsXs); }
    WD_DEV float x_at(int e) const { return xt()[(e & 31) * kResXtRow + (e >> 5)]; }
    WD_DEV int8_t *xq() const { return reinterpret_cast<int8_t *>(lds + kResLdsXq); }
    WD_DEV float *xd() const { return reinterpret_cast<float *>(lds + kResLdsXd); }
    WD_DEV int8_t *x0q() const { return reinterpret_cast<int8_t *>(lds + kResLdsX0q); }
    WD_DEV uint16_t *x0d() const { return reinterpret_cast<uint16_t *>(lds + kResLdsX0d); }
    WD_DEV uint8_t *area() const { return lds + kResLdsWave + slot * kResWaveBytes; }
    WD_DEV float *ybuf() const { return reinterpret_cast<float *>(lds + kResLdsY); }
    WD_DEV float *actv() const { return reinterpret_cast<float *>(lds + kResLdsActv); }
    WD_DEV float *land() const { return reinterpret_cast<float *>(lds + kResLdsLand); }
};
// The context of one layer: the indices made opaque (see fresh_v); `base` is the workgroup's dynamic LDS.
WD_DEV ResCtx res_ctx(uint8_t *base, int r, int lane, int wave, int slot, __amdgpu_buffer_rsrc_t hb) {
    ResCtx c;
    c.lds = base + fresh_s(0);
    c.r = fresh_s(r), c.lane = fresh_v(lane), c.wave = fresh_s(wave), c.slot = fresh_s(slot);
    c.hb = hb;
    return c;
}
// Time stamp i of this wave in layer l.  trace_wg >= 0: every wave of that workgroup ([12][16] stamps);
// trace_wg == -1: waves 0, 9, 10 and 11 of every workgroup ([wg][4][16] stamps).
// (STAMPS: the time stamps are compiled in; the variant without them keeps their pointers and tests out of the layer loop)
template <bool STAMPS>
WD_DEV void res_mark(const ResidentArgs &a, const ResCtx &c, int l, int i) {
    if (!STAMPS) return;
    if (!a.trace || l != a.trace_layer || c.lane != 0) return;
    if (a.trace_wg >= 0) {
        if (c.r == a.trace_wg) a.trace[c.wave * 16 + i] = wall_clock64();
    } else if (c.wave == 0 || c.wave >= 9) {
        a.trace[(c.r * 4 + (c.wave == 0 ? 0 : c.wave - 8)) * 16 + i] = wall_clock64();
    }
}
// A pointer field of a layer descriptor, read again (the descriptors lie in global memory) and made wave-uniform.
template <typename T>
WD_DEV T *res_field(T *const *field) {
    return uniform_ptr(*const_cast<T *const volatile *>(field));
}

// Between the gate/up rows and the down rows of a layer (every wave of the workgroup calls it; `mine`: this wave's
// activation, for routed rungs in use and the shared expert).  The workgroup's eleven activations go out as one store
// of its record; waves 0..7 then wait for the records of all 512 workgroups and lay the values out in LDS by slot;
// v0, v1 receive values 8 lane .. 8 lane + 7 of this wave's slot.
template <bool STAMPS>
WD_DEV void res_exchange(const ResidentArgs &a, const ResCtx &c, int l, bool has, float mine, float4 &v0, float4 &v1, bool &dead) {
    const int lane = c.lane, wave = c.wave;
    if (has && lane == 0) c.actv()[c.slot] = mine;
    __syncthreads();  // B2: the workgroup's activations are in LDS, and no slot area is in use any more
    if (wave == 0 && lane < 3 * kResCopies) {  // piece lane % 3 of the workgroup's 48 bytes, to copy lane / 3
        const int piece = lane % 3, copy = lane / 3;
        const float4 p = reinterpret_cast<const float4 *>(c.actv())[piece];
        hand_store16(c.hb, ac_off(l, copy) + kAcRec * c.r + 16u * piece, make_uint4(f_bits(p.x), f_bits(p.y), f_bits(p.z), f_bits(p.w)));
    }
    if (wave < 8) {  // the group's copy, three 16-byte words per lane: word w is piece w % 3 of workgroup w / 3
        const int i = wave * 64 + lane;
        const unsigned base = ac_off(l, c.r & (kResCopies - 1)) + 16u * i;
        const unsigned off[3] = {base, base + 16u * 512, base + 16u * 1024};
        uint4 v[3];
        hand_wait16<3>(a, c.hb, off, true, v, dead);
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const int w = i + 512 * t, wg = w / 3, piece = w - 3 * wg;
            float *land = c.land() + (4 * piece) * 512 + wg;
            land[0] = bits_f(v[t].x), land[512] = bits_f(v[t].y), land[1024] = bits_f(v[t].z);
            if (piece < 2) land[1536] = bits_f(v[t].w);
        }
    }
    __syncthreads();  // B3: every activation of the layer is in LDS
    res_mark<STAMPS>(a, c, l, 6);
    if (has) {
        const float4 *row = reinterpret_cast<const float4 *>(c.land() + c.slot * 512 + 8 * lane);
        v0 = row[0], v1 = row[1];
    }
    __syncthreads();  // B4: the slot areas are free again
}

// The down rows 4r..4r+3 of one matrix against the activation values v0, v1 (8 lane .. 8 lane + 7) of slot `c.slot`:
// quantises them to Q8_0 and runs the four row chains; the result of row 4r + i lands in ybuf[slot * 4 + i].
template <bool STAMPS>
WD_DEV void res_down(const ResidentArgs &a, const ResCtx &c, int l, const Q8CoalRaw<0, 16> &draw, const float4 &v0, const float4 &v1) {
    const int lane = c.lane;
    uint8_t *area = c.area();
    int8_t *aq = reinterpret_cast<int8_t *>(area + kResTileBytes);
    uint16_t *ad = reinterpret_cast<uint16_t *>(area + kResTileBytes + kResF);
    lds_quantize_q8_0_step(v0, v1, true, lane * 8, aq, ad, lane);
    float y = 1.0f;
    if (!(a.debug & 8)) y = q8_rows4_coal_finish<0, 16>(draw, aq, ad, *reinterpret_cast<Q8TileNB<16> *>(area), lane);
    if ((lane & 15) == 0) c.ybuf()[c.slot * 4 + (lane >> 4)] = y;
    res_mark<STAMPS>(a, c, l, 7);
}

// ---- the ten routed waves -------------------------------------------------------------------------------------
// Waves 0..7 (always rungs 0..7) also fetch and quantise the layer's input, and in workgroup 0 select the experts.
template <int TYPE, bool STAMPS>
WD_DEV void res_routed_role(const ResidentArgs &a, uint8_t *lds_base, int r0, int lane0, int wave0, int slot0,
                            __amdgpu_buffer_rsrc_t hb, unsigned set_base, bool &dead) {
    constexpr int kRow = 8 * ((TYPE == 21) ? 110 : 82);
    const bool shared = a.shared != 0;
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, slot0, hb);
        const int r = c.r, lane = c.lane, wave = c.wave, rung = c.slot;
        const IqTables &tables = *reinterpret_cast<const IqTables *>(c.lds + kResLdsTables);
        const ResidentLayer *L = a.layers + l;
        const bool last = l == a.n_layers - 1;
        const bool gate_row = shared && r == 1 && rung == 9;  // the shared expert's gate logit: one more row of the router's kind
        // ---- the layer's input: 16 bytes per lane of waves 0..7, quantised from the registers they arrive in
        res_mark<STAMPS>(a, c, l, 0);
        if (wave < 8) {
            const int i = wave * 64 + lane;
            float4 xv;
            if (l == 0) {
                xv = reinterpret_cast<const float4 *>(a.x)[i];
            } else {
                // (the other waves of the workgroup come here while rung 0 still folds the previous layer: nothing
                // can have arrived yet)
                if (rung != 0 && WD_RES_XDELAY) __builtin_amdgcn_s_sleep(WD_RES_XDELAY);
                const unsigned off[1] = {xc_off(l, r & (kResCopies - 1)) + kXcStride * i};
                uint4 v[1];
                hand_wait16<1>(a, c.hb, off, true, v, dead);
                xv = make_float4(bits_f(v[0].x), bits_f(v[0].y), bits_f(v[0].z), bits_f(v[0].w));
            }
            res_mark<STAMPS>(a, c, l, 1);
            {   // values 4 i .. 4 i + 3 are accumulators 4 (i % 8) .. + 3 at step i / 8
                float *dst = c.xt() + (4 * (i & 7)) * kResXtRow + (i >> 3);
                dst[0] = xv.x, dst[kResXtRow] = xv.y, dst[2 * kResXtRow] = xv.z, dst[3 * kResXtRow] = xv.w;
            }
            wave_quantize_q8_k_regs(xv, c.xq() + 256 * wave, c.xd() + wave, lane);
            if (shared) {  // Q8_0: a block is eight lanes
                float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(xv.x), __builtin_fabsf(xv.y)),
                                             __builtin_fmaxf(__builtin_fabsf(xv.z), __builtin_fabsf(xv.w)));
                amax = quad_max(amax);
                amax = __builtin_fmaxf(amax, dpp_f<0x141>(amax, amax));  // row_half_mirror pairs the two quads of a block
                reinterpret_cast<uint32_t *>(c.x0q())[i] = q8_0_pack4(xv, amax);
                if ((lane & 7) == 0) c.x0d()[i >> 3] = f2h_ref(amax / 127.0f);
            }
        }
        __syncthreads();  // B1: x and its quantised forms are in LDS
        res_mark<STAMPS>(a, c, l, 2);
        const float res_pre = c.x_at(4 * r + (lane & 3));  // (rung 0 adds the layer's output to these)
        // this layer's routed tensors (the wave has nothing else to do until the ids appear)
        const uint8_t *const gate_base = res_field(&L->gate), *const up_base = res_field(&L->up), *const down_base = res_field(&L->down);

        if (gate_row) {  // (needed by the combine only: its weights are requested now)
            float gw[32];
            res_router_fetch(res_field(&L->sh_inp), gw, lane);
            const float s = res_router_dot(gw, c.xt(), lane);
            if (lane == 32) hand_store4(c.hb, rec_off(l, 1) + 4u, f_bits(s));
        }

        // ---- selection (workgroup 0): waves 0..7 hold one logit per lane
        if (r == 0) {
            uint8_t *sel = c.lds + kResLdsSel;
            int32_t *lds_ids = reinterpret_cast<int32_t *>(sel + kTopkLdsBytes1);
            float *lds_w = reinterpret_cast<float *>(sel + kTopkLdsBytes1 + 64);
            const TopkLds<1> s(sel);
            const int32_t *ids_given = a.ids_trace ? a.ids_trace + l * a.k : nullptr;
            int id_given = 0;
            if (ids_given && wave == 0 && lane < a.k) id_given = ids_given[lane];
            const float w_scale = *const_cast<const volatile float *>(&L->w_scale);  // (asked for ahead of the logits)
            float lv[1] = {-INFINITY};
            const int id = wave * 64 + lane;
            if (wave < 8) {
                const uint32_t b = hand_wait4(a, c.hb, rec_off(l, id), id < a.E, dead);
                if (id < a.E) lv[0] = bits_f(b);
                res_mark<STAMPS>(a, c, l, 3);
                topk_block_step1<1>(lv, s, lane, wave);
            }
            __syncthreads();
            res_mark<STAMPS>(a, c, l, 12);
            if (wave < 8) topk_block_step2<1>(lv, a.E, a.k, s, lane, wave);
            __syncthreads();
            res_mark<STAMPS>(a, c, l, 13);
            if (wave == 0) {
#ifdef WD_RES_SEL_STAMPS
                unsigned long long *st3 = (STAMPS && a.trace && l == a.trace_layer && a.trace_wg == 0) ? a.trace + 11 * 16 + 5 : nullptr;
#else
                unsigned long long *st3 = nullptr;
#endif
                topk_block_step3<1>(a.E, a.k, w_scale, lds_ids, lds_w, ids_given != nullptr, id_given, s, lane, st3,
                                    reinterpret_cast<uint32_t *>(a.hand + set_base + kHandIdh) + static_cast<size_t>(l) * kResIdCopies * 16, kResIdCopies);
                res_mark<STAMPS>(a, c, l, 14);
                wave_lds_fence();
                if (lane < a.k) {
                    hand_store4(c.hb, kHandWh + static_cast<unsigned>((l * 16 + lane) * 4), f_bits(lds_w[lane]));
                    if (last) {
                        a.views->ids[lane] = lds_ids[lane];
                        a.views->weights[lane] = lds_w[lane];
                    }
                }
            }
            if (last && wave < 8 && id < a.E) a.views->logits[id] = lv[0];
        }

        // ---- routed rung: gate/up row r, then down rows 4r..4r+3
        const bool on = rung < a.k;
        Q8CoalRaw<0, 16> draw;
        draw.u[0] = draw.u[1] = draw.u[2] = make_uint4(0u, 0u, 0u, 0u);
        float act = 0.0f;
#if WD_RES_DOWN_AT != 0
        uint32_t e_keep = 0;
#endif
        if (on) {
            uint32_t e = hand_wait4(a, c.hb, kHandIdh + static_cast<unsigned>(((l * kResIdCopies + (r & (kResIdCopies - 1))) * 16 + rung) * 4), true, dead);
            e = __builtin_amdgcn_readfirstlane(e);
            if (e >= static_cast<uint32_t>(a.E)) e = 0;  // only after a wait that ran out (status is set)
            res_mark<STAMPS>(a, c, l, 4);
            const uint8_t *const rows[2] = {gate_base + e * a.gate_stride + static_cast<size_t>(r) * kRow,
                                            up_base + e * a.up_stride + static_cast<size_t>(r) * kRow};
            IqRows8Raw<TYPE, 2> raw;
            raw.u[0] = raw.u[1] = make_uint4(0u, 0u, 0u, 0u);
            if (!(a.debug & 2)) raw = iq_rows8_coal_request<TYPE, 2>(rows, lane);
            float gu[2] = {1.0f, 1.0f};
            iq_rows8_coal_park<TYPE, 2>(raw, lane, c.area());
            // the down rows are asked for once the gate/up rows are here: requested together, the down rows of the
            // waves served first would delay the gate/up rows of the others, which the whole grid waits for
#if WD_RES_DOWN_AT == 0
            if (!(a.debug & 2)) draw = q8_rows4_coal_request<0, 16>(down_base + e * a.down_stride + static_cast<size_t>(r) * (4 * 16 * 34), lane);
#else
            e_keep = e;
#endif
            res_mark<STAMPS>(a, c, l, 11);
            if (!(a.debug & 1)) iq_rows8_coal_dots<TYPE, 2>(tables, c.xq(), c.xd(), lane, gu, c.area());
            act = silu_ggml(gu[0]) * gu[1];
            res_mark<STAMPS>(a, c, l, 5);
#if WD_RES_DOWN_AT == 1
            draw = q8_rows4_coal_request<0, 16>(down_base + e_keep * a.down_stride + static_cast<size_t>(r) * (4 * 16 * 34), lane);
#endif
        }
        // rung 0 folds the results with the router's weights and the shared expert's gate: published long before this
        // point as a rule, so one request now, answered while the activations are exchanged, replaces a round trip
        // between the down rows and the fold
        const bool wlane = rung == 0 && (lane < a.k || (shared && lane == 16));
        const unsigned woff = kHandWh + static_cast<unsigned>((l * 16 + (lane == 16 ? kResGateSlot : lane)) * 4);
        uint32_t wbits = kResEmpty;
        if (wlane && !dead) wbits = hand_load4(c.hb, woff);
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        res_exchange<STAMPS>(a, c, l, on, act, v0, v1, dead);
#if WD_RES_DOWN_AT == 2
        if (on) draw = q8_rows4_coal_request<0, 16>(down_base + e_keep * a.down_stride + static_cast<size_t>(r) * (4 * 16 * 34), lane);
#endif
        if (on) res_down<STAMPS>(a, c, l, draw, v0, v1);
        float wreg = 0.0f;
        if (rung == 0) {
            if (__builtin_amdgcn_ballot_w64(wlane && wbits == kResEmpty) != 0ull) wbits = hand_wait4(a, c.hb, woff, wlane, dead);
            wreg = wlane ? bits_f(wbits) : 0.0f;
        }
        __syncthreads();  // B5: the eleven results of rows 4r..4r+3 are in LDS

        // ---- ordered weighted sum, shared branch, next input
        if (rung == 0) {
            res_mark<STAMPS>(a, c, l, 8);
            const float *ybuf = c.ybuf();
            float acc = 0.0f;
            for (int m = 0; m < a.k; ++m) {
                const float wm = lane_get(wreg, m);
                const float prod = ybuf[m * 4 + (lane & 3)] * wm;
                acc = acc + prod;
            }
            float o = acc, ysh = 0.0f;
            if (shared) {
                ysh = ybuf[kResSharedSlot * 4 + (lane & 3)];
                const float prod = ysh * lane_get(wreg, 16);
                o = acc + prod;
            }
            const float scaled = o * a.residual_scale;
            float xn = res_pre + scaled;
            if (last) {
                // a wait that ran out anywhere in the grid: the caller sees it in its data, without a synchronisation
                if (dead || __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) xn = o = acc = __builtin_nanf("");
                if (lane < 4) {
                    const int row = 4 * r + lane;
                    a.x[row] = xn;
                    a.out[row] = o;
                    a.views->accum[row] = acc;
                    if (shared) a.views->down_f32[row] = ysh;
                }
            } else {
                const uint4 piece = make_uint4(f_bits(readlane_f(xn, 0)), f_bits(readlane_f(xn, 1)), f_bits(readlane_f(xn, 2)),
                                               f_bits(readlane_f(xn, 3)));
                if (lane < kResCopies) hand_store16(c.hb, xc_off(l + 1, lane) + kXcStride * r, piece);
            }
            res_mark<STAMPS>(a, c, l, 9);
        }
    }
}

// ---- the shared expert's wave ------------------------------------------------------------------------------------
template <bool STAMPS>
WD_DEV void res_shared_role(const ResidentArgs &a, uint8_t *lds_base, int r0, int lane0, int wave0,
                            __amdgpu_buffer_rsrc_t hb, bool &dead) {
    Q8Block gb[2];
    Q8CoalRaw<0, 16> draw;
    auto fetch = [&](const ResidentLayer *L, int r, int lane) {
        gb[0] = q8_load<0>(res_field(&L->sh_gate) + static_cast<size_t>(r) * (64 * 34) + lane * 34);
        gb[1] = q8_load<0>(res_field(&L->sh_up) + static_cast<size_t>(r) * (64 * 34) + lane * 34);
        draw = q8_rows4_coal_request<0, 16>(res_field(&L->sh_down) + static_cast<size_t>(r) * (4 * 16 * 34), lane);
    };
    if (a.shared) fetch(a.layers, r0, lane0);
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, kResSharedSlot, hb);
        const int r = c.r, lane = c.lane;
        __syncthreads();  // B1
        if (r == 0) {     // the selection's two barriers
            __syncthreads();
            __syncthreads();
        }
        float act = 0.0f;
        if (a.shared) {
            res_mark<STAMPS>(a, c, l, 2);
            Q8RowTile &tile = *reinterpret_cast<Q8RowTile *>(c.area());
            float acc[2] = {0.0f, 0.0f};
            q8_row_wave_pass<2>(gb, true, lane, c.x0q(), c.x0d(), tile, lane, acc);
            const float g = close_lanes8(acc[0]), u = close_lanes8(acc[1]);
            act = silu_ggml(g) * u;
            res_mark<STAMPS>(a, c, l, 5);
        }
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        res_exchange<STAMPS>(a, c, l, a.shared != 0, act, v0, v1, dead);
        if (a.shared) res_down<STAMPS>(a, c, l, draw, v0, v1);
        __syncthreads();  // B5
        // the next layer's rows, asked for on this side of the barrier: the fold of this layer must not wait for a
        // wave that is busy issuing requests
        if (a.shared && l + 1 < a.n_layers) fetch(a.layers + l + 1, r, lane);
    }
}

// ---- the router wave: row r --------------------------------------------------------------------------------------------
// It also puts the other set of hand-off buffers (`ob`) back to "not yet written": in layer l this workgroup's share of
// layers l, l + n, l + 2n, ... of that set (all kResMaxLayers layers, whatever the launch that wrote them used).
template <bool STAMPS>
WD_DEV void res_router_role(const ResidentArgs &a, uint8_t *lds_base, int r0, int lane0, int wave0,
                            __amdgpu_buffer_rsrc_t hb, __amdgpu_buffer_rsrc_t ob, bool &dead) {
    const bool on = r0 < a.E;
    float wv[32];
    if (on) res_router_fetch(res_field(&a.layers->router) + static_cast<size_t>(r0) * kResH, wv, lane0);
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, -1, hb);
        const int r = c.r, lane = c.lane;
        const bool last = l == a.n_layers - 1;
        __syncthreads();  // B1
        res_mark<STAMPS>(a, c, l, 2);
        if (on) {
            const float s = res_router_dot(wv, c.xt(), lane);
            if (lane == 32) hand_store4(c.hb, rec_off(l, r), f_bits(s));
            res_mark<STAMPS>(a, c, l, 3);
            if (!last) res_router_fetch(res_field(&a.layers[l + 1].router) + static_cast<size_t>(r) * kResH, wv, lane);
        }
        for (int ll = l; ll < kResMaxLayers; ll += a.n_layers) {
            const uint4 empty4 = make_uint4(kResEmpty, kResEmpty, kResEmpty, kResEmpty);
            // lane 0 the workgroup's record (of the first 8 lanes), 8 lanes its 128 bytes of the layer's input copies, 24 its 384 bytes of the activations'
            const unsigned off = lane < 8 ? rec_off(ll, r) + 16u * lane
                               : lane < 16 ? xc_off(ll, 0) + kXcStride * (8 * r + lane - 8) : ac_off(ll, 0) + 16u * (24 * r + lane - 16);
            if (lane < 8 ? lane < static_cast<int>(kRecBytes / 16) : lane < 40) hand_store16(ob, off, empty4);
            if (r == 0) {
                hand_store16(ob, kHandIdh + static_cast<unsigned>(ll * kResIdCopies * 64 + 16 * lane), empty4);
                if (lane < 4) hand_store16(ob, kHandWh + static_cast<unsigned>(ll * 64 + 16 * lane), empty4);
            }
        }
        if (r == 0) {
            __syncthreads();
            __syncthreads();
            if (a.shared) {  // the shared expert's gate
                const float g = bits_f(hand_wait4(a, c.hb, rec_off(l, 1) + 4u, true, dead));
                const float sg = sigmoid_ggml(g);
                if (lane == 0) {
                    hand_store4(c.hb, kHandWh + static_cast<unsigned>((l * 16 + kResGateSlot) * 4), f_bits(sg));
                    if (last) a.views->shared_gate[0] = sg;
                }
            }
        }
        float4 v0, v1;
        res_exchange<STAMPS>(a, c, l, false, 0.0f, v0, v1, dead);
        __syncthreads();  // B5
    }
}

template <int TYPE, bool STAMPS>
__global__ __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(6, 6))) void k_stack_resident(ResidentArgs a) {
    extern __shared__ __align__(16) uint8_t lds_res[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x;
    if (__hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {  // an earlier launch failed
        if (threadIdx.x < 4) a.x[4 * r + threadIdx.x] = a.out[4 * r + threadIdx.x] = __builtin_nanf("");
        return;
    }
    const unsigned epoch = __hip_atomic_load(reinterpret_cast<const unsigned *>(a.hand + kHandEpoch), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned set_base = (epoch & 1u) ? kHandSet : 0u;
    const __amdgpu_buffer_rsrc_t hb = hand_rsrc(a.hand + set_base, kHandSet), ob = hand_rsrc(a.hand + (kHandSet - set_base), kHandSet);
    stage_tables<TYPE == 21, TYPE == 22>(*reinterpret_cast<IqTables *>(lds_res + kResLdsTables), threadIdx.x, kResThreads);

    // Roles.  The twelve waves of a workgroup sit three to a SIMD (waves w, w + 4, w + 8 share one), and two
    // workgroups share a compute unit (r and r + 256).  The two light roles - shared expert and router row - go to
    // third waves of SIMDs 0 and 1 in one of the two workgroups and of SIMDs 2 and 3 in the other, so that every SIMD
    // of the compute unit carries five of the twenty routed waves.
    if (threadIdx.x < 16) reinterpret_cast<float *>(lds_res + kResLdsActv)[threadIdx.x] = 0.0f;  // slots not in use hand on zeros
    int *simd_of = reinterpret_cast<int *>(lds_res + kResLdsRoles);
    if (lane == 0) simd_of[wave] = static_cast<int>((__builtin_amdgcn_s_getreg(4 | (31 << 11)) >> 4) & 3u);  // HW_ID.SIMD_ID
    __syncthreads();
    int slot;
    {
        bool regular = true;
        for (int w = 0; w < 4; ++w) regular = regular && simd_of[w] == simd_of[w + 4] && simd_of[w] == simd_of[w + 8];
        const int lo = (r & 256) ? 2 : 0;  // the light roles take SIMDs lo and lo + 1
        int shared_wave = 10, router_wave = 11;
        if (regular) {
            for (int w = 8; w < 12; ++w) {
                if (simd_of[w] == lo) shared_wave = w;
                if (simd_of[w] == lo + 1) router_wave = w;
            }
            if (shared_wave == router_wave) shared_wave = 10, router_wave = 11;
        }
        if (wave == shared_wave) {
            slot = kResSharedSlot;
        } else if (wave == router_wave) {
            slot = -1;
        } else {
            slot = wave;
            if (wave >= 8) slot = 8 + ((wave > 8 && 8 != shared_wave && 8 != router_wave) ? 1 : 0) +
                                  ((wave > 9 && 9 != shared_wave && 9 != router_wave) ? 1 : 0) +
                                  ((wave > 10 && 10 != shared_wave && 10 != router_wave) ? 1 : 0);
        }
        slot = __builtin_amdgcn_readfirstlane(slot);
    }

    bool dead = false;
    if (slot < 0)
        res_router_role<STAMPS>(a, lds_res, r, lane, wave, hb, ob, dead);
    else if (slot == kResSharedSlot)
        res_shared_role<STAMPS>(a, lds_res, r, lane, wave, hb, dead);
    else
        res_routed_role<TYPE, STAMPS>(a, lds_res, r, lane, wave, slot, hb, set_base, dead);

    // the next launch takes the other set (workgroup 0 can only get here after every workgroup has read the number)
    if (r == 0 && threadIdx.x == 0 && !dead)
        __hip_atomic_store(reinterpret_cast<unsigned *>(a.hand + kHandEpoch), epoch + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace wd
