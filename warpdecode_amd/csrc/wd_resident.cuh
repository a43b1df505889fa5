// A whole stack of MoE layers in ONE launch: 512 resident workgroups walk the layers together.
//
// The per-layer dispatches (wd_fused.cuh) pay two launches per layer and fetch every weight only after the value it is
// multiplied with exists.  Here the workgroups stay on their compute units for the whole decode step, so
//   * no launch lies between two dependent stages - values are handed from workgroup to workgroup through small
//     buffers in global memory whose words say themselves whether they have been written (see below);
//   * weights that do not depend on a value still being computed are already on the compute unit when that value
//     arrives: the router row and the shared expert's rows of layer l + 1 are fetched during layer l; the routed rows
//     are requested the moment the expert ids are known - with a routing trace (the caller names the experts of every
//     layer) a layer ahead, while the rungs still work on the layer before.
//
// Geometry (the C2 layer shape): hidden 2048, expert ffn 512, at most 512 experts, top-k <= 10, IQ3_S or IQ2_S gate/up,
// Q8_0 down, Q8_0 shared expert.  Workgroup r (0..511) has 12 waves:
//   ten routed rungs  rung j: row r of gate and up of the j-th selected expert, then rows 4r..4r+3 of its down tensor
//   one wave          the shared expert: row r of its gate/up, rows 4r..4r+3 of its down tensor
//   one wave          router row r, and the selection
// and rung 0 folds the eleven results of rows 4r..4r+3 in the reference order and publishes these four values of the
// next layer's input.
// The selection is central.  Every router wave hands its logit to workgroup 0 (a 16-byte record per workgroup and
// layer); workgroup 0's router wave gathers the 512 logits, eight per lane, and ranks them in registers (sel_wave_ids,
// wd_fused.cuh).  Without a routing trace it publishes the ids at once, in sixteen replicas that the rungs of the grid
// poll, and only then works out the denominator and the weights, which nothing needs before the fold at the end of the
// layer.  With a routing trace the ids are inputs of the launch: the rungs request the next layer's gate/up and down rows
// while they still work on this one - at points chosen so that no request is under way when the grid exchanges values,
// because a poll comes back behind every row its wave has asked for -, decode the gate/up rows in the stretches in
// which the vector units would idle (res_routed_role), and workgroup 0 ranks between the barriers of its own
// activation exchange, so that it never holds up its own rungs (the whole grid waits for the slowest workgroup of a layer).  The shared expert's wave of
// workgroup 0 computes the softmax denominator meanwhile.  The router waves run at a raised wave priority, as do all
// waves of workgroup 0: their few instructions are on everybody's critical path.
// Routed experts in a slot pool (the expert cache's stack, with a routing trace): the pool is addressed as one tensor of
// slots, a second trace names the slot of every expert, and a layer whose slots are still being filled when the launch
// begins is waited for inside the launch (fill_need / fill_done in ResidentArgs): the fills run beside the launch on
// another stream and count the layers off.
// The float operations and their order are those of the per-layer kernels: results are bit-identical.
//
// Hand-off buffers.  Every layer of a launch has its own copy of each buffer, so no word is written twice during a
// launch.  A word holds kResEmpty (0xffffffff) until its producer stores the value; consumers poll the data words
// themselves with device-scope loads, so no flag, counter or ordering between stores is needed.  What a workgroup
// hands on in a layer: its logit (a 16-byte record that only workgroup 0 reads), its eleven activations (48 bytes) and
// its four values of the next input (16 bytes), the latter two pushed into eight contiguous copies, one per group of
// workgroups, each of which polls its own.
// A line that many compute units write piece by piece while the whole grid polls it changes hands once per write:
// thirty-two writers per line made a hand-off take 17 us, hence pieces of 16 bytes or more.  A value whose bits are
// kResEmpty (one particular NaN) is stored as the default quiet NaN instead (hand_word): it would be taken for "not yet".
// There are two sets of these buffers: a launch works in one and resets the other as it goes (the router waves, which
// have time to spare), so nothing has to be cleaned up when a launch ends.  Waits are bounded: a wait that runs out sets
// status[0] (and its mirror in host memory), after which every wait in the grid ends at once and later launches return
// immediately until the scratch is reset.
#pragma once

#include "wd_fused.cuh"
#include "wd_handword.hpp"

namespace wd {

constexpr int kResMaxLayers = 64;
constexpr int kResWgs = 512, kResWaves = 12, kResThreads = kResWaves * 64;
constexpr int kResH = 2048, kResF = 512, kResMaxK = 10, kResSharedSlot = 10, kResActSlots = 11;
constexpr uint32_t kResEmpty = kHandEmpty;
constexpr int kResXtRow = 68;      // floats per row of the transposed input in LDS (64 + bank spread)
constexpr int kResGateSlot = 15;   // word of the weights record that holds the shared expert's sigmoid gate
constexpr int kResSleepPoll = 2;   // s_sleep between two polls of a wait (flat from 1 to 8 in measurements)
constexpr int kResSleepFold = 24;  // waves that reach a layer while rung 0 still folds the one before wait this long first
constexpr int kResSgprs = 96;       // scalar registers per wave (see k_stack_resident)
constexpr int kResFillSleeps = 2;  // s_sleep 127 (about 4 us each) between two polls of a layer's fills
constexpr int kResPrioFold = 1;     // s_setprio of rung 0 while it folds (the other rungs decode the next layer's rows meanwhile)
constexpr int kResPrioDots = 1;     // s_setprio of a rung from the input's arrival to its activation, with a routing trace (-1.5 %)
constexpr int kResPrioRouter = 3, kResPrioWg0 = 2;  // s_setprio of the router waves / of workgroup 0's other waves (measured: 2-4 % each)

// The bits a value is handed on with: kResEmpty means "not yet written", so that one NaN travels as the default quiet NaN
// (wd_handword.hpp, checked on the host).
WD_DEV uint32_t hand_word(float v) { return hand_word_bits(f_bits(v)); }

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
// What every workgroup needs from every other - four values of the next input, eleven activations - is
// written by its producer into kResCopies copies, one per group of workgroups (r % kResCopies; on this device the
// workgroups of a group share an L2), laid out contiguously: the consumers of a group fetch their copy with coalesced
// requests, and a line is polled from one L2 only.
constexpr int kResCopies = 8;
constexpr unsigned kRecBytes = 16;        // a logit record: word 0 the router logit of row r, word 1 (workgroup 1) the shared expert's gate logit
constexpr unsigned kHandRec = 0;                                                        // [layers][512] records, gathered by workgroup 0 only
constexpr unsigned kXcStride = 16;        // bytes from one workgroup's four values of a layer input to the next one's
constexpr unsigned kXcBytes = kXcStride * kResWgs;                                     // one copy
constexpr unsigned kHandXc = kHandRec + kRecBytes * kResWgs * kResMaxLayers;            // [layers][copies][512] pieces of four f32: layer inputs
constexpr unsigned kAcRec = 48;                                                        // bytes of a workgroup's activations: slots 0..10, a zero
constexpr unsigned kAcBytes = kAcRec * kResWgs;                                        // 24 KB per copy
constexpr unsigned kHandAc = kHandXc + kXcBytes * kResMaxLayers * kResCopies;          // f32 [layers][copies][512][12] activations
constexpr int kResIdCopies = 16;          // replicas of the published ids (pollers spread over lines)
constexpr unsigned kHandIdh = kHandAc + kAcBytes * kResMaxLayers * kResCopies;         // u32 [layers][replicas][16] selected ids
constexpr unsigned kHandWh = kHandIdh + 4u * kResMaxLayers * kResIdCopies * 16;        // u32 [layers][16] router weights, [15] the shared gate
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
    const int32_t *ids_trace;     // null, or [n_layers][k]: the experts of every layer (the weights stay the router's)
    // Routed experts that live in a slot pool (with a routing trace only): the tensors of every layer then start at the
    // pool, one slot apart, and rows_trace names the slot of every traced expert.  A slot may still be on its way from the
    // host when the launch begins: fill_need[l] != 0 says that layer l's rows may be read once fill_done[l] has reached
    // that number (fill_done counts up, one number per token; see k_fill_slots).
    const int32_t *rows_trace;    // null (the trace's ids address the tensors), or [n_layers][k] slot numbers
    const uint32_t *fill_need;    // null, or [n_layers]
    const uint32_t *fill_done;    // [n_layers], written by the fills while the launch runs
    unsigned row_limit;           // ids (or slot numbers) that address the tensors are below this
    const struct ResidentViews *views;  // device: where the last layer's values go
    uint8_t *hand;   // the hand-off block (kHand* offsets below)
    unsigned *status;
    unsigned *status_host;        // null, or the status word's mirror in pinned host memory (the host reads it without a synchronisation)
    unsigned spin_limit;
    unsigned long long *trace;  // null, or [12][16] time stamps (100 MHz) of workgroup trace_wg in layer trace_layer
    int trace_wg, trace_layer;
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
        if (a.status_host) __hip_atomic_store(a.status_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        dead = true;
    } else if ((spins & 63u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
        dead = true;
    }
    return dead;
}
WD_DEV bool res_full(const uint4 &v) { return v.x != kResEmpty && v.y != kResEmpty && v.z != kResEmpty && v.w != kResEmpty; }

// N 16-byte pieces per lane (lanes with on == false take no part): returns when every word of every piece has been
// written.  Only pieces that are still incomplete are requested again, one poll at a time: two or three polls in flight
// measured slower (more device-scope loads compete with the stores they wait for).
template <int N>
WD_DEV void hand_wait16(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, const unsigned (&off)[N], const bool (&on)[N], uint4 (&v)[N], bool &dead) {
    bool need[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        need[i] = on[i];
        if (on[i]) v[i] = make_uint4(0u, 0u, 0u, 0u);
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
        __builtin_amdgcn_s_sleep(kResSleepPoll);
    }
}
template <int N>
WD_DEV void hand_wait16(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, const unsigned (&off)[N], bool on, uint4 (&v)[N], bool &dead) {
    bool each[N];
#pragma unroll
    for (int i = 0; i < N; ++i) each[i] = on;
    hand_wait16<N>(a, rs, off, each, v, dead);
}
// N words per lane, word i at off + i * stride (words with on[i] == false take no part; they read as zero).
// stop(): looked at after every unsuccessful round; true ends the wait early.  Returns whether every word has arrived.
template <int N, typename Stop>
WD_DEV bool hand_wait4(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, unsigned off, unsigned stride, const bool (&on)[N], uint32_t (&v)[N], bool &dead, Stop &&stop) {
    bool need[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        need[i] = on[i];
        v[i] = 0u;
    }
    if (dead) return false;
    unsigned spins = 0;
    for (;;) {
        bool any = false;
#pragma unroll
        for (int i = 0; i < N; ++i)
            if (need[i]) v[i] = hand_load4(rs, off + static_cast<unsigned>(i) * stride);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            need[i] = need[i] && v[i] == kResEmpty;
            any = any || need[i];
        }
        if (__builtin_amdgcn_ballot_w64(any) == 0ull) return true;
        if (stop() || res_give_up(a, spins, dead)) return false;
        __builtin_amdgcn_s_sleep(kResSleepPoll);
    }
}
template <int N>
WD_DEV void hand_wait4(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, unsigned off, unsigned stride, const bool (&on)[N], uint32_t (&v)[N], bool &dead) {
    (void)hand_wait4<N>(a, rs, off, stride, on, v, dead, [] { return false; });
}
// One word per lane.
WD_DEV uint32_t hand_wait4(const ResidentArgs &a, __amdgpu_buffer_rsrc_t rs, unsigned off, bool on, bool &dead) {
    const bool each[1] = {on};
    uint32_t v[1];
    hand_wait4<1>(a, rs, off, 0u, each, v, dead);
    return v[0];
}

// Whether the fills of a layer have reached `need` (numbers wrap: compared as a signed difference).
WD_DEV bool fill_reached(const ResidentArgs &a, int l, uint32_t need) {
    const uint32_t got = __hip_atomic_load(a.fill_done + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return static_cast<int32_t>(got - need) >= 0;
}
// Returns when they have (all lanes ask for the same word).  A fill takes hundreds of microseconds and crosses the host
// link: the grid asks seldom (about every 8 us per wave), each unsuccessful poll counting as 32 of the waits' polls.
WD_DEV void fill_wait(const ResidentArgs &a, int l, uint32_t need, bool &dead) {
    if (dead) return;
    unsigned spins = 0;
    while (!fill_reached(a, l, need)) {
        spins += 31u;
        if (res_give_up(a, spins, dead)) return;
#pragma unroll
        for (int i = 0; i < kResFillSleeps; ++i) __builtin_amdgcn_s_sleep(127);
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
    // (the input in two batches of 16 values: with all 32 next to the 32 weights the wave runs out of registers)
    auto run_half = [&](float start) {
        float v = start;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float4 xv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) xv[q] = xp[4 * h + q];
            asm volatile("" ::: "memory");  // (keeps the second batch's reads behind the first batch's arithmetic)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                v = __builtin_fmaf(wv[16 * h + 4 * q + 0], xv[q].x, v);
                v = __builtin_fmaf(wv[16 * h + 4 * q + 1], xv[q].y, v);
                v = __builtin_fmaf(wv[16 * h + 4 * q + 2], xv[q].z, v);
                v = __builtin_fmaf(wv[16 * h + 4 * q + 3], xv[q].w, v);
            }
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
constexpr int kResLdsActv = kResLdsRoles + 64;                        // f32 [12] this workgroup's activations (word 11 zero), u32 [1] arrivals
constexpr int kResLdsKept = kResLdsActv + 64;                         // per routed rung: 2048 bytes, the next layer's up row decoded ahead
constexpr int kResLdsBytes = kResLdsKept + kResMaxK * 2048;
constexpr int kResLdsLand = kResLdsWave;  // f32 [11][512] all activations of the layer, while no slot area is in use
static_assert(kResLdsXq % 16 == 0 && kResLdsTables % 16 == 0 && kResLdsWave % 16 == 0 && kResWaveBytes % 16 == 0 && kResLdsSel % 16 == 0, "LDS alignment");
static_assert(sizeof(Q8RowTile) <= sizeof(Q8TileNB<16>) && 2 * kIqStageBytes <= kResTileBytes, "a slot's area serves every stage");
static_assert(kResLdsBytes <= 81920, "LDS of the resident stack kernel: two workgroups per compute unit");
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
    // how many waves have handed in their activation of a layer, summed over the layers so far (every wave but the router's: 11 per layer)
    WD_DEV unsigned *arrived() const { return reinterpret_cast<unsigned *>(lds + kResLdsActv + 48); }
    WD_DEV float *land() const { return reinterpret_cast<float *>(lds + kResLdsLand); }
    WD_DEV uint8_t *kept() const { return lds + kResLdsKept + slot * 2048; }  // (routed rungs only)
};
// The context of one layer: the indices made opaque (see fresh_v); `base` is the workgroup's dynamic LDS.
// The lane number, counted anew from a mask the compiler cannot see through: one number kept from the start of the kernel
// would hold a vector register for the whole launch - one that is spilled to scratch memory when registers are short,
// and a kernel with scratch memory costs tens of microseconds more per launch.
WD_DEV int fresh_lane() {
    const unsigned all = static_cast<unsigned>(fresh_s(-1));
    return static_cast<int>(__builtin_amdgcn_mbcnt_hi(all, __builtin_amdgcn_mbcnt_lo(all, 0u)));
}
WD_DEV ResCtx res_ctx(uint8_t *base, int r, int lane, int wave, int slot, __amdgpu_buffer_rsrc_t hb) {
    ResCtx c;
    c.lds = base + fresh_s(0);
    (void)lane;
    c.lane = fresh_lane();
    c.r = fresh_s(r), c.wave = fresh_s(wave), c.slot = fresh_s(slot);
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

// The same through the scalar path (the descriptors are written before the launch): the value is wave-uniform, costs no
// vector register and no vector-memory wait, and is there long before the request that needs it.
template <typename T>
WD_DEV T *res_field_s(T *const *field) {
    const uintptr_t at = reinterpret_cast<uintptr_t>(field);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(at));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(at >> 32));
    const uint64_t v = *((const __attribute__((address_space(4))) uint64_t *)((static_cast<uintptr_t>(hi) << 32) | lo));
    return reinterpret_cast<T *>(static_cast<uintptr_t>(v));
}

// Between the gate/up rows and the down rows of a layer (every wave of the workgroup calls it, the router wave through its
// own three barriers; `mine`: this wave's activation, for routed rungs in use and the shared expert).  The workgroup's
// eleven activations go out as one store of its record; waves 0..7 then wait for the records of all 512 workgroups and
// lay the values out in LDS by slot; v0, v1 receive values 8 lane .. 8 lane + 7 of this wave's slot.
// before(): work between handing in the activation and the barrier; early(): work of every wave once the workgroup's
// record is on its way (no record can be complete before the slowest workgroup's has crossed the device); meanwhile():
// work for a wave that does not gather (waves 8..11) while the others wait for the records.
template <bool STAMPS, typename Before, typename Early, typename Meanwhile>
WD_DEV void res_exchange(const ResidentArgs &a, const ResCtx &c, int l, bool has, float mine, float4 &v0, float4 &v1, bool &dead, Before &&before,
                         Early &&early, Meanwhile &&meanwhile) {
    const int lane = c.lane, wave = c.wave;
    if (lane == 0) {
        if (has) c.actv()[c.slot] = mine;
        __hip_atomic_fetch_add(c.arrived(), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    before();
    __syncthreads();  // B2: the workgroup's activations are in LDS, and no slot area is in use any more
    if (wave == 0 && lane < 3 * kResCopies) {  // piece lane % 3 of the workgroup's 48 bytes, to copy lane / 3
        const int piece = lane % 3, copy = lane / 3;
        const float4 p = reinterpret_cast<const float4 *>(c.actv())[piece];
        hand_store16(c.hb, ac_off(l, copy) + kAcRec * c.r + 16u * piece, make_uint4(hand_word(p.x), hand_word(p.y), hand_word(p.z), hand_word(p.w)));
    }
    res_mark<STAMPS>(a, c, l, 10);
    early();
    if (wave < 8) {  // the group's copy, three 16-byte words per lane: word w is piece w % 3 of workgroup w / 3
        const int i = wave * 64 + lane;
        const unsigned base = ac_off(l, c.r & (kResCopies - 1)) + 16u * i;
        const unsigned off[3] = {base, base + 16u * 512, base + 16u * 1024};
        uint4 v[3];
        {
            // the first third alone until it is complete, then the rest: by then most of it is there, and a third of the
            // volume per poll goes through the fabric while the grid waits for its slowest workgroup (1.5 % of the step).
            // (The rest read through the L2 once the first third is complete, with the pieces that are behind there polled
            // past it, measured the same: the volume of the polls is not what this hand-off waits for.)
            const unsigned o1[1] = {off[0]}, o2[2] = {off[1], off[2]};
            uint4 v1[1], v2[2];
            hand_wait16<1>(a, c.hb, o1, true, v1, dead);
            hand_wait16<2>(a, c.hb, o2, true, v2, dead);
            v[0] = v1[0], v[1] = v2[0], v[2] = v2[1];
        }
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const int w = i + 512 * t, wg = w / 3, piece = w - 3 * wg;
            float *land = c.land() + (4 * piece) * 512 + wg;
            land[0] = bits_f(v[t].x), land[512] = bits_f(v[t].y), land[1024] = bits_f(v[t].z);
            if (piece < 2) land[1536] = bits_f(v[t].w);
        }
    } else {
        meanwhile();
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
// staged(): called when the rows lie in LDS and their registers are free (it may fill `draw` again).
template <bool STAMPS, typename Staged>
WD_DEV void res_down(const ResidentArgs &a, const ResCtx &c, int l, Q8CoalRaw<0, 16> &draw, const float4 &v0, const float4 &v1, Staged &&staged) {
    const int lane = c.lane;
    uint8_t *area = c.area();
    int8_t *aq = reinterpret_cast<int8_t *>(area + kResTileBytes);
    uint16_t *ad = reinterpret_cast<uint16_t *>(area + kResTileBytes + kResF);
    Q8TileNB<16> &tile = *reinterpret_cast<Q8TileNB<16> *>(area);
    uint8_t *stage = reinterpret_cast<uint8_t *>(&tile);  // (q8_rows4_coal_finish, with the request of the next rows in between)
    wave_lds_fence();
    q8_rows4_coal_stage<0, 16>(draw, stage, lane);
    staged();
    lds_quantize_q8_0_step(v0, v1, true, lane * 8, aq, ad, lane);
    wave_lds_fence();
    const float y = q8_rows4_coal_dots<0, 16>(stage, aq, ad, tile, lane);
    if ((lane & 15) == 0) c.ybuf()[c.slot * 4 + (lane >> 4)] = y;
    res_mark<STAMPS>(a, c, l, 7);
}

// ---- the ten routed waves -------------------------------------------------------------------------------------
// Rungs 0..7 (always waves 0..7) also fetch and quantise the layer's input.
// Barriers of a layer, the same for every wave of the workgroup: B1 (input in LDS), B2..B4 (exchange of the
// activations), B5 (down results in LDS).
// TRACED: the launch has a routing trace (the two forms of the role differ in when they can ask for what: one body for
// both, chosen at run time, costs the compiler's merging of registers that either form defines in its own place).
template <int TYPE, bool STAMPS, bool TRACED>
WD_DEV void res_routed_role(const ResidentArgs &a, uint8_t *lds_base, int r0, int lane0, int wave0, int slot0,
                            __amdgpu_buffer_rsrc_t hb, bool &dead) {
    // TYPE 21 / 22: gate/up rows of eight IQ3_S / IQ2_S super-blocks against the Q8_K form of the input; TYPE 8: Q8_0 rows,
    // one 34-byte block per lane, against its Q8_0 form (the row routine of the shared expert's wave).
    constexpr bool kQ8 = TYPE == 8;
    constexpr int kIq = kQ8 ? 21 : TYPE;  // (the type the super-block routines are instantiated with; unused when kQ8)
    constexpr int kRow = kQ8 ? 64 * 34 : 8 * ((TYPE == 21) ? 110 : 82);
    const bool shared = a.shared != 0;
    constexpr bool traced = TRACED;
    auto expert_in_range = [&](uint32_t e) { return e < a.row_limit ? e : 0u; };  // (out of range: a wrong trace, or a wait that ran out)
    // the expert of this rung in layer l according to the routing trace, by the number that addresses the tensors
    // (any layer number: past the end it is the last layer's)
    const int32_t *const addressed = a.rows_trace ? a.rows_trace : a.ids_trace;
    auto traced_expert = [&](int l, int rung) {
        return expert_in_range(static_cast<uint32_t>(sld_i32(addressed + (l < a.n_layers ? l : a.n_layers - 1) * a.k + rung)));
    };
    // fill_need of layer l, 0 when nothing has to be waited for
    auto fill_needed = [&](int l) { return a.fill_need && l < a.n_layers ? static_cast<uint32_t>(sld_i32(reinterpret_cast<const int32_t *>(a.fill_need) + l)) : 0u; };
    IqRows8Raw<kIq, 2> raw;
    raw.u[0] = raw.u[1] = make_uint4(0u, 0u, 0u, 0u);
    Q8Block gb[2];
    gb[0].q0 = gb[0].q1 = gb[1].q0 = gb[1].q1 = make_uint4(0u, 0u, 0u, 0u), gb[0].d = gb[1].d = 0;
    // requests row r of expert e's gate and up matrix (into raw, or into gb)
    auto gate_up_rows = [&](const uint8_t *gate_base, const uint8_t *up_base, uint32_t e, int r, int lane) {
        const uint8_t *const rows[2] = {gate_base + e * a.gate_stride + static_cast<size_t>(r) * kRow,
                                        up_base + e * a.up_stride + static_cast<size_t>(r) * kRow};
        if constexpr (kQ8) {
            gb[0] = q8_load<0>(rows[0] + lane * 34);
            gb[1] = q8_load<0>(rows[1] + lane * 34);
        } else {
            raw = iq_rows8_coal_request<kIq, 2>(rows, lane);
        }
    };
    // With a routing trace the gate/up rows of a layer are requested while the layer before decodes its own (the
    // registers they arrive in are free from the moment the rows before them lie in LDS), those of the first layer here.
    if (traced && slot0 < a.k) {
        if (const uint32_t need = fill_needed(0)) fill_wait(a, 0, need, dead);
        gate_up_rows(res_field_s(&a.layers->gate), res_field_s(&a.layers->up), traced_expert(0, slot0), r0, lane0);
    }
    bool rows_asked = true;  // with a routing trace: this layer's gate/up rows were requested during the layer before
    // With a routing trace the rows of a layer are also DECODED before the layer begins - between the end of the layer
    // before and the arrival of its output, when the vector units have nothing to do: codebook and sign lookups need no
    // activation.  What is left for the time after the input has arrived are the dot products, the fold and the chains.
    IqRows8Decoded<1> dec;
#pragma unroll
    for (int i = 0; i < 1; ++i) {
        dec.d[i] = 0u, dec.ls[i][0] = dec.ls[i][1] = 0;
#pragma unroll
        for (int c0 = 0; c0 < 8; ++c0) dec.w[i][c0] = 0u;
    }
    IqRowKept kept;  // (the up row: its weights lie in LDS)
    kept.ls[0] = kept.ls[1] = 0, kept.d = 0u;
    bool decoded = false;  // dec, kept and the wave's 2048 bytes of LDS hold this layer's rows
    // With a routing trace the down rows of a layer are requested a layer ahead as well: at the moment the rows of the layer
    // before have gone from their registers into LDS.  They then arrive while the down rows are worked through, the output
    // folded and the next input awaited - not while the activations are exchanged, where every poll of a wave comes back
    // behind the rows the wave has asked for (a wave's loads return in order) and the whole grid waits for the last poll.
    Q8CoalRaw<0, 16> draw_ahead;
    draw_ahead.u[0] = draw_ahead.u[1] = draw_ahead.u[2] = make_uint4(0u, 0u, 0u, 0u);
    bool draw_asked = false;  // draw_ahead holds (or will hold) this layer's down rows
    if (traced && slot0 < a.k) {
        draw_ahead = q8_rows4_coal_request<0, 16>(res_field_s(&a.layers->down) + traced_expert(0, slot0) * a.down_stride + static_cast<size_t>(r0) * (4 * 16 * 34), lane0);
        draw_asked = true;
    }
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, slot0, hb);
        const int r = c.r, lane = c.lane, wave = c.wave, rung = c.slot;
        // (the tables at an LDS address written out as a number - the kernel has no LDS but its dynamic block, which
        // therefore starts at 0, as the kernel checks when it begins)
        const IqTablesAt<kResLdsTables> tables;
        const ResidentLayer *L = a.layers + l;
        const bool last = l == a.n_layers - 1;
        const bool on = rung < a.k;
        res_mark<STAMPS>(a, c, l, 0);
        Q8CoalRaw<0, 16> draw_now;
        draw_now.u[0] = draw_now.u[1] = draw_now.u[2] = make_uint4(0u, 0u, 0u, 0u);
        Q8CoalRaw<0, 16> &draw = traced ? draw_ahead : draw_now;
        // what the requests below are made of, asked for now (scalar loads): the tensors of this layer and, with a routing
        // trace, the gate/up tensors and the expert of the next one
        const ResidentLayer *const Ln = a.layers + (last ? l : l + 1);
        const uint8_t *const down_base = res_field_s(&L->down);
        const uint8_t *const gate_base = res_field_s(traced ? &Ln->gate : &L->gate), *const up_base = res_field_s(traced ? &Ln->up : &L->up);
        uint32_t e = 0, e_next = 0;
        if (traced && on) e = traced_expert(l, rung), e_next = traced_expert(l + 1, rung);
        const uint32_t need_next = traced && on ? fill_needed(l + 1) : 0u;
        // ---- the layer's input: 16 bytes per lane of waves 0..7, quantised from the registers they arrive in
        if (wave < 8) {
            const int i = wave * 64 + lane;
            float4 xv;
            if (l == 0) {
                xv = reinterpret_cast<const float4 *>(a.x)[i];
            } else {
                // (the other waves of the workgroup come here while rung 0 still folds the previous layer: nothing
                // can have arrived yet)
                if (rung != 0 && !decoded) __builtin_amdgcn_s_sleep(kResSleepFold);
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
            if constexpr (!kQ8) wave_quantize_q8_k_regs(xv, c.xq() + 256 * wave, c.xd() + wave, lane);
            if (shared || kQ8) {  // Q8_0: a block is eight lanes
                float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(xv.x), __builtin_fabsf(xv.y)),
                                             __builtin_fmaxf(__builtin_fabsf(xv.z), __builtin_fabsf(xv.w)));
                amax = oct_max_nonneg(amax);
                reinterpret_cast<uint32_t *>(c.x0q())[i] = q8_0_pack4(xv, amax);
                if ((lane & 7) == 0) c.x0d()[i >> 3] = f2h_ref(amax / 127.0f);
            }
        }
        __syncthreads();  // B1: x and its quantised forms are in LDS
        res_mark<STAMPS>(a, c, l, 2);
        const float res_pre = c.x_at(4 * r + (lane & 3));  // (rung 0 adds the layer's output to these)
        if (!traced && on) {  // the id this rung works on, from one of the replicas workgroup 0 publishes
            e = hand_wait4(a, c.hb, kHandIdh + static_cast<unsigned>(((l * kResIdCopies + (r & (kResIdCopies - 1))) * 16 + rung) * 4), true, dead);
            e = expert_in_range(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(e)));
            gate_up_rows(gate_base, up_base, e, r, lane);
        }
        if (traced && on && !rows_asked) {  // the layer's slots were still being filled when the layer before asked
            fill_wait(a, l, fill_needed(l), dead);
            gate_up_rows(res_field_s(&L->gate), res_field_s(&L->up), e, r, lane);
        }
        res_mark<STAMPS>(a, c, l, 4);

        // ---- routed rung: gate/up row r, then down rows 4r..4r+3
        float act = 0.0f;
        // (with a routing trace the other workgroup of the compute unit may be decoding rows ahead: what the grid waits for goes first)
        if (traced && r != 0) __builtin_amdgcn_s_setprio(kResPrioDots);
        if (on) {
            float gu[2] = {1.0f, 1.0f};
            if constexpr (!kQ8) {
                if (!decoded) {
                    iq_rows8_coal_park<kIq, 2>(raw, lane, c.area());
                    iq_rows8_coal_decode<kIq, 1>(tables, lane, c.area(), dec);
                }
            }
            // Nothing below may be requested before the gate/up rows are here (the wave's loads return in order, and
            // requested together, the down rows of the waves served first would delay the gate/up rows of the others,
            // which the whole grid waits for): the expert's number passes through a statement the compiler cannot
            // look into, so that the addresses below do not exist before this point.
            asm volatile("" : "+s"(e) : : "memory");
            if (!traced || !draw_asked) draw = q8_rows4_coal_request<0, 16>(down_base + e * a.down_stride + static_cast<size_t>(r) * (4 * 16 * 34), lane);
            // With a routing trace the next layer's gate/up rows are requested here, ahead of the dot products: the rows of
            // this layer are decoded or parked, so their registers are free, and the earlier the rows arrive, the less the
            // polls for the activations - which come back behind them - have to wait (-0.9 % against a request behind
            // the dot products).  Q8_0 rows are still in their registers: those are asked for behind the dot products.
            constexpr bool rows_first = traced && !kQ8;
            if constexpr (rows_first) {
                rows_asked = need_next == 0u || dead || fill_reached(a, l + 1, need_next);
                if (rows_asked) gate_up_rows(gate_base, up_base, e_next, r, lane);
            }
            res_mark<STAMPS>(a, c, l, 11);
            if constexpr (kQ8) {
                Q8RowTile &tile = *reinterpret_cast<Q8RowTile *>(c.area());
                float acc[2] = {0.0f, 0.0f};
                q8_row_wave_pass<2>(gb, true, lane, c.x0q(), c.x0d(), tile, lane, acc);
                gu[0] = close_lanes8(acc[0]), gu[1] = close_lanes8(acc[1]);
            } else {
                if (decoded) iq_rows8_kept_decoded_dots<kIq>(dec, kept, c.kept(), c.xq(), c.xd(), lane, gu);
                else iq_rows8_half_decoded_dots<kIq>(dec, tables, c.xq(), c.xd(), lane, gu, c.area());
            }
            act = silu_ggml(gu[0]) * gu[1];
            if constexpr (traced && !rows_first) {
                rows_asked = need_next == 0u || dead || fill_reached(a, l + 1, need_next);
                if (rows_asked) gate_up_rows(gate_base, up_base, e_next, r, lane);
            }
            res_mark<STAMPS>(a, c, l, 5);
        }
        // rung 0 folds the results with the router's weights and the shared expert's gate: published long before this
        // point as a rule, so one request now, answered while the activations are exchanged, replaces a round trip
        // between the down rows and the fold
        if (traced && r != 0) __builtin_amdgcn_s_setprio(0);
        const bool wlane = rung == 0 && (lane < a.k || (shared && lane == 16));
        const unsigned woff = kHandWh + static_cast<unsigned>((l * 16 + (lane == 16 ? kResGateSlot : lane)) * 4);
        uint32_t wbits = kResEmpty;
        if (wlane && !dead) wbits = hand_load4(c.hb, woff);
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        res_exchange<STAMPS>(a, c, l, on, act, v0, v1, dead, [] {},
            [&] {  // the next layer's up row, requested behind this layer's dot products: decoded while the records travel
                if constexpr (!kQ8) {
                    if (traced && on && !last && rows_asked) iq_row8_coal_decode_kept<kIq>(raw.u[1], tables, lane, c.kept(), kept);
                }
            },
            [] {});
        if (on) {
            res_down<STAMPS>(a, c, l, draw, v0, v1, [&] {
                if constexpr (traced) {  // the next layer's down rows (its slots filled, if they are slots)
                    draw_asked = !last && rows_asked;
                    if (draw_asked) draw = q8_rows4_coal_request<0, 16>(res_field_s(&Ln->down) + e_next * a.down_stride + static_cast<size_t>(r) * (4 * 16 * 34), lane);
                }
            });
        }
        float wreg = 0.0f;
        if (rung == 0) {
            if (__builtin_amdgcn_ballot_w64(wlane && wbits == kResEmpty) != 0ull) wbits = hand_wait4(a, c.hb, woff, wlane, dead);
            wreg = wlane ? bits_f(wbits) : 0.0f;
        }
        __syncthreads();  // B5: the eleven results of rows 4r..4r+3 are in LDS

        // ---- ordered weighted sum, shared branch, next input
        if (rung == 0) {
            // (the other rungs start decoding the next layer's rows now: the fold, which the whole grid waits for, goes first)
            if (r != 0) __builtin_amdgcn_s_setprio(kResPrioFold);
            res_mark<STAMPS>(a, c, l, 8);
            const float *ybuf = c.ybuf();
            // (all eleven results requested from LDS at once, then the chain: a loop that reads each term when it needs it
            // pays the LDS latency eleven times, about half a microsecond between the barrier and the next input's store)
            float yv[kResMaxK];
#pragma unroll
            for (int m = 0; m < kResMaxK; ++m) yv[m] = ybuf[m * 4 + (lane & 3)];
            float ysh = ybuf[kResSharedSlot * 4 + (lane & 3)];
            float acc = 0.0f;
            if (traced && fresh_s(a.k) == kResMaxK) {  // (with a routing trace only: the other form of the role came out slower with it)
                // (every term in use, the usual case: no select between two additions of the one chain the whole grid waits
                // for - the compiler keeps the selects' ten lane masks parked in lanes of a vector register and fetches one
                // back, two instructions and their wait states, per term)
#pragma unroll
                for (int m = 0; m < kResMaxK; ++m) {
                    const float prod = yv[m] * readlane_f(wreg, m);
                    acc = acc + prod;
                }
            } else {
#pragma unroll
                for (int m = 0; m < kResMaxK; ++m) {
                    const float prod = yv[m] * readlane_f(wreg, m);
                    const float next = acc + prod;
                    acc = m < a.k ? next : acc;
                }
            }
            float o = acc;
            if (!shared) ysh = 0.0f;
            if (shared) {
                const float prod = ysh * readlane_f(wreg, 16);
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
                const uint4 piece = make_uint4(hand_word(readlane_f(xn, 0)), hand_word(readlane_f(xn, 1)), hand_word(readlane_f(xn, 2)),
                                               hand_word(readlane_f(xn, 3)));
                if (lane < kResCopies) hand_store16(c.hb, xc_off(l + 1, lane) + kXcStride * r, piece);
            }
            res_mark<STAMPS>(a, c, l, 9);
            if (r != 0) __builtin_amdgcn_s_setprio(0);
        }
        // The next layer's gate/up rows, requested behind this layer's dot products, have long arrived: they are decoded
        // now, while the next input is on its way.
        decoded = false;
        if constexpr (!kQ8) {
            if (traced && on && !last && rows_asked) {
                IqRows8Raw<kIq, 1> gate_row;  // (the up row was decoded during the exchange)
                gate_row.u[0] = raw.u[0];
                iq_rows8_coal_park<kIq, 1>(gate_row, lane, c.area());
                iq_rows8_coal_decode<kIq, 1>(tables, lane, c.area(), dec);
                decoded = true;
            }
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
    const bool traced = a.ids_trace != nullptr;
    if (a.shared) fetch(a.layers, r0, lane0);
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, kResSharedSlot, hb);
        const int r = c.r, lane = c.lane;
        const bool with_shared = fresh_s(a.shared) != 0;  // (a scalar of this layer, not a vector register kept for the launch)
        __syncthreads();  // B1
        float act = 0.0f;
        if (with_shared) {
            res_mark<STAMPS>(a, c, l, 2);
            Q8RowTile &tile = *reinterpret_cast<Q8RowTile *>(c.area());
            float acc[2] = {0.0f, 0.0f};
            q8_row_wave_pass<2>(gb, true, lane, c.x0q(), c.x0d(), tile, lane, acc);
            const float g = close_lanes8(acc[0]), u = close_lanes8(acc[1]);
            act = silu_ggml(g) * u;
            res_mark<STAMPS>(a, c, l, 5);
        }
        // Workgroup 0: this wave has time to spare where the router wave has none, so it takes the half of the selection
        // that nobody waits for until the fold - every exponential of the row and the reference's 1/sum - and leaves it in
        // LDS for the router wave.  Without a routing trace at once (the rungs are waiting for the ids anyway); with one,
        // while the other waves wait for the activations: this workgroup's activations must not be late, so ahead of
        // the barrier the wave only looks for the logits for as long as some other wave is still at work.
        bool want[8];
        float lv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) want[j] = 64 * j + lane < a.E, lv[j] = -INFINITY;
        // all logits of the layer, eight per lane (expert 64 j + lane); patient == false: only until every other wave of the
        // workgroup has handed in its activation.  True when they are all there.
        auto gather_logits = [&](bool patient) {
            uint32_t lb[8];
            const unsigned all_in = 11u * static_cast<unsigned>(l + 1);
            const bool got = hand_wait4<8>(a, c.hb, rec_off(l, lane), 64u * kRecBytes, want, lb, dead, [&] {
                return !patient && __hip_atomic_load(c.arrived(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= all_in;
            });
#pragma unroll
            for (int j = 0; j < 8; ++j) lv[j] = want[j] ? bits_f(lb[j]) : -INFINITY;
            return got;
        };
        auto denominator = [&]() {
            const TopkLds<1> scratch(c.lds + kResLdsSel);
            bool dead_row;
            const float inv = sel_wave_denominator(lv, a.E, scratch, lane, dead_row);
            if (lane == 0) scratch.rest[0] = inv, scratch.rest[1] = dead_row ? 1.0f : 0.0f;
        };
        if (r == 0 && !traced) {
            (void)gather_logits(true);
            denominator();
        }
        bool got = false;
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        res_exchange<STAMPS>(a, c, l, with_shared, act, v0, v1, dead,
            [&] { if (r == 0 && traced) got = gather_logits(false); },  // the logits ahead of the barrier, if that holds nobody up
            [] {},
            [&] {
                if (r == 0 && traced) {
                    if (!got) (void)gather_logits(true);
                    denominator();
                }
            });
        if (with_shared) res_down<STAMPS>(a, c, l, draw, v0, v1, [] {});
        __syncthreads();  // B5
        // the next layer's rows, asked for on this side of the barrier: the fold of this layer must not wait for a
        // wave that is busy issuing requests
        if (with_shared && l + 1 < a.n_layers) fetch(a.layers + l + 1, r, lane);
    }
}

// ---- the router wave: row r; in workgroup 0 the selection ----------------------------------------------------------------
// Workgroup 0's router wave gathers the 512 logits and ranks them (sel_wave_ids, wd_fused.cuh); the workgroup's shared
// expert's wave takes the denominator (sel_wave_denominator) and leaves it in LDS.  Without a routing trace the ids go
// out to the rungs of every workgroup (kResIdCopies replicas) as soon as they are known, and the weights - which only
// the fold at the end of the layer needs - follow behind the next barrier.  With a routing trace nobody waits for the
// ids, and workgroup 0 must not hold up its own rungs: ranks and weights are then taken between the barriers of the
// activation exchange, while the rungs wait for the activations.
// The wave also puts the other set of hand-off buffers (`ob`) back to "not yet written": in layer l this workgroup's
// share of layers l, l + n, l + 2n, ... of that set (all kResMaxLayers layers, whatever the launch that wrote them used).
template <bool STAMPS>
WD_DEV void res_router_role(const ResidentArgs &a, uint8_t *lds_base, int r0, int lane0, int wave0,
                            __amdgpu_buffer_rsrc_t hb, __amdgpu_buffer_rsrc_t ob, bool &dead) {
    const bool has_row = r0 < a.E;
    const bool traced = a.ids_trace != nullptr;
    // The wave's few instructions are on the critical path of the whole grid (the logit; in workgroup 0 the ranks), while
    // the rungs next to it work through thousands: it goes first whenever it has something to issue.
    __builtin_amdgcn_s_setprio(kResPrioRouter);
    // (a workgroup without a row keeps row 0 company: one definition of the row's registers per layer, no merge of an
    // old and a new value - the compiler then holds them as 32 registers, not as one value of 32 that it copies whole)
    float wv[32];
    res_router_fetch(res_field(&a.layers->router) + static_cast<size_t>(has_row ? r0 : 0) * kResH, wv, lane0);
    for (int l = 0; l < a.n_layers; ++l) {
        const ResCtx c = res_ctx(lds_base, r0, lane0, wave0, -1, hb);
        const int r = c.r, lane = c.lane;
        const bool last = l == a.n_layers - 1;
        const ResidentLayer *L = a.layers + l;
        uint8_t *sel = c.lds + kResLdsSel;
        int32_t *lds_ids = reinterpret_cast<int32_t *>(sel + kTopkLdsBytes1);
        float *lds_w = reinterpret_cast<float *>(sel + kTopkLdsBytes1 + 64);
        const TopkLds<1> scratch(sel);
        // (both asked for ahead of the logits)
        int id_given = 0;
        if (traced && r == 0 && lane < a.k) id_given = a.ids_trace[l * a.k + lane];  // (the expert's name, whatever addresses its rows)
        const float w_scale = *const_cast<const volatile float *>(&L->w_scale);
        __syncthreads();  // B1
        res_mark<STAMPS>(a, c, l, 2);
        {
            const float s = res_router_dot(wv, c.xt(), lane);
            if (has_row && lane == 32) hand_store4(c.hb, rec_off(l, r), hand_word(s));
            res_mark<STAMPS>(a, c, l, 3);
        }
        // (before the selection's values exist: this dot and they together would not fit the registers)
        if (a.shared && r == 1) {  // the shared expert's gate logit: one more row of the router's kind (the fold needs it)
            float gw[32];  // (an array of its own: the router row's registers keep one definition per layer)
            res_router_fetch(res_field(&L->sh_inp), gw, lane);
            const float s = res_router_dot(gw, c.xt(), lane);
            if (lane == 32) hand_store4(c.hb, rec_off(l, 1) + 4u, hand_word(s));
        }
        bool want[8];
        float lv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) want[j] = 64 * j + lane < a.E, lv[j] = -INFINITY;
        SelWaveState st;
        st.mx = 0.0f, st.e = 0.0f, st.id = 0, st.fast = false;
        // all logits of the layer, eight per lane (expert 64 j + lane); patient == false: only until every other wave of the
        // workgroup has handed in its activation.  True when they are all there.
        auto gather_logits = [&](bool patient) {
            uint32_t lb[8];
            const unsigned all_in = 11u * static_cast<unsigned>(l + 1);
            const bool got = hand_wait4<8>(a, c.hb, rec_off(l, lane), 64u * kRecBytes, want, lb, dead, [&] {
                return !patient && __hip_atomic_load(c.arrived(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= all_in;
            });
#pragma unroll
            for (int j = 0; j < 8; ++j) lv[j] = want[j] ? bits_f(lb[j]) : -INFINITY;
            if (got) res_mark<STAMPS>(a, c, l, 12);
            return got;
        };
        // the ids to every rung of the grid: replica c, rung j at word c * 16 + j
        auto publish_ids = [&]() {
            wave_lds_fence();
            const int j = lane & 15;
#pragma unroll
            for (int c0 = 0; c0 < kResIdCopies; c0 += 4)
                if (j < a.k) hand_store4(c.hb, kHandIdh + static_cast<unsigned>(((l * kResIdCopies + c0 + (lane >> 4)) * 16 + j) * 4), static_cast<uint32_t>(lds_ids[j]));
            res_mark<STAMPS>(a, c, l, 13);
        };
        // what every fold needs: the weights and the shared expert's gate; the last layer's values for the caller
        auto publish_weights = [&]() {
            wave_lds_fence();
            if (lane < a.k) {
                hand_store4(c.hb, kHandWh + static_cast<unsigned>((l * 16 + lane) * 4), hand_word(lds_w[lane]));
                if (last) {
                    a.views->ids[lane] = lds_ids[lane];
                    a.views->weights[lane] = lds_w[lane];
                }
            }
            if (last) {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (want[j]) a.views->logits[64 * j + lane] = lv[j];
            }
            if (a.shared) {
                const float g = bits_f(hand_wait4(a, c.hb, rec_off(l, 1) + 4u, true, dead));
                const float sg = sigmoid_ggml(g);
                if (lane == 0) {
                    hand_store4(c.hb, kHandWh + static_cast<unsigned>((l * 16 + kResGateSlot) * 4), hand_word(sg));
                    if (last) a.views->shared_gate[0] = sg;
                }
            }
            res_mark<STAMPS>(a, c, l, 14);
        };
        // the weights from this wave's ranks and the 1/sum the shared expert's wave left in LDS (on the far side of a barrier)
        auto weights_from_lds = [&]() {
            const float inv = scratch.rest[0];
            const bool dead_row = scratch.rest[1] != 0.0f;
            sel_wave_weights(a.E, a.k, w_scale, scratch, lane, st, inv, dead_row, lds_ids, lds_w, traced, id_given);
            publish_weights();
        };
        bool weights_out = false;
        if (r == 0 && !traced) {
            (void)gather_logits(true);
            sel_wave_ids(lv, a.E, a.k, lane, st);
            if (st.fast) {
                if (lane < a.k) lds_ids[lane] = st.id;
                publish_ids();
            } else {
                // the reference's rungs need every probability, and the rungs of the grid are waiting: no time for the
                // other wave (which computes the very same values into the same places)
                bool dead_row;
                const float inv = sel_wave_denominator(lv, a.E, scratch, lane, dead_row);
                sel_wave_weights(a.E, a.k, w_scale, scratch, lane, st, inv, dead_row, lds_ids, lds_w, false, 0);
                publish_ids();
                publish_weights();
                weights_out = true;
            }
        }
        for (int ll = l; ll < kResMaxLayers; ll += a.n_layers) {
            const uint4 empty4 = make_uint4(kResEmpty, kResEmpty, kResEmpty, kResEmpty);
            // lane 0 the workgroup's logit record, 8 lanes its 128 bytes of the layer's input copies, 24 its 384 bytes of the activations'
            const unsigned off = lane < 8 ? rec_off(ll, r)
                               : lane < 16 ? xc_off(ll, 0) + kXcStride * (8 * r + lane - 8) : ac_off(ll, 0) + 16u * (24 * r + lane - 16);
            if (lane == 0 || (lane >= 8 && lane < 40)) hand_store16(ob, off, empty4);
            if (r == 0) {
                hand_store16(ob, kHandIdh + static_cast<unsigned>(ll * kResIdCopies * 64 + 16 * lane), empty4);
                if (lane < 4) hand_store16(ob, kHandWh + static_cast<unsigned>(ll * 64 + 16 * lane), empty4);
            }
        }
        // The exchange of the activations: this wave (never one of waves 0..7) only keeps its three barriers company.
        // With a routing trace nobody waits for the ranks before the fold: they are taken while the activations travel;
        // the logits are gathered ahead of the barrier if that holds nobody up.
        bool got = false;
        if (r == 0 && traced) got = gather_logits(false);
        __syncthreads();  // B2
        if (r == 0 && !traced && !weights_out) weights_from_lds();
        if (r == 0 && traced) {
            if (!got) (void)gather_logits(true);
            sel_wave_ids(lv, a.E, a.k, lane, st);
            res_mark<STAMPS>(a, c, l, 13);
        }
        __syncthreads();  // B3
        __syncthreads();  // B4
        if (r == 0 && traced) weights_from_lds();
        // the next layer's row: requested behind the selection, so that its registers are not held while the selection runs,
        // and behind the exchange, whose polls it would delay
        res_router_fetch(res_field(&a.layers[last ? l : l + 1].router) + static_cast<size_t>(has_row ? r : 0) * kResH, wv, lane);
        __syncthreads();  // B5
    }
}

template <int TYPE, bool STAMPS>
// Registers: six waves per SIMD are resident (two workgroups per compute unit), which leaves a wave 80 vector registers.
// The scalar registers are capped below what six waves could share out (102 each): at 96 a SIMD keeps scalar registers
// free for the waves of another stream's small kernel - the copy kernel that fills expert slots while the stack runs
// found no room beside waves of 106.  (The cap is only honoured when the upper bound of waves_per_eu is above six.)
__global__ __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(6, 7), amdgpu_num_sgpr(kResSgprs))) void k_stack_resident(ResidentArgs a) {
    extern __shared__ __align__(16) uint8_t lds_res[];
    // (the wave's number as a scalar, the lane's counted where it is needed: no vector register is held for the whole launch)
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = blockIdx.x;
    // (the codebook lookups address the tables by number: this block of LDS has to be the first thing in the workgroup's LDS)
    const bool lds_at_zero = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t *)lds_res)) == 0u;
    if (!lds_at_zero && threadIdx.x == 0) {
        __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (a.status_host) __hip_atomic_store(a.status_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    if (!lds_at_zero || __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {  // or an earlier launch failed
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
    if (fresh_lane() == 0) simd_of[wave] = static_cast<int>((__builtin_amdgcn_s_getreg(4 | (31 << 11)) >> 4) & 3u);  // HW_ID.SIMD_ID
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

    // Workgroup 0 carries the selection on top of its share of the rows: its waves go ahead of those of the workgroup it
    // shares a compute unit with, so that it is not the one the grid waits for.
    if (r == 0) __builtin_amdgcn_s_setprio(kResPrioWg0);
    bool dead = false;
    if (slot < 0)
        res_router_role<STAMPS>(a, lds_res, r, fresh_lane(), wave, hb, ob, dead);
    else if (slot == kResSharedSlot)
        res_shared_role<STAMPS>(a, lds_res, r, fresh_lane(), wave, hb, dead);
    else
        if (a.ids_trace) res_routed_role<TYPE, STAMPS, true>(a, lds_res, r, fresh_lane(), wave, slot, hb, dead);
        else res_routed_role<TYPE, STAMPS, false>(a, lds_res, r, fresh_lane(), wave, slot, hb, dead);

    // the next launch takes the other set (workgroup 0 can only get here after every workgroup has read the number)
    if (r == 0 && wave == 0 && fresh_lane() == 0 && !dead)
        __hip_atomic_store(reinterpret_cast<unsigned *>(a.hand + kHandEpoch), epoch + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace wd
