// One MoE layer pass for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
// that forbid hipMalloc.  wd_moe_layer_f32 keeps its intermediate values (logits, ids, weights, activations, partial
// sums, hand-off words) in a wd_moe_scratch object, which is device memory the library allocates.  Here that memory is
// a file-scope device array of fixed size: nothing is allocated or freed, by this file or by anything it calls.
//
// Every call on a GPU shares that GPU's array, which keeps what the last call left: calls that overlap on one GPU
// (two streams, two threads) race.  The words that must start clean are reset by a small fill kernel on the caller's
// stream at the head of every call.
#include "wd_common.h"
#include "wd_fused.cuh"

using namespace wd;

namespace {

// Largest geometry served: hidden 4096, expert ffn 1024, 1024 experts, top-k 16 -> 4 KiB of logits, 68 KiB of
// activations, 2 x 16 KiB of output-sized vectors and a few words; 128 KiB holds it with room to spare.
constexpr size_t kNoAllocBytes = 128 * 1024;
constexpr int kNoAllocMaxHidden = 4096, kNoAllocMaxFfn = 1024, kNoAllocMaxExperts = 1024, kNoAllocMaxK = 16;
static __device__ __align__(256) uint8_t scratch[kNoAllocBytes];

constexpr int kNoAllocMaxDevices = 64;
uint8_t *g_scratch_ptr[kNoAllocMaxDevices];  // the array's address on each device (every GPU holds its own copy)
int g_compute_units[kNoAllocMaxDevices];

// Offsets inside the array (fixed, so that the head of the array is the same whatever the layer).
constexpr size_t kOffStatus = 0, kOffArrive = 256, kOffTagged = 512;              // words that must start clean: 512 + 1024 bytes
constexpr size_t kOffIds = kOffTagged + sizeof(uint32_t) * kTagCopies * 16;        // int32 [16]
constexpr size_t kOffWeights = kOffIds + 256, kOffGate = kOffWeights + 256;       // f32 [16], f32 [1]
constexpr size_t kOffLogits = kOffGate + 256;                                      // f32 [experts]
constexpr size_t kOffVectors = kOffLogits + sizeof(float) * kNoAllocMaxExperts;    // accum, down_f32: f32 [hidden] each; then act

// status, arrive = 0; the published ids = "not yet"
__global__ void k_noalloc_clean(uint32_t *head) {
    const int i = threadIdx.x;
    if (i < static_cast<int>(kOffTagged / 4)) head[i] = 0u;
    if (i < kTagCopies * 16) head[kOffTagged / 4 + i] = kTagInvalid;
}

}  // namespace

// The array's address on the current device, looked up once per device (wd_init calls this; so does the first call
// of the entry point on a device that wd_init has not seen).
int wd::noalloc_setup_current_device() {
    int dev = 0;
    WD_HIP(hipGetDevice(&dev));
    WD_REQUIRE(dev >= 0 && dev < kNoAllocMaxDevices, "no-alloc layer pass: device %d out of range", dev);
    if (g_scratch_ptr[dev]) return WD_OK;
    uint8_t *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail(WD_ERR_HIP, "hipGetSymbolAddress of the static scratch array failed: %s", hipGetErrorString(e));
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    g_compute_units[dev] = cus;
    g_scratch_ptr[dev] = ptr;
    return WD_OK;
}

extern "C" int wd_moe_layer_noalloc_f32(const wd_moe_layer *L, const float *d_x, float *d_out, unsigned flags, void *stream) {
    WD_REQUIRE(L && d_x && d_out, "no-alloc layer pass: null layer, activation or output pointer");
    WD_REQUIRE(flags == 0 || flags == WD_MOE_SPLIT_AB, "no-alloc layer pass: only the fused dispatches are served (flags 0x%x)", flags);
    WD_REQUIRE(L->hidden > 0 && L->hidden % 256 == 0 && L->hidden <= kNoAllocMaxHidden, "no-alloc layer pass: hidden %d exceeds the static scratch (at most %d, a multiple of 256)",
               L->hidden, kNoAllocMaxHidden);
    WD_REQUIRE(L->expert_ffn > 0 && L->expert_ffn % 32 == 0 && L->expert_ffn <= kNoAllocMaxFfn, "no-alloc layer pass: expert ffn %d exceeds the static scratch (at most %d, a multiple of 32)",
               L->expert_ffn, kNoAllocMaxFfn);
    WD_REQUIRE(L->n_experts > 0 && L->n_experts <= kNoAllocMaxExperts && L->top_k > 0 && L->top_k <= kNoAllocMaxK,
               "no-alloc layer pass: %d experts / top-%d exceed the static scratch (at most %d / %d)", L->n_experts, L->top_k,
               kNoAllocMaxExperts, kNoAllocMaxK);
    if (const int rc = noalloc_setup_current_device()) return rc;
    int dev = 0;
    WD_HIP(hipGetDevice(&dev));
    uint8_t *const ptr = g_scratch_ptr[dev];  // never the array's name: in host code that is not a device address

    const size_t H = L->hidden, F = L->expert_ffn, K1 = L->top_k + 1;
    const size_t off_accum = kOffVectors, off_down = off_accum + sizeof(float) * H, off_act = off_down + sizeof(float) * H;
    const size_t need = off_act + sizeof(float) * K1 * F;
    WD_REQUIRE(need <= kNoAllocBytes, "no-alloc layer pass: the layer needs %zu bytes of scratch, the static array has %zu", need, kNoAllocBytes);

    wd_moe_scratch view;  // a host-side description of where things lie in the array; owns nothing
    view.hidden = L->hidden, view.ffn = L->expert_ffn, view.n_experts = L->n_experts, view.max_k = L->top_k;
    view.status = reinterpret_cast<unsigned *>(ptr + kOffStatus);
    view.arrive = reinterpret_cast<unsigned *>(ptr + kOffArrive);
    view.tagged = reinterpret_cast<uint32_t *>(ptr + kOffTagged);
    view.ids = reinterpret_cast<int32_t *>(ptr + kOffIds);
    view.weights = reinterpret_cast<float *>(ptr + kOffWeights);
    view.shared_gate = reinterpret_cast<float *>(ptr + kOffGate);
    view.logits = reinterpret_cast<float *>(ptr + kOffLogits);
    view.accum = reinterpret_cast<float *>(ptr + off_accum);
    view.down_f32 = reinterpret_cast<float *>(ptr + off_down);
    view.act = reinterpret_cast<float *>(ptr + off_act);
    view.compute_units = g_compute_units[dev];
    if (const int rc = check_layer(L, &view, flags)) return rc;
    const hipStream_t st = as_stream(stream);
    k_noalloc_clean<<<dim3(1), dim3(512), 0, st>>>(reinterpret_cast<uint32_t *>(ptr));
    WD_LAUNCH_CHECK();
    return layer_fused(L, d_x, d_out, &view, flags, nullptr, nullptr, 0.0f, st);
}
