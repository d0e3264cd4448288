// Host layer behind the C ABI: device plumbing, the weight registry and the
// `pytorch_linear` dispatcher (QW/src/utils.cpp:758-823, LF/src/utils.cpp:1263-1374).
#include "../../include/mi_linear.h"
#include "common.h"

#include <atomic>
#include <cstring>
#include <mutex>
#include <unordered_map>

// Scratch of mi_linear_argmax_static: lives in the code object, so no call ever allocates it.
// Every device that runs this library holds its own copy at its own address; the name below is
// only a host-side handle for hipGetSymbolAddress, never a pointer a kernel can use.
constexpr size_t kStaticScratchBytes = static_cast<size_t>(mi::kGemvArgmaxMaxSlots) * 8;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace mi {
namespace {

// Written by mi_init under g_init_mu; every other entry point reads them only after it has seen
// g_inited true (acquire), so host threads that arrive together at a first call initialise once.
DeviceInfo g_dev;
std::atomic<bool> g_inited{false};
std::mutex g_init_mu;
// Process defaults of the two arithmetic modes; a stream can carry its own (mi_stream_set_modes),
// so that host threads driving different streams do not change each other's arithmetic.
std::atomic<int> g_gemm_mode{0};
std::atomic<int> g_gemv_mode{1};

// Side table W pointer -> {kind, scale, N, K}; the counterpart of s_int8_aux / s_q4_aux
// (LF/src/utils.cpp:194-231).  The reference is single threaded and takes no lock; here the
// registry, the streams' workspaces and their modes sit behind one mutex, the process-wide mode
// defaults are atomics and one-time kernel attributes go through std::call_once, so several
// host threads can drive different streams.
struct Entry {
    WeightKind kind;
    const void* scale;
    int N, K;
};
std::unordered_map<const void*, Entry> g_registry;
std::mutex g_registry_mu;

// One GEMM workspace per stream made by mi_stream_create, and one for the null stream made by
// mi_init: allocated there, never inside a compute call.  Work on one stream is ordered, so the
// calls of a stream can share its workspace; a stream from elsewhere has none and its GEMMs
// simply do not slice K.
constexpr size_t kWorkspaceBytes = 16u << 20;
std::unordered_map<hipStream_t, void*> g_workspace;
struct StreamModes { int gemv = -1, gemm = -1; };      // -1: the process default
std::unordered_map<hipStream_t, StreamModes> g_stream_modes;

// Device address of `scratch` (top of this file) per device.
static_assert(kStaticScratchBytes >= kArgmaxScratchBytes, "the two-launch argmax fits as well");
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};     // device address of `scratch` per device, set by mi_init

void* workspace_of(hipStream_t s) {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    auto it = g_workspace.find(s);
    return it == g_workspace.end() ? nullptr : it->second;
}

void add_workspace(hipStream_t s) {
    void* p = nullptr;
    if (hipMalloc(&p, kWorkspaceBytes) != hipSuccess) {
        (void)hipGetLastError();      // no workspace: that stream's GEMMs run unsliced
        return;
    }
    std::lock_guard<std::mutex> lk(g_registry_mu);
    g_workspace[s] = p;
}

bool lookup(const void* W, Entry* out) {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    auto it = g_registry.find(W);
    if (it == g_registry.end()) return false;
    *out = it->second;
    return true;
}

bool resolve(const char* who, const void* W, int N, int K, Entry* e) {
    if (!lookup(W, e)) {
        *e = Entry{WK_F16, nullptr, N, K};
        return true;
    }
    if (e->N != N || e->K != K) {
        // The reference's registration comment: "N, K ... must match the GEMV call site
        // exactly" (LF/src/utils.h:126-128).
        MI_ERROR_FMT("%s: W registered as [%d,%d] but called with N=%d K=%d", who, e->N, e->K, N, K);
        return false;
    }
    return true;
}

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

}  // namespace

const DeviceInfo& device_info() { return g_dev; }

bool ensure_init() {
    if (g_inited.load(std::memory_order_acquire)) return true;
    return mi_init(0) == 1;
}

bool registered_weight(const void* W, int N, int K, WeightKind* kind, const void** scale) {
    Entry e;
    if (!resolve("decode step", W, N, K, &e)) return false;
    *kind = e.kind;
    *scale = e.scale;
    return true;
}

bool fused_gemv_kind(const void* W, int N, int K, WeightKind* kind) {
    Entry e;
    if (!resolve("decode step", W, N, K, &e)) return false;
    *kind = e.kind;
    return true;
}

bool fused_gemv(hipStream_t s, int n, const int* N, int K, const void* x, const void* const* W, void* const* y,
                const void* norm_w, float norm_eps, Epilogue epi) {
    GemvCall group[kMaxSegments];
    if (n < 1 || n > kMaxSegments) return false;
    for (int i = 0; i < n; ++i) {
        Entry e;
        if (!resolve("decode step", W[i], N[i], K, &e)) return false;
        GemvCall& d = group[i];
        d.x = x; d.W = W[i]; d.scale = e.scale; d.y = y[i];
        d.M = 1; d.N = N[i]; d.K = K; d.kind = e.kind;
        d.epi = epi;
        d.norm_w = norm_w; d.norm_eps = norm_eps; d.add_mode = epi == EPI_ADD ? ADD_ROUNDED : ADD_FUSED;
    }
    return launch_gemv_group(s, group, n);
}

bool linear_argmax_in(void* ws, hipStream_t s, int N, int K, const void* x, const void* W, void* logits,
                      const void* norm_w, float norm_eps, int num_partials, void* token_out, int* token_copy,
                      int* counter, bool* taken) {
    *taken = false;
    Entry e;
    if (!resolve("linear_argmax", W, N, K, &e)) return false;
    GemvCall c;
    c.x = x; c.W = W; c.scale = e.scale; c.y = logits;
    c.M = 1; c.N = N; c.K = K; c.kind = e.kind; c.epi = EPI_STORE;
    c.norm_w = norm_w; c.norm_eps = norm_eps;
    if (!ws || !gemv_takes_argmax(s, c) || (norm_w && !gemv_takes_norm(e.kind, K))) return true;
    static_assert(kGemvArgmaxMaxSlots * 8 <= kWorkspaceBytes, "candidates fit the workspace");
    static_assert(kGemvArgmaxMaxSlots * 8 <= kStaticScratchBytes, "candidates fit the static scratch");
    c.am_v = static_cast<float*>(ws);
    c.am_i = reinterpret_cast<int*>(c.am_v + kGemvArgmaxMaxSlots);
    c.am_np = num_partials;
    const int slots = gemv_argmax_slots(c);
    if (slots > kGemvArgmaxMaxSlots) return true;
    *taken = true;
    return launch_gemv(s, c) && launch_argmax_finish(s, c.am_v, c.am_i, slots, N, num_partials, token_out, token_copy, counter);
}

bool linear_argmax(hipStream_t s, int N, int K, const void* x, const void* W, void* logits, const void* norm_w,
                   float norm_eps, int num_partials, void* token_out, int* token_copy, int* counter, bool* taken) {
    return linear_argmax_in(workspace_of(s), s, N, K, x, W, logits, norm_w, norm_eps, num_partials, token_out,
                            token_copy, counter, taken);
}

int gemv_mode(hipStream_t s) {
    {
        std::lock_guard<std::mutex> lk(g_registry_mu);
        auto it = g_stream_modes.find(s);
        if (it != g_stream_modes.end() && it->second.gemv >= 0) return it->second.gemv;
    }
    return g_gemv_mode.load(std::memory_order_relaxed);
}

int gemm_mode(hipStream_t s) {
    {
        std::lock_guard<std::mutex> lk(g_registry_mu);
        auto it = g_stream_modes.find(s);
        if (it != g_stream_modes.end() && it->second.gemm >= 0) return it->second.gemm;
    }
    return g_gemm_mode.load(std::memory_order_relaxed);
}

}  // namespace mi

using namespace mi;

extern "C" {

int mi_init(int device) {
    std::lock_guard<std::mutex> init_lk(g_init_mu);
    int count = 0;
    if (!MI_HIP_OK(hipGetDeviceCount(&count))) return 0;
    if (device < 0 || device >= count) {
        MI_ERROR_FMT("mi_init: device %d not present (%d devices)", device, count);
        return 0;
    }
    if (!MI_HIP_OK(hipSetDevice(device))) return 0;
    hipDeviceProp_t prop;
    if (!MI_HIP_OK(hipGetDeviceProperties(&prop, device))) return 0;
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        MI_ERROR_FMT("mi_init: device %d is %s; this library holds gfx950 code only", device,
                     prop.gcnArchName);
        return 0;
    }
    if (device < kMaxDevices && !g_static_scratch[device]) {
        // with this device current: the address is the one of this device's copy of the array
        void* p = nullptr;
        if (!MI_HIP_OK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) || !p) return 0;
        g_static_scratch[device] = p;
    }
    g_dev.device = device;
    g_dev.cus = prop.multiProcessorCount;
    std::snprintf(g_dev.arch, sizeof(g_dev.arch), "%s", prop.gcnArchName);
    if (!workspace_of(nullptr)) add_workspace(nullptr);      // the null stream's GEMM workspace
    g_inited.store(true, std::memory_order_release);
    return 1;
}

const char* mi_device_arch(void) { return g_dev.arch; }
int mi_device_cus(void) { return g_dev.cus; }

void* mi_malloc(size_t bytes) {
    if (!ensure_init()) return nullptr;
    void* p = nullptr;
    if (!MI_HIP_OK(hipMalloc(&p, bytes ? bytes : 1))) return nullptr;
    return p;
}

int mi_free(void* p) {
    if (!p) return 1;
    mi_unregister_weight(p);
    return MI_HIP_OK(hipFree(p)) ? 1 : 0;
}

int mi_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (!MI_HIP_OK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)))) return 0;
    return MI_HIP_OK(hipStreamSynchronize(as_stream(stream))) ? 1 : 0;
}

int mi_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    if (!MI_HIP_OK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)))) return 0;
    return MI_HIP_OK(hipStreamSynchronize(as_stream(stream))) ? 1 : 0;
}

int mi_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    return MI_HIP_OK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream))) ? 1 : 0;
}

int mi_memset(void* dst, int byte, size_t bytes, void* stream) {
    return MI_HIP_OK(hipMemsetAsync(dst, byte, bytes, as_stream(stream))) ? 1 : 0;
}

void* mi_stream_create(void) {
    if (!ensure_init()) return nullptr;
    hipStream_t s = nullptr;
    if (!MI_HIP_OK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking))) return nullptr;
    add_workspace(s);
    return s;
}

int mi_stream_destroy(void* s) {
    if (!s) return 1;
    const int ok = MI_HIP_OK(hipStreamDestroy(as_stream(s))) ? 1 : 0;    // waits for the stream's work
    void* ws = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_registry_mu);
        auto it = g_workspace.find(as_stream(s));
        if (it != g_workspace.end()) {
            ws = it->second;
            g_workspace.erase(it);
        }
        g_stream_modes.erase(as_stream(s));
    }
    if (ws) (void)hipFree(ws);
    return ok;
}
int mi_stream_sync(void* s) { return MI_HIP_OK(hipStreamSynchronize(as_stream(s))) ? 1 : 0; }

void* mi_event_create(void) {
    if (!ensure_init()) return nullptr;
    hipEvent_t e = nullptr;
    if (!MI_HIP_OK(hipEventCreate(&e))) return nullptr;
    return e;
}
int mi_event_destroy(void* e) { return e ? (MI_HIP_OK(hipEventDestroy(static_cast<hipEvent_t>(e))) ? 1 : 0) : 1; }
int mi_event_record(void* e, void* s) {
    return MI_HIP_OK(hipEventRecord(static_cast<hipEvent_t>(e), as_stream(s))) ? 1 : 0;
}
int mi_event_sync(void* e) { return MI_HIP_OK(hipEventSynchronize(static_cast<hipEvent_t>(e))) ? 1 : 0; }
float mi_event_elapsed_ms(void* a, void* b) {
    float ms = -1.0f;
    if (!MI_HIP_OK(hipEventElapsedTime(&ms, static_cast<hipEvent_t>(a), static_cast<hipEvent_t>(b)))) return -1.0f;
    return ms;
}

// ---- registry --------------------------------------------------------------------

int mi_register_int8_weight(const void* W, const void* scale, int N, int K) {
    if (!W || !scale || N <= 0 || K <= 0) return 0;          // LF/src/utils.cpp:358
    std::lock_guard<std::mutex> lk(g_registry_mu);
    g_registry[W] = Entry{WK_I8, scale, N, K};
    return 1;
}

int mi_register_q4_weight(const void* W, const void* scale, int N, int K) {
    if (!W || !scale || N <= 0 || K <= 0) return 0;          // LF/src/utils.cpp:585
    if (K % 32 != 0) {
        // the quantizer refuses such a K (LF/scripts/quantize_q4.py:68-69)
        MI_ERROR_FMT("mi_register_q4_weight: K=%d is not a multiple of the block size 32", K);
        return 0;
    }
    std::lock_guard<std::mutex> lk(g_registry_mu);
    g_registry[W] = Entry{WK_Q4, scale, N, K};
    return 1;
}

int mi_unregister_weight(const void* W) {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    return g_registry.erase(W) ? 1 : 0;
}

int mi_weight_kind(const void* W) {
    Entry e;
    return lookup(W, &e) ? static_cast<int>(e.kind) : 0;
}

void mi_set_gemm_mode(int mode) { g_gemm_mode.store(mode, std::memory_order_relaxed); }
void mi_set_gemv_mode(int mode) { g_gemv_mode.store(mode, std::memory_order_relaxed); }

int mi_stream_set_modes(void* stream, int gemv_mode, int gemm_mode) {
    if (gemv_mode < -1 || gemv_mode > 1 || gemm_mode < -1) {
        MI_ERROR_FMT("mi_stream_set_modes: bad argument (gemv_mode=%d gemm_mode=%d)", gemv_mode, gemm_mode);
        return 0;
    }
    std::lock_guard<std::mutex> lk(g_registry_mu);
    if (gemv_mode < 0 && gemm_mode < 0) g_stream_modes.erase(as_stream(stream));
    else g_stream_modes[as_stream(stream)] = StreamModes{gemv_mode, gemm_mode};
    return 1;
}

// ---- hot path --------------------------------------------------------------------

// M > 1: a real contraction goes to the MFMA GEMM.  Every batch in mode 1, and shapes the GEMM
// does not take, run the GEMV once per row of x, as the reference's quantised prefill does; so
// do batches below 16 rows while that is estimated to be faster.  The rows of one launch run side by
// side and all but the first find W in the caches: measured under graph replay, every kind of
// weights, 2.45 us + 0.15 us per row and million weights (int8 1152 x 896: 2.7 / 3.2 / 3.7 us for 2 / 4 / 8
// rows, 4864 x 896: 3.7 / 4.8 / 7.4 us, 9728 x 896: 5.6 / 8.5 / 13.6 us; fp16 and Q4 within a tenth of
// that), against 3.8 to 4.6 us for the GEMM of a small matrix whatever its rows.
static bool takes_gemm(hipStream_t s, const Entry& e, int M, int N, int K, const void* x, const void* W) {
    const int mode = gemm_mode(s);
    if (M < 2 || mode == 1 || !gemm_supported(e.kind, M, N, K, x, W, e.scale)) return false;
    if (M >= 16 || mode != 0) return true;
    // (fp16 rows cost 1.15 times that, 1.8 times at a K of 4096 and more, where a lane holds one row;
    //  Q4 rows 0.05 us more)
    const double kind_factor = e.kind == WK_F16 ? (K >= 4096 ? 1.8 : 1.15) : 1.0;
    const double row_us = 0.02 + (e.kind == WK_Q4 ? 0.05 : 0.0) + kind_factor * 0.15e-6 * static_cast<double>(N) * K;
    return gemm_estimate_us(e.kind, M, N, K, workspace_of(s) ? kWorkspaceBytes : 0) < 2.45 + M * row_us;
}

int mi_linear(void* stream, int M, int N, int K, const void* x, const void* W, void* out) {
    if (!ensure_init()) return 0;
    if (M <= 0 || N <= 0 || K <= 0 || !x || !W || !out) {
        MI_ERROR_FMT("mi_linear: bad argument (M=%d N=%d K=%d x=%p W=%p out=%p)", M, N, K, x, W, out);
        return 0;
    }
    Entry e;
    if (!resolve("mi_linear", W, N, K, &e)) return 0;
    if (takes_gemm(as_stream(stream), e, M, N, K, x, W))
        return launch_gemm(as_stream(stream), e.kind, M, N, K, x, W, e.scale, out, workspace_of(as_stream(stream)),
                           kWorkspaceBytes) ? 1 : 0;
    GemvCall c;
    c.x = x; c.W = W; c.scale = e.scale; c.y = out;
    c.M = M; c.N = N; c.K = K; c.kind = e.kind; c.epi = EPI_STORE;
    return launch_gemv(as_stream(stream), c) ? 1 : 0;
}

int mi_linear_plan(void* stream, int M, int N, int K, const void* x, const void* W, int* tile_rows, int* k_slices) {
    if (!ensure_init()) return -1;
    Entry e;
    if (M <= 0 || N <= 0 || K <= 0 || !x || !W || !resolve("mi_linear_plan", W, N, K, &e)) return -1;
    if (tile_rows) *tile_rows = 0;
    if (k_slices) *k_slices = 1;
    if (!takes_gemm(as_stream(stream), e, M, N, K, x, W)) return 0;
    const GemmPlan p = plan_gemm(as_stream(stream), e.kind, M, N, K, workspace_of(as_stream(stream)) ? kWorkspaceBytes : 0);
    if (tile_rows) *tile_rows = p.tile_rows;
    if (k_slices) *k_slices = p.k_slices;
    return p.kernel;
}

int mi_argmax_f16(void* stream, const void* logits, int N, int num_partials, void* token_out) {
    if (!ensure_init()) return 0;
    if (!logits || !token_out || N <= 0 || num_partials <= 0 || reinterpret_cast<uintptr_t>(logits) % 2 ||
        reinterpret_cast<uintptr_t>(token_out) % 4) {
        MI_ERROR_FMT("mi_argmax_f16: bad argument (logits=%p N=%d num_partials=%d token_out=%p)", logits, N,
                     num_partials, token_out);
        return 0;
    }
    // the stream's workspace doubles as scratch: work on a stream is ordered, and nothing is kept there between calls
    static_assert(kArgmaxScratchBytes <= kWorkspaceBytes, "scratch fits the workspace");
    return launch_argmax_f16(as_stream(stream), logits, N, num_partials, token_out, workspace_of(as_stream(stream))) ? 1 : 0;
}

int mi_linear_argmax(void* stream, int N, int K, const void* x, const void* W, void* logits, int num_partials,
                     void* token_out) {
    if (!ensure_init()) return 0;
    if (N <= 0 || K <= 0 || !x || !W || !logits || !token_out || num_partials <= 0 ||
        reinterpret_cast<uintptr_t>(token_out) % 4) {
        MI_ERROR_FMT("mi_linear_argmax: bad argument (N=%d K=%d num_partials=%d token_out=%p)", N, K, num_partials,
                     token_out);
        return 0;
    }
    // One launch computes the logits and each wavefront's best row, a second reduces those; for
    // the kernels that cannot (Q4, other K, a stream without workspace) the argmax reads the logits back.
    bool taken = false;
    if (!linear_argmax(as_stream(stream), N, K, x, W, logits, nullptr, 0.0f, num_partials, token_out, nullptr, nullptr, &taken)) return 0;
    if (taken) return 1;
    if (!mi_linear(stream, 1, N, K, x, W, logits)) return 0;
    return mi_argmax_f16(stream, logits, N, num_partials, token_out);
}

int mi_linear_argmax_static(void* stream, int N, int K, const void* x, const void* W, void* logits, int num_partials,
                            void* token_out) {
    // (no lazy set-up here: mi_init allocates the null stream's workspace, and this entry point allocates nothing)
    if (!g_inited.load(std::memory_order_acquire)) {
        MI_ERROR_FMT("mi_linear_argmax_static: mi_init has not run on this process");
        return 0;
    }
    if (N <= 0 || K <= 0 || !x || !W || !logits || !token_out || num_partials <= 0 ||
        reinterpret_cast<uintptr_t>(token_out) % 4) {
        MI_ERROR_FMT("mi_linear_argmax_static: bad argument (N=%d K=%d num_partials=%d token_out=%p)", N, K,
                     num_partials, token_out);
        return 0;
    }
    if (N > MI_LINEAR_ARGMAX_STATIC_MAX_N) {
        MI_ERROR_FMT("mi_linear_argmax_static: N=%d is beyond the %d rows this entry point takes", N,
                     MI_LINEAR_ARGMAX_STATIC_MAX_N);
        return 0;
    }
    int device = -1;
    if (!MI_HIP_OK(hipGetDevice(&device))) return 0;
    void* ws = device >= 0 && device < kMaxDevices ? g_static_scratch[device] : nullptr;
    if (!ws) {
        MI_ERROR_FMT("mi_linear_argmax_static: device %d was not set up by mi_init", device);
        return 0;
    }
    // The candidates of the fused launch (one per wavefront of its grid, every one of them written
    // by every launch, "none" included) or the 64 partials of the two-launch argmax: nothing in the
    // scratch has to start at zero, and nothing of an earlier call is read.
    bool taken = false;
    if (!linear_argmax_in(ws, as_stream(stream), N, K, x, W, logits, nullptr, 0.0f, num_partials, token_out, nullptr,
                          nullptr, &taken)) return 0;
    if (taken) return 1;
    Entry e;
    if (!resolve("mi_linear_argmax_static", W, N, K, &e)) return 0;
    GemvCall c;
    c.x = x; c.W = W; c.scale = e.scale; c.y = logits;
    c.M = 1; c.N = N; c.K = K; c.kind = e.kind; c.epi = EPI_STORE;
    if (!launch_gemv(as_stream(stream), c)) return 0;
    return launch_argmax_f16(as_stream(stream), logits, N, num_partials, token_out, ws) ? 1 : 0;
}

// True when [a, a+na) and [b, b+nb) share a byte.
static bool overlaps(const void* a, size_t na, const void* b, size_t nb) {
    const auto pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + nb && pb < pa + na;
}

int mi_linear_batch(void* stream, const mi_linear_call* calls, int n) {
    if (!ensure_init()) return 0;
    if (!calls || n < 0) { MI_ERROR_FMT("mi_linear_batch: bad argument"); return 0; }
    // Consecutive GEMV calls that read the same x with the same K and weight kind, and
    // whose outputs touch neither that x nor each other, cannot observe one another: they
    // go out as one launch (q/k/v and gate/up of a decode step do).  Everything else is
    // enqueued call by call, in order.
    int i = 0;
    while (i < n) {
        const mi_linear_call& c0 = calls[i];
        Entry e0;
        const bool groupable = c0.M >= 1 && c0.M < 16 && c0.N > 0 && c0.K > 0 && c0.x && c0.W && c0.out &&
                               resolve("mi_linear_batch", c0.W, c0.N, c0.K, &e0) &&
                               !takes_gemm(as_stream(stream), e0, c0.M, c0.N, c0.K, c0.x, c0.W);
        if (!groupable) {
            if (!mi_linear(stream, c0.M, c0.N, c0.K, c0.x, c0.W, c0.out)) return i;
            ++i;
            continue;
        }
        GemvCall group[kMaxSegments];
        int g = 0;
        const size_t xbytes = static_cast<size_t>(c0.M) * c0.K * 2;
        while (i + g < n && g < kMaxSegments) {
            const mi_linear_call& c = calls[i + g];
            Entry e;
            if (g > 0) {
                if (c.x != c0.x || c.K != c0.K || c.M != c0.M || c.N <= 0 || !c.W || !c.out) break;
                if (!lookup(c.W, &e)) e = Entry{WK_F16, nullptr, c.N, c.K};
                if (e.kind != e0.kind || e.N != c.N || e.K != c.K) break;
            } else e = e0;
            const size_t obytes = static_cast<size_t>(c.M) * c.N * 2;
            bool clash = overlaps(c.out, obytes, c0.x, xbytes);
            for (int j = 0; j < g && !clash; ++j)
                clash = overlaps(c.out, obytes, group[j].y, static_cast<size_t>(group[j].M) * group[j].N * 2);
            if (clash) break;
            GemvCall& d = group[g];
            d.x = c.x; d.W = c.W; d.scale = e.scale; d.y = c.out;
            d.M = c.M; d.N = c.N; d.K = c.K; d.kind = e.kind; d.epi = EPI_STORE;
            ++g;
        }
        if (g == 0) {                                   // out aliases x: leave it to mi_linear
            if (!mi_linear(stream, c0.M, c0.N, c0.K, c0.x, c0.W, c0.out)) return i;
            ++i;
            continue;
        }
        if (!launch_gemv_group(as_stream(stream), group, g)) return i;
        i += g;
    }
    return n;
}

// An executable graph remembers the stream it was recorded on: the launches inside it use that
// stream's workspace (K slices of a GEMM, argmax candidates), which only that stream's order protects.
struct RecordedGraph {
    hipGraphExec_t exec;
    hipStream_t origin;
};

int mi_graph_begin(void* stream) {
    if (!ensure_init()) return 0;
    if (!stream) { MI_ERROR_FMT("mi_graph_begin: needs a stream made by mi_stream_create"); return 0; }
    return MI_HIP_OK(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal)) ? 1 : 0;
}

void* mi_graph_end(void* stream) {
    hipGraph_t g = nullptr;
    if (!MI_HIP_OK(hipStreamEndCapture(as_stream(stream), &g)) || !g) return nullptr;
    hipGraphExec_t exec = nullptr;
    const bool ok = MI_HIP_OK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
    (void)hipGraphDestroy(g);      // the executable graph keeps what it needs
    return ok ? new RecordedGraph{exec, as_stream(stream)} : nullptr;
}

int mi_graph_launch(void* graph, void* stream) {
    if (!graph) { MI_ERROR_FMT("mi_graph_launch: null graph"); return 0; }
    auto* g = static_cast<RecordedGraph*>(graph);
    if (as_stream(stream) != g->origin) {
        MI_ERROR_FMT("mi_graph_launch: graph recorded on stream %p launched on stream %p; its launches use the "
                     "recording stream's workspace, so it replays on that stream only",
                     static_cast<void*>(g->origin), stream);
        return 0;
    }
    return MI_HIP_OK(hipGraphLaunch(g->exec, g->origin)) ? 1 : 0;
}

int mi_graph_destroy(void* graph) {
    if (!graph) return 1;
    auto* g = static_cast<RecordedGraph*>(graph);
    const int ok = MI_HIP_OK(hipGraphExecDestroy(g->exec)) ? 1 : 0;
    delete g;
    return ok;
}

int mi_linear_add(void* stream, int M, int N, int K, const void* x, const void* W, void* residual) {
    if (!ensure_init()) return 0;
    if (M != 1) return 0;                                     // predicate miss, not an error
    if (N <= 0 || K <= 0 || !x || !W || !residual) {
        MI_ERROR_FMT("mi_linear_add: bad argument (N=%d K=%d)", N, K);
        return 0;
    }
    Entry e;
    if (!resolve("mi_linear_add", W, N, K, &e)) return 0;
    GemvCall c;
    c.x = x; c.W = W; c.scale = e.scale; c.y = residual;
    c.M = 1; c.N = N; c.K = K; c.kind = e.kind; c.epi = EPI_ADD;
    return launch_gemv(as_stream(stream), c) ? 1 : 0;
}

int mi_linear_silu_gate(void* stream, int N, int K, const void* x, const void* W, void* gate_inout) {
    if (!ensure_init()) return 0;
    if (N <= 0 || K <= 0 || !x || !W || !gate_inout) {
        MI_ERROR_FMT("mi_linear_silu_gate: bad argument (N=%d K=%d)", N, K);
        return 0;
    }
    Entry e;
    if (!resolve("mi_linear_silu_gate", W, N, K, &e)) return 0;
    GemvCall c;
    c.x = x; c.W = W; c.scale = e.scale; c.y = gate_inout;
    c.M = 1; c.N = N; c.K = K; c.kind = e.kind; c.epi = EPI_ADD; c.add_mode = ADD_SILU_GATE;
    return launch_gemv(as_stream(stream), c) ? 1 : 0;
}

int mi_linear_gate_up_silu(void* stream, int N, int K, const void* x, const void* Wg, const void* Wu,
                           void* out) {
    if (!ensure_init()) return 0;
    if (N <= 0 || K <= 0 || !x || !Wg || !Wu || !out) {
        MI_ERROR_FMT("mi_linear_gate_up_silu: bad argument (N=%d K=%d)", N, K);
        return 0;
    }
    Entry eg, eu;
    if (!resolve("mi_linear_gate_up_silu", Wg, N, K, &eg)) return 0;
    if (!resolve("mi_linear_gate_up_silu", Wu, N, K, &eu)) return 0;
    if (eg.kind != eu.kind || eg.kind == WK_Q4) return 0;     // predicate miss
    return launch_gate_up_silu(as_stream(stream), eg.kind, N, K, x, Wg, eg.scale, Wu, eu.scale, out) ? 1 : 0;
}

int mi_dequant_int8_to_fp16(void* stream, const void* W, const void* scale, int N, int K, void* w16) {
    if (!ensure_init()) return 0;
    if (!W || !scale || !w16) { MI_ERROR_FMT("mi_dequant_int8_to_fp16: null argument"); return 0; }
    return launch_dequant_int8(as_stream(stream), W, scale, N, K, w16) ? 1 : 0;
}

int mi_unpack_q4_to_int8(void* stream, const void* W, int N, int K, void* w8) {
    if (!ensure_init()) return 0;
    if (!W || !w8) { MI_ERROR_FMT("mi_unpack_q4_to_int8: null argument"); return 0; }
    return launch_unpack_q4(as_stream(stream), W, N, K, w8) ? 1 : 0;
}

}  // extern "C"
