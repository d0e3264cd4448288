// Shared declarations of the host layer and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <mutex>

// Error convention of the reference (QW/src/debug_utils.h:56-64): always on, stderr,
// "ERROR: <message> (<file>:<line>)".
#define MI_ERROR_FMT(fmt, ...) \
    std::fprintf(stderr, "ERROR: " fmt " (%s:%d)\n", ##__VA_ARGS__, __FILE__, __LINE__)

#define MI_HIP_OK(call)                                                          \
    ([&]() -> bool {                                                             \
        hipError_t e_ = (call);                                                  \
        if (e_ != hipSuccess) {                                                  \
            MI_ERROR_FMT("%s failed: %s", #call, hipGetErrorString(e_));         \
            return false;                                                        \
        }                                                                        \
        return true;                                                             \
    }())

namespace mi {

enum WeightKind : int { WK_F16 = 0, WK_Q4 = 4, WK_I8 = 8 };
// EPI_SWIGLU: two segments, gate and up, of equal N: y_gate[n] = swiglu(fp16(gate row n), fp16(up row n)),
// the unfused sequence of two GEMVs and the element-wise kernel; y_up is not written.
enum Epilogue : int { EPI_STORE = 0, EPI_ADD = 1, EPI_SWIGLU = 2 };
// EPI_ADD combines the product with the value y holds: y = fp16(y + product) in one rounding
// (ADD_FUSED), y = fp16(fp16(product) + y) as a GEMV followed by an element-wise add gives
// (ADD_ROUNDED), or y = fp16((y * sigmoid(y)) * product), y being the gate of a SwiGLU (ADD_SILU_GATE).
enum AddMode : int { ADD_FUSED = 0, ADD_ROUNDED = 1, ADD_SILU_GATE = 2 };

struct DeviceInfo {
    int  device = -1;
    int  cus = 0;
    char arch[64] = {0};
};
const DeviceInfo& device_info();
// First call of any entry point: mi_init(0) unless mi_init has run; safe from several host threads.
bool ensure_init();
// 0 = every GEMV evaluates the reference kernels' sum in their order (bit-exact);
// 1 = Q4 may use the throughput kernel (same fp32 sum, other order).
// Both are looked up for the stream a call is enqueued on: the value mi_stream_set_modes gave that
// stream, else the process default of mi_set_gemv_mode / mi_set_gemm_mode.
int gemv_mode(hipStream_t s);
int gemm_mode(hipStream_t s);   // 0 auto, 1 rows of GEMV, others pin a GEMM kernel

// Runs `raise` (a hipFuncSetAttribute call) once per call site and process, also when several host
// threads arrive together; later calls return what it returned.
#define MI_ONCE_OK(raise)                                          \
    ([&]() -> bool {                                               \
        static std::once_flag once_;                               \
        static bool ok_ = false;                                   \
        std::call_once(once_, [&] { ok_ = (raise); });             \
        return ok_;                                                \
    }())

// M rows of x (stride K) against one W; y rows have stride N.
struct GemvCall {
    const void* x = nullptr;      // fp16 [M,K]
    const void* W = nullptr;      // fp16 [N,K] | int8 [N,K] | u8 [N,K/2]
    const void* scale = nullptr;  // fp16 [N] (int8) | fp16 [N,K/32] (Q4) | null
    void*       y = nullptr;      // fp16 [M,N]; read-modify-write for EPI_ADD
    int M = 1, N = 0, K = 0;
    WeightKind kind = WK_F16;
    Epilogue   epi = EPI_STORE;
    // Decode-step fusions (no counterpart at the C boundary):
    const void* norm_w = nullptr; // fp16 [K]: x is RMS-normalised with these weights first (M = 1, see gemv_takes_norm)
    float       norm_eps = 0.0f;
    int         add_mode = 0;         // EPI_ADD: an AddMode
    // Greedy token: every wavefront of the launch also leaves the best (fp16 value, row) of the rows
    // it computed, by the reference's argmax order for num_partials = am_np, in am_v / am_i
    // [gemv_argmax_slots() entries]; one segment, M = 1, calls that gemv_takes_argmax accepts.
    float*      am_v = nullptr;
    int*        am_i = nullptr;
    int         am_np = 0;
};

// gemv.hip
constexpr int kMaxSegments = 4;
bool launch_gemv(hipStream_t s, const GemvCall& c);
// n <= kMaxSegments calls that share x, K, M, weight kind and epilogue, as one launch.
bool launch_gemv_group(hipStream_t s, const GemvCall* calls, int n);
bool gemv_takes_norm(WeightKind kind, int K);    // GemvCall::norm_w is supported for this kind and K
bool gemv_takes_swiglu(WeightKind kind, int K);  // EPI_SWIGLU is supported for this kind and K
// Candidates a launch with GemvCall::am_v writes (one per wavefront of its grid), and their upper bound.
bool gemv_takes_argmax(hipStream_t s, const GemvCall& c);   // GemvCall::am_v is supported for this call (kind, K, M, epilogue) on this stream
int  gemv_argmax_slots(const GemvCall& c);
constexpr int kGemvArgmaxMaxSlots = 8192;
bool launch_gate_up_silu(hipStream_t s, WeightKind kind, int N, int K, const void* x,
                         const void* Wg, const void* sg, const void* Wu, const void* su, void* out);
bool launch_dequant_int8(hipStream_t s, const void* q, const void* scale, int N, int K, void* w16);
bool launch_unpack_q4(hipStream_t s, const void* p, int N, int K, void* w8);

// runtime.hip: n <= kMaxSegments projections of one x (M = 1) as one GEMV launch, weight kinds and
// scales from the registry, with the decode-step fusions of GemvCall: the RMSNorm of x ahead
// (norm_w != null; all W of a kind and K that gemv_takes_norm accepts), the unfused residual
// add behind (EPI_ADD: y[i] = fp16(fp16(W[i] x) + y[i])) or the SwiGLU of a gate / up pair (EPI_SWIGLU).
bool fused_gemv(hipStream_t s, int n, const int* N, int K, const void* x, const void* const* W, void* const* y,
                const void* norm_w, float norm_eps, Epilogue epi);
// Logits of one x (RMS-normalised first when norm_w is not null) and their greedy token, the argmax
// fused into the GEMV.  *taken = false, nothing launched: this weight kind, K or stream cannot, and the
// caller runs the GEMV and launch_argmax_f16 itself.
bool linear_argmax(hipStream_t s, int N, int K, const void* x, const void* W, void* logits, const void* norm_w,
                   float norm_eps, int num_partials, void* token_out, int* token_copy, int* counter, bool* taken);
bool fused_gemv_kind(const void* W, int N, int K, WeightKind* kind);   // kind W is registered as (fp16 if not)
// The same with the scales W was registered with (null for fp16 weights).
bool registered_weight(const void* W, int N, int K, WeightKind* kind, const void** scale);

// argmax.hip: index of the greatest of N fp16 values, ties as the reference's two argmax kernels break them.
// scratch: kArgmaxScratchBytes of device memory that belongs to stream s, or null (then one block does all the work).
constexpr size_t kArgmaxScratchBytes = 512;
bool launch_argmax_f16(hipStream_t s, const void* logits, int N, int num_partials, void* token_out, void* scratch);
// The second step alone, over `count` candidates (value, index) left by another kernel (a GEMV with GemvCall::am_v).
// token_copy, counter: null, or a second int the token is written to and an int that is incremented
// (a decode step's "current token" and position, which saves the step a launch).
bool launch_argmax_finish(hipStream_t s, const float* cand_v, const int* cand_i, int count, int N, int num_partials,
                          void* token_out, int* token_copy, int* counter);

// gemm.hip: out[M,N] = x[M,K] W^T on MFMA with the dequant fused into the tile load.
// Shapes and pointers the GEMM kernels take (M >= 2, K a multiple of 64, 16-byte aligned x and W).
bool gemm_supported(WeightKind kind, int M, int N, int K, const void* x, const void* W, const void* scale);
// Estimated time (us) of the kernel launch_gemm would pick in mode 0.
double gemm_estimate_us(WeightKind kind, int M, int N, int K, size_t workspace_bytes);
// What launch_gemm would run for this call on this stream: kernel 1 = the wide kernel (tile_rows
// rows of x per block, K in k_slices slices, `terms` fp16 terms per Q4 weight), 2 / 3 = 64 x 64 /
// 128 x 128 tiles, 4 = the streaming kernel for up to 64 rows of x (k_slices wavefronts of a block
// share a strip of W), 5 = the kernel with 256 x 256 blocks (int8 weights); kernel -1 = a mode that
// cannot serve this call.
struct GemmPlan { int kernel = -1, tile_rows = 0, k_slices = 1, terms = 1; };
GemmPlan plan_gemm(hipStream_t s, WeightKind kind, int M, int N, int K, size_t workspace_bytes);
// workspace: device memory that belongs to stream s (or null): the wide kernel may cut K into
// slices and park fp32 partial sums there; calls on one stream are ordered, so they can share it.
bool launch_gemm(hipStream_t s, WeightKind kind, int M, int N, int K, const void* x,
                 const void* W, const void* scale, void* out, void* workspace, size_t workspace_bytes);

}  // namespace mi
