// Greedy token on the device: argmax over the fp16 logits that the lm_head GEMV has just
// written, so that the token never visits the host (the next step's embedding lookup reads it
// from device memory).
//
// The reference does this with two kernels (QW/kernels/gemv_m1.cl:198-280, enqueued by
// QW/src/model.cpp:436-482): argmax_partial cuts the N logits into num_partials contiguous
// chunks, a work-group of 64 scans each (work-item t takes chunk elements t, t + 64, ... and
// keeps the first maximum), a tree keeps the lower work-item on ties; argmax_finalize repeats
// that over the partial results.  Both comparisons are strict, so which index wins a tie is
// fixed: two equal maxima held by work-items a and b meet in the tree at the lowest bit in which
// a and b differ, and the one with a 0 there stays - the smaller bit-reversed work-item number
// wins.  Hence: the chunk p with the lowest (bitrev6(p % 64), p), inside it the work-item
// (i - chunk start) % 64 with the lowest bit-reversed number, and for that work-item the lowest
// index.  A logit is a candidate only if it is greater than -FLT_MAX (NaN and -inf never are);
// with no candidate the reference returns index 0.
//
// Here the same winner is found by a total order - larger value first, then that tie rule - which
// can be reduced in any grouping.  The comparisons are what costs (about ten vector
// instructions per logit; one block needs 18 us for 151 936 of them), so kParts blocks each reduce a
// strided share of the logits to one candidate in scratch memory and a second, single-block
// launch reduces those; without scratch memory one block does everything.
#include "common.h"
#include "argmax_rule.h"
#include <hip/hip_fp16.h>

namespace mi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr float kNone = kArgmaxNone;

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(h)));
}

// The blocks of the grid share the logits in strides of 16 bytes per thread; block b leaves its
// candidate in part_v[b], part_i[b], or, when it is the only block (part_v null), the result in out.
__global__ __launch_bounds__(kThreads) void argmax_f16_kernel(const uint16_t* __restrict__ x, int N,
                                                              int num_partials, float* __restrict__ part_v,
                                                              int* __restrict__ part_i, int* __restrict__ out) {
    const TieRule rule{(N + num_partials - 1) / num_partials};
    const int tid = blockIdx.x * kThreads + threadIdx.x, nthreads = gridDim.x * kThreads;
    Cand c{kNone, 0};
    auto offer = [&](float v, int i) {
        if (v > kNone) c = rule.best(c, Cand{v, i});
    };
    // body: 8 values per thread and step, from the first 16-byte boundary on
    const int head = static_cast<int>((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) / 2;
    const int lead = head < N ? head : N;                 // scalar elements before the aligned body
    const int groups = (N - lead) / 8;
    // kUnroll loads of 16 bytes are issued before the first comparison, so that one block keeps
    // 128 KB in flight instead of paying a memory latency per 16 KB
    constexpr int kUnroll = 8;
    for (int g0 = tid; g0 < groups; g0 += nthreads * kUnroll) {
        u32x4 q[kUnroll];
        #pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int g = g0 + u * nthreads;
            q[u] = *reinterpret_cast<const u32x4*>(x + lead + 8 * (g < groups ? g : g0));
        }
        #pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int g = g0 + u * nthreads;
            if (g >= groups) break;
            const int base = lead + 8 * g;
            #pragma unroll
            for (int e = 0; e < 4; ++e) {
                offer(half_bits_to_float(q[u][e] & 0xffffu), base + 2 * e);
                offer(half_bits_to_float(q[u][e] >> 16), base + 2 * e + 1);
            }
        }
    }
    for (int i = tid; i < lead; i += nthreads) offer(half_bits_to_float(x[i]), i);
    for (int i = lead + 8 * groups + tid; i < N; i += nthreads) offer(half_bits_to_float(x[i]), i);

    // wavefront, then block
    c = rule.best_of_wave(c);
    __shared__ float sv[kThreads / 64];
    __shared__ int si[kThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        sv[wave] = c.v;
        si[wave] = c.i;
    }
    __syncthreads();
    if (wave == 0) {
        Cand r = lane < kThreads / 64 ? Cand{sv[lane], si[lane]} : Cand{kNone, 0};
        r = rule.best_of_wave(r);
        if (lane != 0) return;
        if (part_v) {
            part_v[blockIdx.x] = r.v;
            part_i[blockIdx.x] = r.i;
        } else {
            out[0] = r.v > kNone ? r.i : 0;
        }
    }
}

// Candidates (the kParts blocks' above, or the wavefronts' of a GEMV) to the token: one block of
// 64 threads per 64 candidates, at most kFinishThreads.  A thread loads its first kAhead
// candidates before it compares any: the launch is a chain of memory latencies otherwise.
constexpr int kFinishThreads = 1024;
__global__ __launch_bounds__(kFinishThreads) void argmax_finish_kernel(const float* __restrict__ part_v,
                                                                 const int* __restrict__ part_i, int parts, int N,
                                                                 int num_partials, int* __restrict__ out,
                                                                 int* __restrict__ out2, int* __restrict__ counter) {
    const TieRule rule{(N + num_partials - 1) / num_partials};
    Cand c{kNone, 0};
    // (the counter is read now so that its round trip does not come after the reduction)
    int count_now = 0;
    if (counter && threadIdx.x == 0) count_now = counter[0];
    constexpr int kAhead = 4;
    Cand pre[kAhead];
    #pragma unroll
    for (int u = 0; u < kAhead; ++u) {
        const int p = threadIdx.x + u * blockDim.x;
        pre[u] = p < parts ? Cand{part_v[p], part_i[p]} : Cand{kNone, 0};
    }
    #pragma unroll
    for (int u = 0; u < kAhead; ++u) c = rule.best(c, pre[u]);
    for (int p = threadIdx.x + kAhead * blockDim.x; p < parts; p += blockDim.x) c = rule.best(c, Cand{part_v[p], part_i[p]});
    c = rule.best_of_wave(c);
    __shared__ float sv[kFinishThreads / 64];
    __shared__ int si[kFinishThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if (waves > 1) {
        if (lane == 0) {
            sv[wave] = c.v;
            si[wave] = c.i;
        }
        __syncthreads();
        if (wave != 0) return;
        c = lane < waves ? Cand{sv[lane], si[lane]} : Cand{kNone, 0};
        c = rule.best_of_wave(c);
    }
    if (threadIdx.x == 0) {
        const int token = c.v > kNone ? c.i : 0;
        out[0] = token;
        if (out2) out2[0] = token;
        if (counter) counter[0] = count_now + 1;
    }
}

}  // namespace

bool launch_argmax_finish(hipStream_t s, const float* cand_v, const int* cand_i, int count, int N, int num_partials,
                          void* token_out, int* token_copy, int* counter) {
    const int threads = count >= kFinishThreads ? kFinishThreads : (count + 63) / 64 * 64;
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(threads), 0, s, cand_v, cand_i, count, N, num_partials,
                       static_cast<int*>(token_out), token_copy, counter);
    return MI_HIP_OK(hipGetLastError());
}

bool launch_argmax_f16(hipStream_t s, const void* logits, int N, int num_partials, void* token_out,
                       void* scratch) {
    const auto* x = static_cast<const uint16_t*>(logits);
    auto* out = static_cast<int*>(token_out);
    constexpr int kParts = 64;                            // kArgmaxScratchBytes = kParts * 8
    if (!scratch || N < 8 * kThreads) {
        hipLaunchKernelGGL(argmax_f16_kernel, dim3(1), dim3(kThreads), 0, s, x, N, num_partials, nullptr, nullptr, out);
        return MI_HIP_OK(hipGetLastError());
    }
    auto* pv = static_cast<float*>(scratch);
    auto* pi = reinterpret_cast<int*>(pv + kParts);
    hipLaunchKernelGGL(argmax_f16_kernel, dim3(kParts), dim3(kThreads), 0, s, x, N, num_partials, pv, pi, out);
    if (!MI_HIP_OK(hipGetLastError())) return false;
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(64), 0, s, pv, pi, kParts, N, num_partials, out,
                       static_cast<int*>(nullptr), static_cast<int*>(nullptr));
    return MI_HIP_OK(hipGetLastError());
}

}  // namespace mi
