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
#include <hip/hip_fp16.h>

namespace mi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr float kNone = -3.402823466e+38f;

struct Cand {
    float v;
    int i;
};

struct TieRule {
    int chunk;      // elements per chunk: ceil(N / num_partials)
    __device__ static unsigned rev6(int a) { return __brev(static_cast<unsigned>(a) & 63u) >> 26; }
    __device__ bool before(int a, int b) const {          // a wins a tie against b
        const int ca = a / chunk, cb = b / chunk;
        if (ca != cb) return (ca & 63) != (cb & 63) ? rev6(ca) < rev6(cb) : ca < cb;
        const int la = (a - ca * chunk) & 63, lb = (b - cb * chunk) & 63;
        if (la != lb) return rev6(la) < rev6(lb);
        return a < b;
    }
    __device__ Cand best(Cand a, Cand b) const {
        if (b.v > a.v) return b;
        if (a.v > b.v || !(b.v > kNone)) return a;         // the tie rule (two divisions) only for a real tie
        return before(b.i, a.i) ? b : a;
    }
};

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
    #pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        Cand o;
        o.v = __shfl_down(c.v, s, 64);
        o.i = __shfl_down(c.i, s, 64);
        c = rule.best(c, o);
    }
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
        #pragma unroll
        for (int s = kThreads / 128; s > 0; s >>= 1) {
            Cand o;
            o.v = __shfl_down(r.v, s, 64);
            o.i = __shfl_down(r.i, s, 64);
            r = rule.best(r, o);
        }
        if (lane != 0) return;
        if (part_v) {
            part_v[blockIdx.x] = r.v;
            part_i[blockIdx.x] = r.i;
        } else {
            out[0] = r.v > kNone ? r.i : 0;
        }
    }
}

// The candidates of the kParts blocks to the token: one wavefront.
__global__ __launch_bounds__(64) void argmax_finish_kernel(const float* __restrict__ part_v,
                                                           const int* __restrict__ part_i, int parts, int N,
                                                           int num_partials, int* __restrict__ out) {
    const TieRule rule{(N + num_partials - 1) / num_partials};
    Cand c{kNone, 0};
    for (int p = threadIdx.x; p < parts; p += 64) c = rule.best(c, Cand{part_v[p], part_i[p]});
    #pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        Cand o;
        o.v = __shfl_down(c.v, s, 64);
        o.i = __shfl_down(c.i, s, 64);
        c = rule.best(c, o);
    }
    if (threadIdx.x == 0) out[0] = c.v > kNone ? c.i : 0;
}

}  // namespace

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
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(64), 0, s, pv, pi, kParts, N, num_partials, out);
    return MI_HIP_OK(hipGetLastError());
}

}  // namespace mi
