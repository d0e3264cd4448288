// The order in which the reference's two argmax kernels (QW/kernels/gemv_m1.cl:198-280) pick a
// winner, as a total order that can be reduced in any grouping: larger value first; among equal
// values the chunk p with the lowest (bitrev6(p % 64), p), inside it the work-item
// (i - chunk start) % 64 with the lowest bit-reversed number, and for that work-item the lowest
// index.  A logit is a candidate only if it is greater than -FLT_MAX (NaN and -inf never are).
#pragma once
#include <hip/hip_runtime.h>

namespace mi {

constexpr float kArgmaxNone = -3.402823466e+38f;

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
        if (a.v > b.v || !(b.v > kArgmaxNone)) return a;   // the tie rule (two divisions) only for a real tie
        return before(b.i, a.i) ? b : a;
    }
    // the best of a wavefront's 64 candidates, in lane 0
    __device__ Cand best_of_wave(Cand c) const {
        #pragma unroll
        for (int s = 32; s > 0; s >>= 1) {
            Cand o;
            o.v = __shfl_down(c.v, s, 64);
            o.i = __shfl_down(c.i, s, 64);
            c = best(c, o);
        }
        return c;
    }
};

}  // namespace mi
