// The order in which the reference's two argmax kernels (QW/kernels/gemv_m1.cl:198-280) pick a
// winner, as a total order that can be reduced in any grouping: larger value first; among equal
// values the chunk p with the lowest (bitrev6(p % 64), p), inside it the work-item
// (i - chunk start) % 64 with the lowest bit-reversed number, and for that work-item the lowest
// index.  A logit is a candidate only if it is greater than -FLT_MAX (NaN and -inf never are).
#pragma once
#include <hip/hip_runtime.h>
#include "device_math.h"

namespace mi {

constexpr float kArgmaxNone = -3.402823466e+38f;

struct Cand {
    float v;
    int i;
};

struct TieRule {
    int chunk;      // elements per chunk: ceil(N / num_partials)
    double inv;     // 1 / chunk
    __device__ explicit TieRule(int c) : chunk(c), inv(1.0 / static_cast<double>(c)) {}
    __device__ static unsigned rev6(int a) { return __brev(static_cast<unsigned>(a) & 63u) >> 26; }
    // a / chunk for a >= 0 without an integer division (two of them per tie were most of the
    // instructions of a reduction step, and candidates tie often: they are the largest fp16 values
    // of their wavefronts): the product with the rounded reciprocal is off by one at most, and
    // the remainder says which way.
    __device__ int chunk_of(int a) const {
        int q = static_cast<int>(static_cast<double>(a) * inv);
        const int r = a - q * chunk;
        q += r < 0 ? -1 : (r >= chunk ? 1 : 0);
        return q;
    }
    __device__ bool before(int a, int b) const {          // a wins a tie against b
        const int ca = chunk_of(a), cb = chunk_of(b);
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
    // the best of a wavefront's 64 candidates, in lane 0: lane g takes in lane g + 32, + 16
    // (register moves), then + 8 .. + 1 inside its row of 16 (DPP row shifts); a lane without
    // such a partner meets its own candidate, which changes nothing
    template <int SH> __device__ static Cand from_above(Cand c) {
        Cand o;
        o.v = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(c.v), __float_as_int(c.v), 0x100 + SH, 0xf, 0xf, false));
        o.i = __builtin_amdgcn_update_dpp(c.i, c.i, 0x100 + SH, 0xf, 0xf, false);
        return o;
    }
    __device__ Cand best_of_wave(Cand c) const {
        c = best(c, Cand{lane_plus32(c.v), __float_as_int(lane_plus32(__int_as_float(c.i)))});
        c = best(c, Cand{lane_plus16(c.v), __float_as_int(lane_plus16(__int_as_float(c.i)))});
        c = best(c, from_above<8>(c));
        c = best(c, from_above<4>(c));
        c = best(c, from_above<2>(c));
        c = best(c, from_above<1>(c));
        return c;
    }
};

}  // namespace mi
