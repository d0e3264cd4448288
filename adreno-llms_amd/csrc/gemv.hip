// Batch-1 (and small-batch) GEMV kernels for gfx950: y[n] = sum_k x[k] * W[n,k] with fp16,
// per-row int8 or block-32 Q4 weights, fp32 accumulation, fp16 output.
//
// Arithmetic contract.  The reference kernels (QW/kernels/gemv_m1.cl:366-462, 580-690,
// LF/kernels/gemv_m1_int8.cl:32-79, LF/kernels/gemv_m1_q4.cl:45-123) give each of 64
// work-items, in K-iteration j, one "pixel" of a row: 4 consecutive elements (fp16, int8)
// or 8 (Q4); the item keeps one fp32 accumulator per row, and the 64 accumulators are
// summed by a tree (t += t+s, s = 32..1).  These kernels evaluate exactly that sum, in that
// order, so results are bit-identical to a literal evaluation of the reference kernels:
// the 64 accumulators of a row are "virtual lanes", and one hardware lane owns VL
// consecutive virtual lanes.  With VL = 4 a lane reads 16 bytes of int8/Q4 weights per
// iteration (one global_load_dwordx4), 16 lanes cover a row-iteration and a 64-wide
// wavefront works on 4 rows at once ("a row batch"); VL = 2 and VL = 1 trade load width
// for more wavefronts when N is small.  Tree steps with s >= VL are cross-lane adds inside
// the 64/VL-lane group (v_permlane32_swap / v_permlane16_swap across rows of 16 lanes, DPP
// row shifts inside one), steps with s < VL are adds between a lane's own accumulators.
//
// A lane's K positions do not depend on the row, so in the fixed-K kernels the lane loads
// its slice of x once into registers and then streams row batches: every byte of W is
// read exactly once, fully coalesced, with non-temporal loads, and while one batch is
// being multiplied the next one is already in flight (two register buffers, the loop is
// unrolled by two so no buffer is ever copied).  Per int8 weight the inner loop is two
// VALU operations (v_cvt_f32_i32 with a byte select, v_fma_mix_f32 / v_fma_f32).  No MFMA:
// at batch 1 the op is HBM-bound.
//
// Several GEMVs that read the same x and have the same K and weight kind (q/k/v, gate/up)
// can be given to one launch as "segments": the row batches of all segments form one
// index space.  A decode step also hangs its small kernels on these launches, each with the
// arithmetic of the separate kernel it replaces: the RMSNorm of x in the prologue, the
// residual add or the SwiGLU of a gate / up pair in the epilogue, and the first step of the
// greedy argmax (every wavefront's best row) behind the lm_head.
#include "common.h"
#include <hip/hip_fp16.h>
#include "device_math.h"
#include "argmax_rule.h"

namespace mi {
namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWave * kWavesPerBlock;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int KIND> struct WT;
template <> struct WT<WK_F16> { static constexpr int EPV = 4, BPV = 8; };  // elements / bytes per virtual lane
template <> struct WT<WK_I8>  { static constexpr int EPV = 4, BPV = 4; };
template <> struct WT<WK_Q4>  { static constexpr int EPV = 8, BPV = 4; };

struct Seg {
    const uint8_t*  W;
    const uint16_t* sc;
    uint16_t*       y;
    int N;
    int first;       // index of the segment's first row batch in the launch
};
struct SegList {
    Seg s[kMaxSegments];
    int nseg;
    int nbatch;      // row batches of all segments
    const uint16_t* norm_w;   // not null: x is RMS-normalised with these weights before use
    float norm_eps;
    int add_mode;             // EPI_ADD: an AddMode
    // not null: every wavefront of gemv_fixed_k leaves the best (fp16 value, row) of its rows here,
    // slot = wavefront number in the grid, by the argmax order for chunks of am_chunk rows
    float* am_v;
    int* am_i;
    int am_chunk;
};

// EPI_ADD, what happens to the value y already holds (res):
//  ADD_FUSED     the reference's residual kernels, one rounding: fp16(res + product)
//  ADD_ROUNDED   the unfused sequence GEMV, then element-wise add of two fp16 vectors: two roundings
//  ADD_SILU_GATE res is the gate of a SwiGLU: fp16((res * sigmoid(res)) * product)
//                (LF/kernels/mlp_fused.cl:70-78: gate * sig * w3x on the fp32 product)
__device__ __forceinline__ float add_residual(float sum, float s, float res, bool scaled, int mode) {
    if (mode == ADD_ROUNDED) return h_f(f_h(scaled ? sum * s : sum)) + res;
    if (mode == ADD_SILU_GATE) {
        const float sig = __fdiv_rn(1.0f, 1.0f + exp_poly(-res));
        return (res * sig) * (scaled ? sum * s : sum);
    }
    return scaled ? fmaf(sum, s, res) : sum + res;
}

__device__ __forceinline__ float lo_f(uint32_t p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p & 0xffffu)));
}
__device__ __forceinline__ float hi_f(uint32_t p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p >> 16)));
}

// Constants that must sit in registers, not in the instruction stream: gfx950's three-operand
// encodings take no literal, and a value the compiler can see through gets folded into
// longer instruction sequences (an fma with a visible -0 addend becomes cvt + cvt + mul).
struct Consts {
    uint32_t magic;     // two halves 1024.0
    float    negzero;   // -0.0f: fma(a, b, -0) == a * b exactly, signed zeros included
};
__device__ __forceinline__ Consts make_consts() {
    Consts c{0x64006400u, -0.0f};
    asm volatile("" : "+v"(c.magic), "+v"(c.negzero));
    return c;
}

// Two nibbles of v -> two fp16 values (nibble - 8), exact.  With the nibbles at bits 0-3 and
// 16-19, magic | n is the half 1024 + n and (1024 + n) - 1032 is exact; with the nibbles
// one place up (bits 4-7 and 20-23) magic | (n << 4) is 1024 + 16 n and
// (1024 + 16 n) / 16 - 72 is exact.  Each pair costs one bit-select and one packed op.
__device__ __forceinline__ uint32_t nib_pair_lo(uint32_t v, const Consts& c) {
    const uint32_t t = (v & 0x000F000Fu) | (c.magic & ~0x000F000Fu);
    const __half2 h = __hsub2(__builtin_bit_cast(__half2, t), __builtin_bit_cast(__half2, 0x64086408u));
    return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint32_t nib_pair_hi(uint32_t v, const Consts& c) {
    const uint32_t t = (v & 0x00F000F0u) | (c.magic & ~0x00F000F0u);
    const __half2 h = __hfma2(__builtin_bit_cast(__half2, t), __builtin_bit_cast(__half2, 0x2C002C00u),
                              __builtin_bit_cast(__half2, 0xD480D480u));      // * 1/16, - 72
    return __builtin_bit_cast(uint32_t, h);
}

// One virtual lane, one K-iteration.  `scale` is used by Q4 only.
template <int KIND>
__device__ __forceinline__ float vlane_step(float acc, const uint32_t* w, const uint32_t* x, float scale,
                                            const Consts& c) {
    if constexpr (KIND == WK_F16) {
        float d = lo_f(x[0]) * lo_f(w[0]);
        d = fmaf(hi_f(x[0]), hi_f(w[0]), d);
        d = fmaf(lo_f(x[1]), lo_f(w[1]), d);
        d = fmaf(hi_f(x[1]), hi_f(w[1]), d);
        return acc + d;
    } else if constexpr (KIND == WK_I8) {
        const uint32_t v = w[0];
        const float w0 = static_cast<float>(static_cast<int8_t>(v & 0xffu));
        const float w1 = static_cast<float>(static_cast<int8_t>((v >> 8) & 0xffu));
        const float w2 = static_cast<float>(static_cast<int8_t>((v >> 16) & 0xffu));
        const float w3 = static_cast<float>(static_cast<int8_t>(v >> 24));
        float d = lo_f(x[0]) * w0;
        d = fmaf(hi_f(x[0]), w1, d);
        d = fmaf(lo_f(x[1]), w2, d);
        d = fmaf(hi_f(x[1]), w3, d);
        return acc + d;
    } else {
        const uint32_t v = w[0];
        const uint32_t v8 = v >> 8;
        const uint32_t p04 = nib_pair_lo(v, c), p15 = nib_pair_hi(v, c);
        const uint32_t p26 = nib_pair_lo(v8, c), p37 = nib_pair_hi(v8, c);
        float d = fmaf(lo_f(x[0]), lo_f(p04), c.negzero);
        d = fmaf(hi_f(x[0]), lo_f(p15), d);
        d = fmaf(lo_f(x[1]), lo_f(p26), d);
        d = fmaf(hi_f(x[1]), lo_f(p37), d);
        d = fmaf(lo_f(x[2]), hi_f(p04), d);
        d = fmaf(hi_f(x[2]), hi_f(p15), d);
        d = fmaf(lo_f(x[3]), hi_f(p26), d);
        d = fmaf(hi_f(x[3]), hi_f(p37), d);
        return fmaf(d, scale, acc);
    }
}

// ND dwords from 4*ND-byte aligned memory; NT = non-temporal (weights are used once).
template <int ND, bool NT> __device__ __forceinline__ void load_dwords(uint32_t* dst, const void* src) {
    if constexpr (ND == 1) {
        dst[0] = NT ? __builtin_nontemporal_load(static_cast<const uint32_t*>(src))
                    : *static_cast<const uint32_t*>(src);
    } else if constexpr (ND == 2) {
        const u32x2 v = NT ? __builtin_nontemporal_load(static_cast<const u32x2*>(src))
                           : *static_cast<const u32x2*>(src);
        dst[0] = v.x; dst[1] = v.y;
    } else {
        static_assert(ND % 4 == 0, "dword count");
        #pragma unroll
        for (int i = 0; i < ND / 4; ++i) {
            const u32x4 v = NT ? __builtin_nontemporal_load(static_cast<const u32x4*>(src) + i)
                               : static_cast<const u32x4*>(src)[i];
            dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
        }
    }
}

// a + (value of lane i+SH), inside a row of 16 lanes: DPP row_shl.  Lanes whose source
// falls outside the row add 0; they are lanes whose result the tree never uses.
template <int SH> __device__ __forceinline__ float add_from_above(float a) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(a), 0x100 + SH, 0xf, 0xf, true);
    return a + __int_as_float(t);
}

// The 64-virtual-lane tree of the reference, on VL accumulators per lane: steps
// s = 32 .. VL pair lane g with lane g + s/VL, steps s < VL pair a lane's own accumulators.
template <int VL> __device__ __forceinline__ float reduce_row(float (&acc)[VL]) {
    constexpr int LPR = kWave / VL;
    #pragma unroll
    for (int v = 0; v < VL; ++v) {
        if constexpr (LPR >= 64) acc[v] = acc[v] + lane_plus32(acc[v]);
        if constexpr (LPR >= 32) acc[v] = acc[v] + lane_plus16(acc[v]);
    }
    #pragma unroll
    for (int v = 0; v < VL; ++v) acc[v] = add_from_above<8>(acc[v]);
    #pragma unroll
    for (int v = 0; v < VL; ++v) acc[v] = add_from_above<4>(acc[v]);
    #pragma unroll
    for (int v = 0; v < VL; ++v) acc[v] = add_from_above<2>(acc[v]);
    #pragma unroll
    for (int v = 0; v < VL; ++v) acc[v] = add_from_above<1>(acc[v]);
    #pragma unroll
    for (int s = VL / 2; s >= 1; s >>= 1) {
        #pragma unroll
        for (int v = 0; v < s; ++v) acc[v] = acc[v] + acc[v + s];
    }
    return acc[0];
}

// Segment that holds row batch rb.  rb must be uniform over the wavefront (it is built
// from readfirstlane values), so the selects below are scalar and the segment table is
// read through the scalar cache: a vector load here would make every fetch wait for all
// outstanding weight loads.
__device__ __forceinline__ Seg find_segment(const SegList& L, int rb) {
    Seg sg = L.s[0];
    #pragma unroll
    for (int i = 1; i < kMaxSegments; ++i)
        if (i < L.nseg && rb >= L.s[i].first) sg = L.s[i];
    return sg;
}

// The first 14 dwords of a kernel's arguments arrive in scalar registers with the wavefront (the
// build asks for 16; two user registers go to the argument pointer itself); everything after them
// is fetched by the kernel's first instructions, and the vector loads that depend on it wait for
// that fetch.  So what the first loads need comes first, as plain arguments, in the order of need:
// x, the first segment's N and the number of row batches, the first segment's W and scales, the
// norm weights, the second segment's W and scales (null: one segment); y, which only the residual
// load and the stores need, is the first to be fetched.  The SegList behind them holds the same and
// the rest.
#define MI_HOT_PARAMS                                                                                         \
    const uint16_t* __restrict__ x, int hN0, int hnbatch, const uint8_t* __restrict__ hW0,                    \
    const uint16_t* __restrict__ hsc0, const uint16_t* __restrict__ hnorm_w, const uint8_t* __restrict__ hW1, \
    const uint16_t* __restrict__ hsc1, uint16_t* __restrict__ hy0
#define MI_HOT_ARGS(x, L)                                                                                     \
    (x), (L).s[0].N, (L).nbatch, (L).s[0].W, (L).s[0].sc, (L).norm_w, (L).nseg > 1 ? (L).s[1].W : nullptr,    \
    (L).nseg > 1 ? (L).s[1].sc : nullptr, (L).s[0].y

// ---- K known at compile time: x lives in registers ---------------------------------
//
// PIPE: each wavefront walks several row batches and keeps the next one in flight while it
// multiplies the current one.  Without PIPE a wavefront is expected to own one batch.
// RB row batches are fetched together, so that narrow rows (Q4, small K) still keep enough
// bytes in flight per wavefront.
template <int KIND, int KT, int VL, int EPI, bool PIPE, int RB, bool AM = false>
__global__ __launch_bounds__(kBlock) void gemv_fixed_k(MI_HOT_PARAMS, const SegList L) {
    using T = WT<KIND>;
    constexpr int LPR = kWave / VL, RPW = VL;
    constexpr int EIT = kWave * T::EPV;                 // elements per K-iteration
    constexpr int NIT = (KT + EIT - 1) / EIT;
    constexpr int XD = VL * T::EPV / 2;                 // x dwords per lane and iteration
    constexpr int WD = VL * T::BPV / 4;                 // weight dwords per lane and iteration
    constexpr int ROWB = KT / T::EPV * T::BPV;          // bytes per weight row
    constexpr int ITB = kWave * T::BPV;                 // weight bytes per row and iteration

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int g = lane % LPR, r = lane / LPR;
    const int koff = g * VL * T::EPV;
    const Consts cst = make_consts();
    const int m = blockIdx.y;
    x += static_cast<size_t>(m) * KT;

    // One row batch in registers: weights, scales and (EPI_ADD) the residual, all fetched
    // together so that the epilogue never waits on a late load.  Addresses are a per-batch
    // scalar base plus a per-lane offset that never changes, so a fetch costs no vector
    // arithmetic beyond one select for rows past N (those re-read the batch's first row).
    struct Batch {
        uint32_t w[NIT][WD];
        uint16_t s[KIND == WK_Q4 ? NIT : 1];
        uint16_t res;
        uint16_t* ybase;    // &y[m][first row of the batch], uniform
        int yoff;           // row inside the batch, -1 when the lane's row is past N
        int row0;           // first row of the batch inside its segment, uniform
    };
    const uint32_t lane_w = r * ROWB + koff / T::EPV * T::BPV;     // byte offset of the lane's weights
    const uint32_t lane_w0 = koff / T::EPV * T::BPV;               // same column, first row of the batch
    auto fetch = [&](Batch& b, int rb) {
        // (one segment, or the two of a SwiGLU launch, whose second starts at batch hnbatch: all from the
        //  arguments that came in registers; more segments: from the list)
        Seg sg{hW0, hsc0, hy0, hN0, 0};
        if constexpr (EPI == EPI_SWIGLU) {
            if (rb >= hnbatch) sg = Seg{hW1, hsc1, hy0, hN0, hnbatch};
        } else if (hW1 != nullptr) {
            sg = find_segment(L, rb);
        }
        const int row0 = (rb - sg.first) * RPW;
        const bool valid = row0 + r < sg.N;
        const int rr = valid ? r : 0;
        const uint8_t* wb = sg.W + static_cast<size_t>(row0) * ROWB;
        const uint32_t wo = valid ? lane_w : lane_w0;
        b.ybase = sg.y + static_cast<size_t>(m) * sg.N + row0;
        b.yoff = valid ? r : -1;
        b.row0 = row0;
        if constexpr (KIND == WK_I8) b.s[0] = (sg.sc + row0)[rr];
        #pragma unroll
        for (int j = 0; j < NIT; ++j) {
            // lanes idle in a partial last iteration re-read the start of their row, so that
            // every lane issues the same number of loads (the value is never used)
            const bool active = j * EIT + koff < KT;
            load_dwords<WD, true>(b.w[j], wb + (active ? wo + j * ITB : wo - lane_w0));
            if constexpr (KIND == WK_Q4)
                b.s[j] = (sg.sc + static_cast<size_t>(row0) * (KT / 32))[rr * (KT / 32) + (active ? j * 16 + (g * VL) / 4 : 0)];
        }
        // (last: y's address is the one argument that does not come in registers)
        if constexpr (EPI == EPI_ADD) b.res = b.ybase[rr];
    };
    const int nw = gridDim.x * kWavesPerBlock;
    int rb = blockIdx.x * kWavesPerBlock + wave;
    const int wid = rb;
    const TieRule rule{L.am_chunk};
    Cand top{kArgmaxNone, 0};                                 // AM: best row so far (lanes with g == 0)
    if (rb >= hnbatch) {
        if constexpr (AM) {
            if (lane == 0) { L.am_v[wid] = kArgmaxNone; L.am_i[wid] = 0; }
        }
        return;
    }
    constexpr int GB = PIPE ? RB : 1;
    struct Group { Batch b[GB]; };
    const int first = rb;
    // A wavefront owns batches rb, rb + nw, rb + 2 nw, ...; it takes them GB at a time.  A batch
    // index past the end is replaced by the wavefront's first batch (a cached re-read whose
    // result is dropped), so every fetch issues the same loads.
    auto fetch_group = [&](Group& gr, int at) {
        #pragma unroll
        for (int u = 0; u < GB; ++u) fetch(gr.b[u], at + u * nw < hnbatch ? at + u * nw : first);
    };
    const int step = nw * GB;
    // x (and the norm weights) are requested first and the first weights right behind them,
    // without a wait in between: loads return in order, so the norm of x can start while the
    // weights are still on their way, and not the other way round.
    uint32_t xr[NIT][XD];
    #pragma unroll
    for (int j = 0; j < NIT; ++j) {
        if (j * EIT + koff < KT) load_dwords<XD, false>(xr[j], x + j * EIT + koff);
        else {
            #pragma unroll
            for (int i = 0; i < XD; ++i) xr[j][i] = 0u;
        }
    }
    [[maybe_unused]] uint32_t nrm[NIT][XD];
    // (Q4: a lane's 8-element pieces are not the norm's 4-element ones, so the sum of squares
    //  takes its own copy of x in the norm's layout: lane l, elements 4 l + 256 j)
    constexpr int NJ = T::EPV == 8 ? (KT + 255) / 256 : 1;
    [[maybe_unused]] uint32_t xsq[NJ][2];
    if (hnorm_w) {
        #pragma unroll
        for (int j = 0; j < NIT; ++j)
            load_dwords<XD, false>(nrm[j], hnorm_w + (j * EIT + koff < KT ? j * EIT + koff : koff));
        if constexpr (T::EPV == 8) {
            #pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (256 * j + 4 * lane < KT) load_dwords<2, false>(xsq[j], x + 256 * j + 4 * lane);
                else xsq[j][0] = xsq[j][1] = 0u;
            }
        }
    }
    Group g0, g1;
    fetch_group(g0, rb);
    if constexpr (EPI == EPI_SWIGLU) fetch(g1.b[0], rb + hnbatch);

    // RMSNorm of x in place of a kernel of its own (QW/kernels/rmsnorm.cl: 64 lanes, each summing
    // the squares of elements 4 lane + 256 j, the same tree as the GEMV's, then
    // fp16((x * inv) * w)): the virtual lanes of this kernel own exactly those elements, so every
    // wavefront repeats the sum in the reference's order while its first weights are in flight.
    {
        if (hnorm_w) {
            float total;
            if constexpr (T::EPV == 4) {
                float part[VL];
                #pragma unroll
                for (int v = 0; v < VL; ++v) part[v] = 0.0f;
                #pragma unroll
                for (int j = 0; j < NIT; ++j) {
                    if (j * EIT + koff < KT) {
                        #pragma unroll
                        for (int v = 0; v < VL; ++v) {
                            const float v0 = lo_f(xr[j][2 * v]), v1 = hi_f(xr[j][2 * v]);
                            const float v2 = lo_f(xr[j][2 * v + 1]), v3 = hi_f(xr[j][2 * v + 1]);
                            float d = v0 * v0;
                            d = fmaf(v1, v1, d);
                            d = fmaf(v2, v2, d);
                            d = fmaf(v3, v3, d);
                            part[v] = part[v] + d;
                        }
                    }
                }
                total = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(reduce_row<VL>(part))));
            } else {
                float part = 0.0f;
                #pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if (256 * j + 4 * lane < KT) {
                        const float v0 = lo_f(xsq[j][0]), v1 = hi_f(xsq[j][0]);
                        const float v2 = lo_f(xsq[j][1]), v3 = hi_f(xsq[j][1]);
                        float d = v0 * v0;
                        d = fmaf(v1, v1, d);
                        d = fmaf(v2, v2, d);
                        d = fmaf(v3, v3, d);
                        part = part + d;
                    }
                }
                float one[1] = {part};
                total = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(reduce_row<1>(one))));
            }
            // (sqrtf: correctly rounded under -fhip-fp32-correctly-rounded-divide-sqrt, which __fsqrt_rn is not)
            const float inv = __fdiv_rn(1.0f, sqrtf(__fdiv_rn(total, static_cast<float>(KT)) + L.norm_eps));
            #pragma unroll
            for (int j = 0; j < NIT; ++j) {
                #pragma unroll
                for (int i = 0; i < XD; ++i) {
                    const uint32_t lo = f_h((lo_f(xr[j][i]) * inv) * lo_f(nrm[j][i]));
                    const uint32_t hi = f_h((hi_f(xr[j][i]) * inv) * hi_f(nrm[j][i]));
                    xr[j][i] = lo | (hi << 16);
                }
            }
        }
    }

    auto row_sum = [&](const Batch& b) {
        float acc[VL];
        #pragma unroll
        for (int v = 0; v < VL; ++v) acc[v] = 0.0f;
        #pragma unroll
        for (int j = 0; j < NIT; ++j) {
            if (j * EIT + koff < KT) {
                const float sf = KIND == WK_Q4 ? h_f(b.s[KIND == WK_Q4 ? j : 0]) : 0.0f;
                #pragma unroll
                for (int v = 0; v < VL; ++v)
                    acc[v] = vlane_step<KIND>(acc[v], &b.w[j][v * T::BPV / 4], &xr[j][v * T::EPV / 2], sf, cst);
            }
        }
        return reduce_row<VL>(acc);
    };

    if constexpr (EPI == EPI_SWIGLU) {
        // g0 holds row batch rb of the gate matrix (segment 0), g1 the same rows of the up
        // matrix (segment 1); the gate and up values are rounded to fp16 as two GEMVs would
        // store them, then gate[n] = fp16((g * sigmoid(g)) * u)  (QW/kernels/mlp.cl swiglu_inplace)
        static_assert(!PIPE, "one batch pair at a time");
        while (true) {
            const float sg_ = row_sum(g0.b[0]), su_ = row_sum(g1.b[0]);
            if (g == 0 && g0.b[0].yoff >= 0) {
                const float sgs = KIND == WK_I8 ? sg_ * h_f(g0.b[0].s[0]) : sg_;
                const float sus = KIND == WK_I8 ? su_ * h_f(g1.b[0].s[0]) : su_;
                const float gv = h_f(f_h(sgs)), uv = h_f(f_h(sus));
                const float sig = __fdiv_rn(1.0f, 1.0f + exp_poly(-gv));
                g0.b[0].ybase[g0.b[0].yoff] = f_h((gv * sig) * uv);
            }
            rb += nw;
            if (rb >= hnbatch) break;
            fetch(g0.b[0], rb);
            fetch(g1.b[0], rb + hnbatch);
        }
        return;
    }

    auto consume = [&](const Batch& b) {
        const float sum = row_sum(b);
        if (g == 0 && b.yoff >= 0) {
            float out;
            if constexpr (KIND == WK_I8) {
                const float s = h_f(b.s[0]);
                out = EPI == EPI_ADD ? add_residual(sum, s, h_f(b.res), true, L.add_mode) : sum * s;
            } else {
                out = EPI == EPI_ADD ? add_residual(sum, 1.0f, h_f(b.res), false, L.add_mode) : sum;
            }
            const uint16_t bits = f_h(out);
            b.ybase[b.yoff] = bits;
            if constexpr (AM) {
                const float v = h_f(bits);
                if (v > kArgmaxNone) top = rule.best(top, Cand{v, b.row0 + b.yoff});
            }
        }
    };

    auto consume_group = [&](const Group& gr, int at) {
        #pragma unroll
        for (int u = 0; u < GB; ++u)
            if (at + u * nw < hnbatch) consume(gr.b[u]);
    };
    if constexpr (!PIPE) {
        while (true) {
            consume_group(g0, rb);
            rb += step;
            if (rb >= hnbatch) break;
            fetch_group(g0, rb);
        }
    } else {
        while (true) {
            fetch_group(g1, rb + step);
            consume_group(g0, rb);
            rb += step;
            if (rb >= hnbatch) break;
            fetch_group(g0, rb + step);
            consume_group(g1, rb);
            rb += step;
            if (rb >= hnbatch) break;
        }
    }
    if constexpr (AM) {
        const Cand w = rule.best_of_wave(top);
        if (lane == 0) { L.am_v[wid] = w.v; L.am_i[wid] = w.i; }
    }
}

// ---- Q4, throughput variant --------------------------------------------------------
//
// The exact Q4 kernel above is bound by the vector ALU, not by HBM: reproducing the
// reference's sum needs one fp32 fma per weight after the nibble has become a number.
// This variant keeps the result inside the stated tolerance (max-abs/rel 1e-3, cosine
// 0.9999; the sum is still fp32, only its order changes) at about half the instructions:
//   - a nibble pair masked in place is read as two fp16 SUBNORMALS, n * 2^-24 (pairs at
//     bits 0-3/16-19) or n * 2^-20 (pairs at bits 4-7/20-23): no conversion at all;
//   - v_dot2_f32_f16 multiplies a pair by the matching pair of activations and accumulates
//     in fp32, two weights per instruction (the activations are held pre-paired);
//   - the "- 8" of every weight is applied once per 32-weight block as -8 * sum(x), and the
//     block scale multiplies the block sum once.
// 16 lanes still share a row and a wavefront still streams row batches of 4 rows with the
// same double-buffered fetch; each lane owns one scale block per K-iteration.
template <int KT, int EPI, bool PIPE, int RB, bool AM = false>
__global__ __launch_bounds__(kBlock) void gemv_q4_fast(MI_HOT_PARAMS, const SegList L) {
    constexpr int EIT = 512;                            // elements per K-iteration (16 lanes x 32)
    constexpr int NIT = (KT + EIT - 1) / EIT;
    constexpr int ROWB = KT / 2;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int g = lane % 16, r = lane / 16;
    const int koff = g * 32;
    const int m = blockIdx.y;
    x += static_cast<size_t>(m) * KT;

    struct Batch {
        uint32_t w[NIT][4];
        uint16_t s[NIT];
        uint16_t res;
        uint16_t* ybase;    // &y[m][first row of the batch], uniform
        int yoff;           // row inside the batch, -1 when the lane's row is past N
        int row0;           // first row of the batch inside its segment, uniform
    };
    const uint32_t lane_w = r * ROWB + g * 16, lane_w0 = g * 16;
    auto fetch = [&](Batch& b, int rb) {
        const Seg sg = hW1 == nullptr ? Seg{hW0, hsc0, hy0, hN0, 0} : find_segment(L, rb);
        const int row0 = (rb - sg.first) * 4;
        const bool valid = row0 + r < sg.N;
        const int rr = valid ? r : 0;
        const uint8_t* wb = sg.W + static_cast<size_t>(row0) * ROWB;
        const uint16_t* sb = sg.sc + static_cast<size_t>(row0) * (KT / 32);
        const uint32_t wo = valid ? lane_w : lane_w0;
        b.ybase = sg.y + static_cast<size_t>(m) * sg.N + row0;
        b.yoff = valid ? r : -1;
        b.row0 = row0;
        if constexpr (EPI == EPI_ADD) b.res = b.ybase[rr];
        #pragma unroll
        for (int j = 0; j < NIT; ++j) {
            const bool active = j * EIT + koff < KT;
            load_dwords<4, true>(b.w[j], wb + (active ? wo + j * 256 : wo - lane_w0));
            b.s[j] = sb[rr * (KT / 32) + (active ? j * 16 + g : 0)];
        }
    };
    // The activations are requested first and the first weights right behind them, without a
    // wait in between: loads return in order, so the pairing of x below can run while the
    // weights are still on their way.
    const int nw = gridDim.x * kWavesPerBlock;
    int rb = blockIdx.x * kWavesPerBlock + wave;
    const int wid = rb;
    const TieRule rule{L.am_chunk};
    Cand top{kArgmaxNone, 0};                                 // AM: best row so far (lanes with g == 0)
    if (rb >= hnbatch) {
        if constexpr (AM) {
            if (lane == 0) { L.am_v[wid] = kArgmaxNone; L.am_i[wid] = 0; }
        }
        return;
    }
    uint32_t raw[NIT][16];
    #pragma unroll
    for (int j = 0; j < NIT; ++j) {
        if (j * EIT + koff < KT) load_dwords<16, false>(raw[j], x + j * EIT + koff);
        else {
            #pragma unroll
            for (int i = 0; i < 16; ++i) raw[j][i] = 0u;
        }
    }
    struct Group { Batch b[PIPE ? RB : 1]; };
    constexpr int GB = PIPE ? RB : 1;
    const int first = rb;
    auto fetch_group = [&](Group& gr, int at) {
        #pragma unroll
        for (int u = 0; u < GB; ++u) fetch(gr.b[u], at + u * nw < hnbatch ? at + u * nw : first);
    };
    Group g0, g1;
    fetch_group(g0, rb);

    // xp[j][4 d + i]: activations paired for dword d of the lane's 16 weight bytes:
    // i = 0: (x0, x4), 1: (x1, x5), 2: (x2, x6), 3: (x3, x7) of elements 8 d .. 8 d + 7.
    uint32_t xp[NIT][16];
    float m8sx[NIT];                                    // -8 * sum of the block's activations
    #pragma unroll
    for (int j = 0; j < NIT; ++j) {
        float sx = 0.0f;
        #pragma unroll
        for (int i = 0; i < 16; ++i) sx += lo_f(raw[j][i]) + hi_f(raw[j][i]);
        m8sx[j] = -8.0f * sx;
        #pragma unroll
        for (int d = 0; d < 4; ++d) {
            xp[j][4 * d + 0] = __builtin_amdgcn_perm(raw[j][4 * d + 2], raw[j][4 * d + 0], 0x05040100u);
            xp[j][4 * d + 1] = __builtin_amdgcn_perm(raw[j][4 * d + 2], raw[j][4 * d + 0], 0x07060302u);
            xp[j][4 * d + 2] = __builtin_amdgcn_perm(raw[j][4 * d + 3], raw[j][4 * d + 1], 0x05040100u);
            xp[j][4 * d + 3] = __builtin_amdgcn_perm(raw[j][4 * d + 3], raw[j][4 * d + 1], 0x07060302u);
        }
    }

    auto consume = [&](const Batch& b) {
        float acc = 0.0f;
        #pragma unroll
        for (int j = 0; j < NIT; ++j) {
            if (j * EIT + koff < KT) {
                float da = 0.0f, db = 0.0f;
                #pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t v = b.w[j][d], v8 = v >> 8;
                    da = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[j][4 * d + 0]),
                                                __builtin_bit_cast(h2, v & 0x000F000Fu), da, false);
                    db = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[j][4 * d + 1]),
                                                __builtin_bit_cast(h2, v & 0x00F000F0u), db, false);
                    da = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[j][4 * d + 2]),
                                                __builtin_bit_cast(h2, v8 & 0x000F000Fu), da, false);
                    db = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[j][4 * d + 3]),
                                                __builtin_bit_cast(h2, v8 & 0x00F000F0u), db, false);
                }
                // sum over the block of x * (n - 8) = 2^24 da + 2^20 db - 8 sum(x)
                const float blk = fmaf(da, 16777216.0f, fmaf(db, 1048576.0f, m8sx[j]));
                acc = fmaf(blk, h_f(b.s[j]), acc);
            }
        }
        acc = add_from_above<8>(acc);
        acc = add_from_above<4>(acc);
        acc = add_from_above<2>(acc);
        acc = add_from_above<1>(acc);
        if (g == 0 && b.yoff >= 0) {
            const float out = EPI == EPI_ADD ? add_residual(acc, 1.0f, h_f(b.res), false, L.add_mode) : acc;
            const uint16_t bits = f_h(out);
            b.ybase[b.yoff] = bits;
            if constexpr (AM) {
                const float v = h_f(bits);
                if (v > kArgmaxNone) top = rule.best(top, Cand{v, b.row0 + b.yoff});
            }
        }
    };

    auto consume_group = [&](const Group& gr, int at) {
        #pragma unroll
        for (int u = 0; u < GB; ++u)
            if (at + u * nw < hnbatch) consume(gr.b[u]);
    };
    const int step = nw * GB;
    if constexpr (!PIPE) {
        while (true) {
            consume_group(g0, rb);
            rb += step;
            if (rb >= hnbatch) break;
            fetch_group(g0, rb);
        }
    } else {
        while (true) {
            fetch_group(g1, rb + step);
            consume_group(g0, rb);
            rb += step;
            if (rb >= hnbatch) break;
            fetch_group(g0, rb + step);
            consume_group(g1, rb);
            rb += step;
            if (rb >= hnbatch) break;
        }
    }
    if constexpr (AM) {
        const Cand w = rule.best_of_wave(top);
        if (lane == 0) { L.am_v[wid] = w.v; L.am_i[wid] = w.i; }
    }
}

// x (K halves, K % 4 == 0, 8-byte aligned) into LDS by the whole block.  Where K is long a thread
// requests four 8-byte pieces before it stores the first (one trip to memory per 4096 halves instead
// of one per 512); what is left goes piece by piece.
__device__ __forceinline__ void stage_x(uint32_t* xs, const uint16_t* x, int K) {
    const uint2* src = reinterpret_cast<const uint2*>(x);
    uint2* dst = reinterpret_cast<uint2*>(xs);
    const int n = K / 4;
    int base = 0;
    for (; base + 4 * kBlock <= n; base += 4 * kBlock) {
        uint2 t[4];
        #pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = src[base + u * kBlock + static_cast<int>(threadIdx.x)];
        #pragma unroll
        for (int u = 0; u < 4; ++u) dst[base + u * kBlock + static_cast<int>(threadIdx.x)] = t[u];
    }
    for (int i = 2 * base + static_cast<int>(threadIdx.x); i < K / 2; i += kBlock) xs[i] = reinterpret_cast<const uint32_t*>(x)[i];
}

// x for the Q4 throughput arithmetic (see gemv_q4_fast) into LDS by the whole block: a thread takes a
// scale block of 32 activations at a time, pairs them as v_dot2_f32_f16 wants them against a lane's 16
// weight bytes, and adds them up.  Layout, for `nit` K-iterations of 16 blocks: 16-byte piece q of block
// 16 j + g at uint4 index (4 j + q) 16 + g (the 16 lanes of a row read consecutive pieces), then -8 sum(x)
// of block b at float index 256 nit + b.  Blocks past K hold zeros.
__device__ __forceinline__ void stage_x_paired(uint32_t* xs, const uint16_t* x, int K, int nit) {
    u32x4* xq = reinterpret_cast<u32x4*>(xs);
    float* m8 = reinterpret_cast<float*>(xs) + 256 * nit;
    const int blocks = K / 32;
    for (int b = threadIdx.x; b < 16 * nit; b += kBlock) {
        uint32_t raw[16];
        if (b < blocks) {
            load_dwords<16, false>(raw, x + 32 * b);
        } else {
            #pragma unroll
            for (int i = 0; i < 16; ++i) raw[i] = 0u;
        }
        float sx = 0.0f;
        #pragma unroll
        for (int i = 0; i < 16; ++i) sx += lo_f(raw[i]) + hi_f(raw[i]);
        const int j = b / 16, g = b % 16;
        #pragma unroll
        for (int d = 0; d < 4; ++d) {
            u32x4 t;
            t.x = __builtin_amdgcn_perm(raw[4 * d + 2], raw[4 * d + 0], 0x05040100u);
            t.y = __builtin_amdgcn_perm(raw[4 * d + 2], raw[4 * d + 0], 0x07060302u);
            t.z = __builtin_amdgcn_perm(raw[4 * d + 3], raw[4 * d + 1], 0x05040100u);
            t.w = __builtin_amdgcn_perm(raw[4 * d + 3], raw[4 * d + 1], 0x07060302u);
            xq[(4 * j + d) * 16 + g] = t;
        }
        m8[b] = -8.0f * sx;
    }
}
constexpr size_t paired_x_lds(int K) { return static_cast<size_t>((K + 511) / 512) * 16 * 68; }

// ---- K known at run time: x is staged once per block in LDS ------------------------
// FAST (Q4, four rows per wavefront): the arithmetic of gemv_q4_fast, inside the stated tolerance, for
// every K that kernel has no instance for (the exact order is bound by the vector ALU at about 2 TB/s).
template <int KIND, int VL, int EPI, bool FAST = false>
__global__ __launch_bounds__(kBlock) void gemv_any_k(MI_HOT_PARAMS, const SegList L, int K) {
    static_assert(!FAST || (KIND == WK_Q4 && VL == 4), "the throughput arithmetic is Q4's, a scale block per lane");
    using T = WT<KIND>;
    constexpr int LPR = kWave / VL, RPW = VL;
    constexpr int EIT = kWave * T::EPV;
    constexpr int XD = VL * T::EPV / 2;
    constexpr int WD = VL * T::BPV / 4;
    constexpr int ITB = kWave * T::BPV;
    constexpr int kChunk = 8;                           // K-iterations per register buffer (at most 32 dwords per lane)
    extern __shared__ __attribute__((aligned(16))) uint32_t xs[];   // K/2 dwords of packed fp16 (FAST: see stage_x_paired)

    const int m = blockIdx.y;
    x += static_cast<size_t>(m) * K;
    const int nit = (K + EIT - 1) / EIT;
    if constexpr (FAST) stage_x_paired(xs, x, K, nit);
    else stage_x(xs, x, K);
    __syncthreads();

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int g = lane % LPR, r = lane / LPR;
    const int koff = g * VL * T::EPV;
    const Consts cst = make_consts();
    const size_t rowb = static_cast<size_t>(K) / T::EPV * T::BPV;

    for (int rb = blockIdx.x * kWavesPerBlock + wave; rb < hnbatch; rb += gridDim.x * kWavesPerBlock) {
        const Seg sg = hW1 == nullptr ? Seg{hW0, hsc0, hy0, hN0, 0} : find_segment(L, rb);
        const int row = (rb - sg.first) * RPW + r;
        const bool valid = row < sg.N;
        const int rowc = valid ? row : sg.N - 1;
        const uint8_t* row0 = sg.W + static_cast<size_t>(rowc) * rowb;
        const uint8_t* wrow = row0 + koff / T::EPV * T::BPV;
        [[maybe_unused]] const uint16_t* srow0 = sg.sc + static_cast<size_t>(rowc) * (K / 32);
        [[maybe_unused]] const uint16_t* srow = srow0 + (g * VL) / 4;
        float acc[VL];
        #pragma unroll
        for (int v = 0; v < VL; ++v) acc[v] = 0.0f;
        // The row's K-iterations go through two register buffers of kChunk iterations each: one chunk
        // is on its way while the other is multiplied, so a long row costs one memory round trip plus
        // its bytes, not a round trip per few iterations (1024 x 4096 int8: 10.5 -> 5.0 us; an lm_head of
        // 100 352 x 2048: 52 -> 38 us).  The order of the additions is the loop's.
        uint32_t wbuf[2][kChunk][WD];
        [[maybe_unused]] uint16_t sbuf[2][kChunk];
        auto fetch_chunk = [&](int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int j = j0 + u;
                if (j >= nit) break;                                  // (uniform: nothing is requested past the row's end)
                // lanes idle in a partial last iteration re-read the first bytes of the row, which every
                // row has (the value is never used; their own offset may lie past the end of the matrix)
                const bool active = j * EIT + koff < K;
                load_dwords<WD, true>(wbuf[b][u], active ? wrow + static_cast<size_t>(j) * ITB : row0);
                if constexpr (KIND == WK_Q4) sbuf[b][u] = active ? srow[j * 16] : srow0[0];
            }
        };
        auto multiply_chunk = [&](int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int j = j0 + u, k = j * EIT + koff;
                if (j < nit && k < K) {
                    if constexpr (FAST) {
                        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                        uint32_t xp[4][4];
                        #pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const u32x4 t = reinterpret_cast<const u32x4*>(xs)[(4 * j + d) * 16 + g];
                            xp[d][0] = t.x; xp[d][1] = t.y; xp[d][2] = t.z; xp[d][3] = t.w;
                        }
                        const float m8sx = reinterpret_cast<const float*>(xs)[256 * nit + 16 * j + g];
                        float da = 0.0f, db = 0.0f;
                        #pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const uint32_t v = wbuf[b][u][d], v8 = v >> 8;
                            da = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[d][0]), __builtin_bit_cast(h2, v & 0x000F000Fu), da, false);
                            db = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[d][1]), __builtin_bit_cast(h2, v & 0x00F000F0u), db, false);
                            da = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[d][2]), __builtin_bit_cast(h2, v8 & 0x000F000Fu), da, false);
                            db = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, xp[d][3]), __builtin_bit_cast(h2, v8 & 0x00F000F0u), db, false);
                        }
                        // sum over the block of x * (n - 8) = 2^24 da + 2^20 db - 8 sum(x), times the block's scale
                        const float blk = fmaf(da, 16777216.0f, fmaf(db, 1048576.0f, m8sx));
                        acc[0] = fmaf(blk, h_f(sbuf[b][u]), acc[0]);
                    } else {
                        uint32_t xr[XD];
                        #pragma unroll
                        for (int i = 0; i < XD; ++i) xr[i] = xs[k / 2 + i];
                        float sf = 0.0f;
                        if constexpr (KIND == WK_Q4) sf = h_f(sbuf[b][u]);
                        #pragma unroll
                        for (int v = 0; v < VL; ++v)
                            acc[v] = vlane_step<KIND>(acc[v], &wbuf[b][u][v * T::BPV / 4], &xr[v * T::EPV / 2], sf, cst);
                    }
                }
            }
        };
        fetch_chunk(0, 0);
        for (int j0 = 0;;) {
            if (j0 + kChunk < nit) fetch_chunk(1, j0 + kChunk);
            multiply_chunk(0, j0);
            j0 += kChunk;
            if (j0 >= nit) break;
            if (j0 + kChunk < nit) fetch_chunk(0, j0 + kChunk);
            multiply_chunk(1, j0);
            j0 += kChunk;
            if (j0 >= nit) break;
        }
        const float sum = reduce_row<VL>(acc);
        if (g == 0 && valid) {
            uint16_t* yp = sg.y + static_cast<size_t>(m) * sg.N + row;
            float out;
            if constexpr (KIND == WK_I8) {
                const float s = h_f(sg.sc[row]);
                out = EPI == EPI_ADD ? add_residual(sum, s, h_f(*yp), true, L.add_mode) : sum * s;
            } else {
                out = EPI == EPI_ADD ? add_residual(sum, 1.0f, h_f(*yp), false, L.add_mode) : sum;
            }
            *yp = f_h(out);
        }
    }
}

// out[c] = fp16( silu(g) * u ), g and u the two row sums (scaled for int8).
// SM/kernels/block_fused_int8.cl:176-236, SM/kernels/block_fused.cl:473-526.
template <int KIND, int VL>
__global__ __launch_bounds__(kBlock) void gate_up_silu_any_k(const uint16_t* __restrict__ x,
                                                             const uint8_t* __restrict__ Wg,
                                                             const uint16_t* __restrict__ sg,
                                                             const uint8_t* __restrict__ Wu,
                                                             const uint16_t* __restrict__ su,
                                                             uint16_t* __restrict__ out, int N, int K) {
    using T = WT<KIND>;
    constexpr int LPR = kWave / VL, RPW = VL;
    constexpr int EIT = kWave * T::EPV;
    constexpr int XD = VL * T::EPV / 2;
    constexpr int WD = VL * T::BPV / 4;
    constexpr int ITB = kWave * T::BPV;
    constexpr int kChunk = 2;                           // K-iterations of each matrix per register buffer (4 and 8 measured no better)
    extern __shared__ uint32_t xs[];
    stage_x(xs, x, K);
    __syncthreads();

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int g = lane % LPR, r = lane / LPR;
    const int koff = g * VL * T::EPV;
    const Consts cst = make_consts();
    const size_t rowb = static_cast<size_t>(K) / T::EPV * T::BPV;
    const int nit = (K + EIT - 1) / EIT;
    const int nbatch = (N + RPW - 1) / RPW;

    for (int rb = blockIdx.x * kWavesPerBlock + wave; rb < nbatch; rb += gridDim.x * kWavesPerBlock) {
        const int row = rb * RPW + r;
        const bool valid = row < N;
        const int rowc = valid ? row : N - 1;
        const size_t off0 = static_cast<size_t>(rowc) * rowb;
        const size_t off = off0 + koff / T::EPV * T::BPV;
        float ag[VL], au[VL];
        #pragma unroll
        for (int v = 0; v < VL; ++v) { ag[v] = 0.0f; au[v] = 0.0f; }
        // two register buffers of kChunk K-iterations of both matrices, as in gemv_any_k: one on its
        // way while the other is multiplied; the additions keep the loop's order
        uint32_t gbuf[2][kChunk][WD], ubuf[2][kChunk][WD];
        auto fetch_chunk = [&](int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int j = j0 + u;
                if (j >= nit) break;
                // lanes idle in a partial last iteration re-read the first bytes of the row, which every
                // row has (the value is never used; their own offset may lie past the end of the matrix)
                const size_t at = j * EIT + koff < K ? off + static_cast<size_t>(j) * ITB : off0;
                load_dwords<WD, true>(gbuf[b][u], Wg + at);
                load_dwords<WD, true>(ubuf[b][u], Wu + at);
            }
        };
        auto multiply_chunk = [&](int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int j = j0 + u, k = j * EIT + koff;
                if (j < nit && k < K) {
                    uint32_t xr[XD];
                    #pragma unroll
                    for (int i = 0; i < XD; ++i) xr[i] = xs[k / 2 + i];
                    #pragma unroll
                    for (int v = 0; v < VL; ++v) {
                        ag[v] = vlane_step<KIND>(ag[v], &gbuf[b][u][v * T::BPV / 4], &xr[v * T::EPV / 2], 0.0f, cst);
                        au[v] = vlane_step<KIND>(au[v], &ubuf[b][u][v * T::BPV / 4], &xr[v * T::EPV / 2], 0.0f, cst);
                    }
                }
            }
        };
        fetch_chunk(0, 0);
        for (int j0 = 0;;) {
            if (j0 + kChunk < nit) fetch_chunk(1, j0 + kChunk);
            multiply_chunk(0, j0);
            j0 += kChunk;
            if (j0 >= nit) break;
            if (j0 + kChunk < nit) fetch_chunk(0, j0 + kChunk);
            multiply_chunk(1, j0);
            j0 += kChunk;
            if (j0 >= nit) break;
        }
        float gs = reduce_row<VL>(ag);
        float us = reduce_row<VL>(au);
        if (g == 0 && valid) {
            if constexpr (KIND == WK_I8) { gs = gs * h_f(sg[row]); us = us * h_f(su[row]); }
            out[row] = f_h((gs / (1.0f + exp_poly(-gs))) * us);
        }
    }
}

// w16[n,k] = fp16(f32(q[n,k]) * f32(scale[n]))   (LV/kernels/lfm2_ops.cl:731-743)
__global__ __launch_bounds__(256) void dequant_int8_kernel(const int8_t* __restrict__ q,
                                                           const uint16_t* __restrict__ sc,
                                                           uint16_t* __restrict__ w16, size_t total, int K) {
    for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull)
        w16[i] = f_h(static_cast<float>(q[i]) * h_f(sc[i / K]));
}

// w8[n,k] = nibble(n,k) - 8   (LF/kernels/gemv_m1_q4.cl:31-40)
__global__ __launch_bounds__(256) void unpack_q4_kernel(const uint8_t* __restrict__ p,
                                                        int8_t* __restrict__ w8, size_t nbytes) {
    for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < nbytes; i += gridDim.x * 256ull) {
        const uint8_t b = p[i];
        w8[2 * i] = static_cast<int8_t>(static_cast<int>(b & 0xF) - 8);
        w8[2 * i + 1] = static_cast<int8_t>(static_cast<int>(b >> 4) - 8);
    }
}

// ---- launch side -------------------------------------------------------------------

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Wavefronts that one launch keeps resident when it streams many row batches: 3 blocks of
// 4 wavefronts per CU (measured best for the pipelined kernels on MI355X).
inline int resident_waves() { return device_info().cus * 3 * kWavesPerBlock; }

// Widest lane tile that still gives every SIMD of the chip a wavefront; when no tile
// reaches that, the narrowest one (most wavefronts).  A tile of VL fits when a lane's
// VL virtual lanes are whole in the K tail.
int pick_vl(WeightKind kind, int M, long rows, int K) {
    const int epv = kind == WK_Q4 ? 8 : 4;
    int max_vl = kind == WK_F16 ? 2 : 4;
    // The kernels that hold x in registers spend K VL / 128 of them on it: at a long K the wide
    // tiles run short (K = 4864 with four rows per lane spills) and stream at half the rate of the
    // one-row tile.  Cold, 16 384 rows, four / two / one row per lane, us: int8 K = 4864 31.0 / 23.1 /
    // 15.0, K = 4608 25.6 / 22.0 / 14.4, K = 2560 11.3 / 9.8 / 9.6; Q4 K = 4608 17.0 / 13.5 / 11.6, K = 2560
    // 7.6 / 7.8 / 8.2; fp16 K = 4864 - / 28.8 / 27.2.  (The kernel with x in LDS, for every other long K,
    // keeps the wide tile: int8 16 384 x 4096 in 18.8 / 19.3 / 25.3 us.)
    // K = 1536, int8 and fp16: 32 768 rows 13.6 / 11.1 / 10.5 us, 49 152 rows 16.7 / 14.6 / 14.4 us (int8), fp16
    // 18.3 / 17.4 and 25.1 / 24.3 us at two / one; Q4 there, and every kind at K = 1024 and 576, is fastest
    // with four.
    if (K == 4608 || K == 4864) max_vl = 1;
    else if ((K == 2560 || K == 2048) && kind != WK_Q4) max_vl = 2;
    else if (K == 1536 && kind != WK_Q4) max_vl = 1;
    const long waves_wanted = 4L * device_info().cus;
    int narrowest = 1;
    for (int vl = max_vl; vl >= 1; vl >>= 1) {
        if (K % (vl * epv) != 0) continue;
        narrowest = vl;
        if (static_cast<long>(M) * ((rows + vl - 1) / vl) >= waves_wanted) return vl;
    }
    return narrowest;
}

// Row batches a pipelined wavefront fetches at once: enough for about 3.5 KB of weights.
constexpr int group_size(int kind, int K, int vl) {
    const int batch_bytes = vl * (K / (kind == WK_Q4 ? 8 : 4)) * (kind == WK_F16 ? 8 : 4);
    return batch_bytes <= 1280 ? 4 : (batch_bytes <= 2560 ? 2 : 1);
}

struct Plan {
    SegList L;
    dim3 grid;
    bool pipe;
};

Plan make_plan(const GemvCall* calls, int n, int vl) {
    Plan p{};
    int first = 0;
    for (int i = 0; i < n; ++i) {
        p.L.s[i] = Seg{static_cast<const uint8_t*>(calls[i].W), static_cast<const uint16_t*>(calls[i].scale),
                       static_cast<uint16_t*>(calls[i].y), calls[i].N, first};
        first += (calls[i].N + vl - 1) / vl;
    }
    p.L.nseg = n;
    p.L.nbatch = first;
    p.L.norm_w = static_cast<const uint16_t*>(calls[0].norm_w);
    p.L.norm_eps = calls[0].norm_eps;
    p.L.add_mode = calls[0].add_mode;
    p.L.am_v = nullptr;
    p.L.am_i = nullptr;
    p.L.am_chunk = 1;
    if (calls[0].am_v && calls[0].am_np > 0) {
        p.L.am_v = calls[0].am_v;
        p.L.am_i = calls[0].am_i;
        p.L.am_chunk = (calls[0].N + calls[0].am_np - 1) / calls[0].am_np;
    }
    const int cap = resident_waves();
    int waves = first;
    p.pipe = false;
    if (first > cap) {
        // several batches per wavefront, the same number for all of them (+-1)
        const int per_wave = (first + cap - 1) / cap;
        waves = (first + per_wave - 1) / per_wave;
        // Long streams: every resident slot gets a wavefront, and the batches that do not divide
        // evenly go to the lowest-numbered wavefronts.  Those belong to the blocks that reach a
        // CU first, and the CU serves its oldest wavefronts first: with equal shares they finish
        // about a microsecond ahead of the second block's and two ahead of the third's (measured
        // with per-wavefront clocks), so they are the ones that can take one batch more.
        if (first >= 8L * cap) waves = cap;
        p.pipe = true;
    }
    p.grid = dim3((waves + kWavesPerBlock - 1) / kWavesPerBlock, calls[0].M, 1);
    return p;
}

template <int KIND, int VL, int EPI>
bool launch_kind_vl(hipStream_t s, const GemvCall* calls, int n) {
    const Plan p = make_plan(calls, n, VL);
    const auto* x = static_cast<const uint16_t*>(calls[0].x);
    const int K = calls[0].K;
#define MI_FIXED(KT, PIPE_OK)                                                                            \
    case KT:                                                                                             \
        if (PIPE_OK && p.pipe) {                                                                         \
            constexpr int kRB = group_size(KIND, KT, VL);                                                \
            hipLaunchKernelGGL((gemv_fixed_k<KIND, KT, VL, EPI, PIPE_OK, kRB>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        } else {                                                                                         \
            hipLaunchKernelGGL((gemv_fixed_k<KIND, KT, VL, EPI, false, 1>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        }                                                                                                \
        break;
    if constexpr (EPI == EPI_STORE && KIND != WK_Q4) {
        if (p.L.am_v) {
#define MI_FIXED_AM(KT, PIPE_OK)                                                                         \
    case KT:                                                                                             \
        if (PIPE_OK && p.pipe) {                                                                         \
            constexpr int kRB = group_size(KIND, KT, VL);                                                \
            hipLaunchKernelGGL((gemv_fixed_k<KIND, KT, VL, EPI, PIPE_OK, kRB, true>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        } else {                                                                                         \
            hipLaunchKernelGGL((gemv_fixed_k<KIND, KT, VL, EPI, false, 1, true>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        }                                                                                                \
        break;
            switch (K) {
                MI_FIXED_AM(576, true)
                MI_FIXED_AM(896, true)
                MI_FIXED_AM(960, true)
                MI_FIXED_AM(1024, true)
                MI_FIXED_AM(1536, true)
                MI_FIXED_AM(2048, false)
                MI_FIXED_AM(4864, false)
                default: MI_ERROR_FMT("gemv: no fused argmax for K=%d", K); return false;
            }
#undef MI_FIXED_AM
            return MI_HIP_OK(hipGetLastError());
        }
    }
    switch (K) {
        MI_FIXED(576, true)
        MI_FIXED(896, true)
        MI_FIXED(960, true)           // SmolLM2-360M's width
        MI_FIXED(1024, true)
        MI_FIXED(1536, true)
        MI_FIXED(2048, false)         // the width of the 1-2 B models of the same families: the kernel with x in LDS
                                      // took 27.3 us for int8 65 536 x 2048 where this one takes 24.0 (Q4: 38.1 -> 16.0)
        MI_FIXED(2560, false)         // LFM2's K values beside 1024: the reference ships kernels for exactly these
        MI_FIXED(4608, false)         // (LF/kernels/gemv_m1_int8.cl:155-255, gemv_m1_q4.cl:128-281)
        MI_FIXED(4864, false)
        default: {
            const size_t lds = static_cast<size_t>(K) * 2;
            hipLaunchKernelGGL((gemv_any_k<KIND, VL, EPI>), p.grid, dim3(kBlock), lds, s, MI_HOT_ARGS(x, p.L), p.L, K);
        }
    }
#undef MI_FIXED
    return MI_HIP_OK(hipGetLastError());
}

// Gate and up projection with the SwiGLU behind them: calls[0] = gate, calls[1] = up.  A
// wavefront takes the same row batch of both matrices, so the launch has as many batches as one
// matrix; the kernels that keep x in registers only, without the pipelined variant.
template <int KIND, int VL>
bool launch_swiglu_vl(hipStream_t s, const GemvCall* calls) {
    Plan p = make_plan(calls, 2, VL);
    p.L.nbatch = p.L.s[1].first;
    const int cap = resident_waves();
    const int waves = p.L.nbatch < cap ? p.L.nbatch : cap;
    p.grid = dim3((waves + kWavesPerBlock - 1) / kWavesPerBlock, 1, 1);
    const auto* x = static_cast<const uint16_t*>(calls[0].x);
#define MI_SWIGLU(KT) \
    case KT: hipLaunchKernelGGL((gemv_fixed_k<KIND, KT, VL, EPI_SWIGLU, false, 1>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); break;
    switch (calls[0].K) {
        MI_SWIGLU(576)
        MI_SWIGLU(896)
        MI_SWIGLU(960)
        MI_SWIGLU(1024)
        MI_SWIGLU(1536)
        MI_SWIGLU(2048)
        default: MI_ERROR_FMT("gemv: no SwiGLU epilogue for K=%d", calls[0].K); return false;
    }
#undef MI_SWIGLU
    return MI_HIP_OK(hipGetLastError());
}

// Throughput variant of Q4 (see gemv_q4_fast): K known at compile time and a whole number of
// 32-weight blocks per lane, i.e. the 16-byte lane tile.
template <int EPI>
bool launch_q4_fast(hipStream_t s, const GemvCall* calls, int n, bool* taken) {
    const int K = calls[0].K;
    *taken = true;
    const Plan p = make_plan(calls, n, 4);
    const auto* x = static_cast<const uint16_t*>(calls[0].x);
#define MI_Q4F(KT, AM)                                                                               \
    case KT:                                                                                         \
        if (p.pipe) {                                                                                \
            constexpr int kRB = group_size(WK_Q4, KT, 4);                                            \
            hipLaunchKernelGGL((gemv_q4_fast<KT, EPI, true, kRB, AM>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        } else {                                                                                     \
            hipLaunchKernelGGL((gemv_q4_fast<KT, EPI, false, 1, AM>), p.grid, dim3(kBlock), 0, s, MI_HOT_ARGS(x, p.L), p.L); \
        }                                                                                            \
        break;
    if constexpr (EPI == EPI_STORE) {
        if (p.L.am_v) {
            switch (K) {
                MI_Q4F(576, true)
                MI_Q4F(896, true)
                MI_Q4F(960, true)
                MI_Q4F(1024, true)
                MI_Q4F(1536, true)
                default: *taken = false; return true;
            }
            return MI_HIP_OK(hipGetLastError());
        }
    }
    switch (K) {
        MI_Q4F(576, false)
        MI_Q4F(896, false)
        MI_Q4F(960, false)
        MI_Q4F(1024, false)
        MI_Q4F(1536, false)
        MI_Q4F(2048, false)
        MI_Q4F(2560, false)
        default: {
            // every other K: the same arithmetic with x in LDS (where it fits the 64 KB a launch gets unasked)
            const size_t lds = paired_x_lds(K);
            if (lds > 65536) { *taken = false; return true; }
            hipLaunchKernelGGL((gemv_any_k<WK_Q4, 4, EPI, true>), p.grid, dim3(kBlock), lds, s, MI_HOT_ARGS(x, p.L), p.L, K);
        }
    }
#undef MI_Q4F
    return MI_HIP_OK(hipGetLastError());
}

template <int KIND, int EPI>
bool launch_kind(hipStream_t s, const GemvCall* calls, int n, int vl) {
    if constexpr (KIND != WK_F16) {
        if (vl == 4) return launch_kind_vl<KIND, 4, EPI>(s, calls, n);
    }
    if (vl == 2) return launch_kind_vl<KIND, 2, EPI>(s, calls, n);
    return launch_kind_vl<KIND, 1, EPI>(s, calls, n);
}

bool check_call(const GemvCall& c) {
    const int epv = c.kind == WK_Q4 ? 32 : 4;               // Q4 needs whole scale blocks
    if (c.M < 1 || c.N < 1 || c.K < 1 || c.K % epv != 0) {
        MI_ERROR_FMT("gemv: unsupported shape M=%d N=%d K=%d (K must be a multiple of %d)", c.M, c.N,
                     c.K, epv);
        return false;
    }
    if (c.K > 32768 || c.M > 65535) {
        MI_ERROR_FMT("gemv: K=%d or M=%d beyond the supported range", c.K, c.M);
        return false;
    }
    if (!c.x || !c.W || !c.y || !aligned(c.x, 16) || !aligned(c.W, 16) || !aligned(c.y, 2) ||
        (c.M > 1 && (static_cast<size_t>(c.K) * 2) % 16 != 0) ||
        (c.kind != WK_F16 && (!c.scale || !aligned(c.scale, 2)))) {
        MI_ERROR_FMT("gemv: null or misaligned operand (x and W need 16-byte alignment)");
        return false;
    }
    return true;
}

}  // namespace

// Kernels that can leave argmax candidates: the ones that keep x in registers (int8, fp16) and the
// Q4 throughput kernel where launch_gemv_group would take it.
bool gemv_takes_argmax(hipStream_t s, const GemvCall& c) {
    if (c.M != 1 || c.epi != EPI_STORE) return false;
    if (c.kind == WK_Q4)
        return !c.norm_w && gemv_mode(s) == 1 && pick_vl(c.kind, 1, c.N, c.K) == 4 &&
               (c.K == 576 || c.K == 896 || c.K == 960 || c.K == 1024 || c.K == 1536);
    return gemv_takes_norm(c.kind, c.K);
}

int gemv_argmax_slots(const GemvCall& c) {
    const Plan p = make_plan(&c, 1, pick_vl(c.kind, c.M, c.N, c.K));
    return static_cast<int>(p.grid.x) * kWavesPerBlock;
}

bool gemv_takes_swiglu(WeightKind, int K) {
    return K == 576 || K == 896 || K == 960 || K == 1024 || K == 1536 || K == 2048;
}

// The kernels that keep x in registers (every weight kind; Q4 through the exact kernel, not the
// throughput one).
bool gemv_takes_norm(WeightKind, int K) {
    return K == 576 || K == 896 || K == 960 || K == 1024 || K == 1536 || K == 2048 || K == 4864;
}

bool launch_gemv_group(hipStream_t s, const GemvCall* calls, int n) {
    if (n < 1 || n > kMaxSegments) {
        MI_ERROR_FMT("gemv: %d segments in one launch (1..%d allowed)", n, kMaxSegments);
        return false;
    }
    long rows = 0;
    for (int i = 0; i < n; ++i) {
        if (!check_call(calls[i])) return false;
        if (calls[i].x != calls[0].x || calls[i].K != calls[0].K || calls[i].kind != calls[0].kind ||
            calls[i].M != calls[0].M || calls[i].epi != calls[0].epi || calls[i].norm_w != calls[0].norm_w ||
            calls[i].norm_eps != calls[0].norm_eps || calls[i].add_mode != calls[0].add_mode) {
            MI_ERROR_FMT("gemv: segments of one launch must share x, K, M, weight kind, epilogue and norm");
            return false;
        }
        rows += calls[i].N;
    }
    const GemvCall& c = calls[0];
    if (c.am_v && !(n == 1 && c.am_i && c.am_np > 0 && gemv_takes_argmax(s, c))) {
        MI_ERROR_FMT("gemv: the fused argmax takes one segment, M = 1 and a kernel that keeps x in registers "
                     "(kind=%d K=%d)", static_cast<int>(c.kind), c.K);
        return false;
    }
    if (c.norm_w && !(gemv_takes_norm(c.kind, c.K) && aligned(c.norm_w, 16))) {
        MI_ERROR_FMT("gemv: no fused RMSNorm for kind=%d K=%d (or misaligned norm weights)", static_cast<int>(c.kind), c.K);
        return false;
    }
    // (SwiGLU: a wavefront takes a row batch of both matrices, and the launch is short: the
    //  narrow tiles win until there are two batch pairs per wavefront and more.  Measured in a
    //  decode step at 2 x 4864 rows, K = 896: one row per wavefront 4 % faster per token than two)
    const int vl = pick_vl(c.kind, c.M, c.epi == EPI_SWIGLU ? rows / 8 : rows, c.K);
    if (c.epi == EPI_SWIGLU) {
        if (n != 2 || calls[0].N != calls[1].N || c.M != 1 || !gemv_takes_swiglu(c.kind, c.K)) {
            MI_ERROR_FMT("gemv: the SwiGLU epilogue takes a gate and an up matrix of equal N, M = 1 "
                         "and K in {576, 896, 960, 1024, 1536, 2048} (n=%d kind=%d K=%d)", n, static_cast<int>(c.kind), c.K);
            return false;
        }
        if (c.kind == WK_I8) {
            if (vl == 4) return launch_swiglu_vl<WK_I8, 4>(s, calls);
            if (vl == 2) return launch_swiglu_vl<WK_I8, 2>(s, calls);
            return launch_swiglu_vl<WK_I8, 1>(s, calls);
        }
        if (c.kind == WK_Q4) {
            if (vl == 4) return launch_swiglu_vl<WK_Q4, 4>(s, calls);
            if (vl == 2) return launch_swiglu_vl<WK_Q4, 2>(s, calls);
            return launch_swiglu_vl<WK_Q4, 1>(s, calls);
        }
        return vl == 2 ? launch_swiglu_vl<WK_F16, 2>(s, calls) : launch_swiglu_vl<WK_F16, 1>(s, calls);
    }
    const bool add = c.epi == EPI_ADD;
    if (c.kind == WK_Q4 && vl == 4 && gemv_mode(s) == 1 && !c.norm_w) {       // (the throughput kernel has no norm)
        bool taken = false;
        const bool ok = add ? launch_q4_fast<EPI_ADD>(s, calls, n, &taken) : launch_q4_fast<EPI_STORE>(s, calls, n, &taken);
        if (taken) return ok;
    }
    switch (c.kind) {
        case WK_F16: return add ? launch_kind<WK_F16, EPI_ADD>(s, calls, n, vl) : launch_kind<WK_F16, EPI_STORE>(s, calls, n, vl);
        case WK_I8:  return add ? launch_kind<WK_I8, EPI_ADD>(s, calls, n, vl) : launch_kind<WK_I8, EPI_STORE>(s, calls, n, vl);
        case WK_Q4:  return add ? launch_kind<WK_Q4, EPI_ADD>(s, calls, n, vl) : launch_kind<WK_Q4, EPI_STORE>(s, calls, n, vl);
    }
    return false;
}

bool launch_gemv(hipStream_t s, const GemvCall& c) { return launch_gemv_group(s, &c, 1); }

bool launch_gate_up_silu(hipStream_t s, WeightKind kind, int N, int K, const void* x, const void* Wg,
                         const void* sg, const void* Wu, const void* su, void* out) {
    if (kind == WK_Q4 || N < 1 || K < 4 || K % 4 != 0 || K > 32768) {
        MI_ERROR_FMT("gate_up_silu: unsupported kind=%d N=%d K=%d", static_cast<int>(kind), N, K);
        return false;
    }
    if (!aligned(x, 16) || !aligned(Wg, 16) || !aligned(Wu, 16)) {
        MI_ERROR_FMT("gate_up_silu: x and W must be 16-byte aligned");
        return false;
    }
    const int vl = pick_vl(kind, 1, N, K);
    const int nbatch = (N + vl - 1) / vl;
    const int cap = resident_waves();
    const int waves = nbatch < cap ? nbatch : cap;
    const dim3 grid((waves + kWavesPerBlock - 1) / kWavesPerBlock, 1, 1);
    const size_t lds = static_cast<size_t>(K) * 2;
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* g8 = static_cast<const uint8_t*>(Wg);
    const auto* u8 = static_cast<const uint8_t*>(Wu);
    const auto* sgp = static_cast<const uint16_t*>(sg);
    const auto* sup = static_cast<const uint16_t*>(su);
    auto* o = static_cast<uint16_t*>(out);
#define MI_GUS(KIND, VL) \
    hipLaunchKernelGGL((gate_up_silu_any_k<KIND, VL>), grid, dim3(kBlock), lds, s, xp, g8, sgp, u8, sup, o, N, K)
    if (kind == WK_I8) {
        if (vl == 4) MI_GUS(WK_I8, 4); else if (vl == 2) MI_GUS(WK_I8, 2); else MI_GUS(WK_I8, 1);
    } else {
        if (vl >= 2) MI_GUS(WK_F16, 2); else MI_GUS(WK_F16, 1);
    }
#undef MI_GUS
    return MI_HIP_OK(hipGetLastError());
}

bool launch_dequant_int8(hipStream_t s, const void* q, const void* scale, int N, int K, void* w16) {
    if (N < 1 || K < 1) { MI_ERROR_FMT("dequant_int8: bad shape N=%d K=%d", N, K); return false; }
    const size_t total = static_cast<size_t>(N) * K;
    const size_t blocks = (total + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks < 65536 ? blocks : 65536);
    hipLaunchKernelGGL(dequant_int8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const int8_t*>(q),
                       static_cast<const uint16_t*>(scale), static_cast<uint16_t*>(w16), total, K);
    return MI_HIP_OK(hipGetLastError());
}

bool launch_unpack_q4(hipStream_t s, const void* p, int N, int K, void* w8) {
    if (N < 1 || K < 2 || K % 2) { MI_ERROR_FMT("unpack_q4: bad shape N=%d K=%d", N, K); return false; }
    const size_t nbytes = static_cast<size_t>(N) * (K / 2);
    const size_t blocks = (nbytes + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks < 65536 ? blocks : 65536);
    hipLaunchKernelGGL(unpack_q4_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(p),
                       static_cast<int8_t*>(w8), nbytes);
    return MI_HIP_OK(hipGetLastError());
}

}  // namespace mi
