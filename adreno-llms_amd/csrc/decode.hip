// A Qwen2-shaped greedy decode step that stays on the device: the small kernels that sit between
// the projections (QW/kernels/{embedding,rmsnorm,bias_add,rope,attention,mlp,utils}.cl), the
// projections themselves as GEMV launches that also carry the RMSNorm ahead of them or the
// residual add behind them, and the argmax.  Graph of a step:
// QW/src/model.cpp:243-376, QW/src/layers/attention.cpp:336-674, QW/src/layers/mlp.cpp:97-237.
//
// Position and token live in device memory (the reference's counter buffer, QW/src/model.cpp:
// 490-500): every kernel reads them there and the last kernel of a step advances them, so a step
// is the same sequence of launches with the same arguments at every position: one captured
// graph replays for the whole generation, and no token returns to the host between steps.
//
// These kernels are the harness around the matmul path, not the path: they are written for
// exactness against the CPU restatement (same operations in the same order, so that the token
// lists can be compared for identity), and are launch-bound at batch 1 whatever they do.
#include "common.h"
#include "device_math.h"
#include "../../include/mi_decode.h"
#include "../../include/mi_linear.h"

#include <cmath>
#include <vector>

namespace mi {
namespace {

struct State {
    int pos;
    int token;
    int next;       // written by the argmax, moved into token by advance_kernel
};

__device__ __forceinline__ float rcp_rn(float x) { return __fdiv_rn(1.0f, x); }

// h[c] = embed[token][c]   (QW/kernels/embedding.cl).  The first launch of a step also copies the
// rotary table's row of the current position to rope_now (cosines, then sines: 2 D values), so
// that the attention launches of the step find it without waiting for the position first.
__global__ void embed_kernel(const uint16_t* __restrict__ embed, const State* __restrict__ st,
                             uint16_t* __restrict__ h, int hidden, int vocab, const uint16_t* __restrict__ cosT,
                             const uint16_t* __restrict__ sinT, uint16_t* __restrict__ rope_now, int D, int max_pos) {
    int t = st->token;
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);
    int pos = st->pos;
    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
        rope_now[c] = cosT[static_cast<size_t>(pos) * D + c];
        rope_now[D + c] = sinT[static_cast<size_t>(pos) * D + c];
    }
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) h[c] = embed[static_cast<size_t>(t) * hidden + c];
}

// out[c] = fp16((x[c] * inv) * w[c]), inv = 1 / sqrt(mean(x^2) + eps); the sum of squares runs
// over 64 work-items in float4 strides and a 32..1 tree (QW/kernels/rmsnorm.cl).  One wavefront.
// Used where the norm cannot ride in the projection's own launch (see mi_decoder_step).
__global__ __launch_bounds__(64) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                     uint16_t* __restrict__ out, int cols, float eps) {
    // Work-item lid owns the float4 groups lid, lid + 64, ...: it squares and normalises the
    // same elements, so x and w are read once, all loads are in flight together, and the
    // kernel costs one memory round trip.  Up to kGroups groups per work-item live in registers
    // (cols <= 256 kGroups); the tail that is not a whole group, and longer rows, go through memory.
    constexpr int kGroups = 8;
    const int lid = threadIdx.x, c4n = cols >> 2;
    x += static_cast<size_t>(blockIdx.x) * cols;       // block b takes row b (a prompt's rows; one row in a decode step)
    out += static_cast<size_t>(blockIdx.x) * cols;
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    u16x4 xv[kGroups], wv[kGroups];
    float acc = 0.0f;
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        const int c4 = lid + 64 * g;
        if (c4 < c4n) {
            xv[g] = *reinterpret_cast<const u16x4*>(x + 4 * c4);
            wv[g] = *reinterpret_cast<const u16x4*>(w + 4 * c4);
        }
    }
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        if (lid + 64 * g < c4n) {
            const float v0 = h_f(xv[g][0]), v1 = h_f(xv[g][1]), v2 = h_f(xv[g][2]), v3 = h_f(xv[g][3]);
            float d = v0 * v0;
            d = fmaf(v1, v1, d);
            d = fmaf(v2, v2, d);
            d = fmaf(v3, v3, d);
            acc = acc + d;
        }
    }
    for (int c4 = lid + 64 * kGroups; c4 < c4n; c4 += 64) {           // rows longer than the registers hold
        float v[4];
        #pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = h_f(x[4 * c4 + e]);
        float d = v[0] * v[0];
        d = fmaf(v[1], v[1], d);
        d = fmaf(v[2], v[2], d);
        d = fmaf(v[3], v[3], d);
        acc = acc + d;
    }
    for (int c = c4n * 4 + lid; c < cols; c += 64) {                    // cols not a multiple of 4
        const float v = h_f(x[c]);
        acc = fmaf(v, v, acc);
    }
    #pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float o = __shfl_down(acc, s, 64);      // work-item t adds work-item t + s
        acc = acc + o;
    }
    const float total = __shfl(acc, 0, 64);
    // sqrtf is the correctly rounded one (-fhip-fp32-correctly-rounded-divide-sqrt); the
    // __fsqrt_rn intrinsic is not, despite its name: it is off by an ulp for one input in six
    const float inv = rcp_rn(sqrtf(__fdiv_rn(total, static_cast<float>(cols)) + eps));
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        const int c4 = lid + 64 * g;
        if (c4 < c4n) {
            u16x4 o;
            #pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = f_h((h_f(xv[g][e]) * inv) * h_f(wv[g][e]));
            *reinterpret_cast<u16x4*>(out + 4 * c4) = o;
        }
    }
    for (int c4 = lid + 64 * kGroups; c4 < c4n; c4 += 64)
        for (int e = 0; e < 4; ++e) out[4 * c4 + e] = f_h((h_f(x[4 * c4 + e]) * inv) * h_f(w[4 * c4 + e]));
    for (int c = c4n * 4 + lid; c < cols; c += 64) out[c] = f_h((h_f(x[c]) * inv) * h_f(w[c]));
}

// One block per query head: q/k/v bias (QW/kernels/bias_add.cl), rotary embedding of q and k at the
// current position (QW/kernels/rope.cl), k and v into the caches (rows as QW/src/layers/
// attention.cpp:560-600), then single-query grouped-query attention (QW/kernels/attention.cl:
// gqa_attn_scores, gqa_softmax, gqa_attn_out); each value rounded to fp16 where the separate
// kernels would store it.  Sums run in the order the CPU restatement uses: the score over D in
// float4 groups, the softmax denominator over the keys in index order, the output over the keys
// in index order.
// Every head of a group prepares the group's k and v of the current position for itself (in
// LDS; the values are the same in all of them) and reads only older rows from the caches; the
// group's first head writes the new row.  raw = the projections' outputs; q_out, k_out, v_out
// receive them after bias and rotary embedding.
// Dynamic LDS: 6 bytes per position (fp32 exponentials, fp16 scores) + 6 D bytes.
__global__ __launch_bounds__(256) void rope_attention_kernel(const uint16_t* __restrict__ q_raw, const uint16_t* __restrict__ k_raw,
                                      const uint16_t* __restrict__ v_raw, const uint16_t* __restrict__ bq,
                                      const uint16_t* __restrict__ bk, const uint16_t* __restrict__ bv,
                                      const uint16_t* __restrict__ cosT, const uint16_t* __restrict__ sinT,
                                      uint16_t* __restrict__ kc, uint16_t* __restrict__ vc,
                                      uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out,
                                      uint16_t* __restrict__ v_out, uint16_t* __restrict__ out,
                                      const State* __restrict__ st, int n_heads, int n_kv_heads, int D, int max_pos,
                                      float scale) {
    extern __shared__ __attribute__((aligned(16))) uint16_t qv[];          // q, then k and v of the current position:
    uint16_t* kcur = qv + D;                                               // 3 D halves (a multiple of 8 bytes)
    uint16_t* vcur = kcur + D;
    float* ex = reinterpret_cast<float*>(vcur + D);                        // [max_pos] exponentials
    uint16_t* sc = reinterpret_cast<uint16_t*>(ex + max_pos);              // [max_pos] scores
    __shared__ float red[64];
    __shared__ float inv_s;
    int pos = st->pos;
    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    const int nrep = n_heads / n_kv_heads;
    const int seq_k = pos + 1, qh = blockIdx.x, kvd = n_kv_heads * D, kvh = qh / nrep, hd2 = D / 2;
    const bool writer = qh % nrep == 0;
    const int tid = threadIdx.x, nt = blockDim.x;
    const uint16_t* cr = cosT + static_cast<size_t>(pos) * D;
    const uint16_t* sr = sinT + static_cast<size_t>(pos) * D;
    for (int i = tid; i < hd2; i += nt) {
        const float c = h_f(cr[i]), sn = h_f(sr[i]);
        {
            const uint16_t* buf = q_raw + qh * D;
            const uint16_t* bias = bq + qh * D;
            const float x1 = h_f(f_h(h_f(buf[i]) + h_f(bias[i])));
            const float x2 = h_f(f_h(h_f(buf[i + hd2]) + h_f(bias[i + hd2])));
            const uint16_t r1 = f_h(fmaf(x1, c, -(x2 * sn))), r2 = f_h(fmaf(x2, c, x1 * sn));
            qv[i] = r1;
            qv[i + hd2] = r2;
            q_out[qh * D + i] = r1;
            q_out[qh * D + i + hd2] = r2;
        }
        {
            const uint16_t* buf = k_raw + kvh * D;
            const uint16_t* bias = bk + kvh * D;
            const float x1 = h_f(f_h(h_f(buf[i]) + h_f(bias[i])));
            const float x2 = h_f(f_h(h_f(buf[i + hd2]) + h_f(bias[i + hd2])));
            const uint16_t r1 = f_h(fmaf(x1, c, -(x2 * sn))), r2 = f_h(fmaf(x2, c, x1 * sn));
            kcur[i] = r1;
            kcur[i + hd2] = r2;
            if (writer) {
                uint16_t* dst = kc + static_cast<size_t>(pos) * kvd + kvh * D;
                dst[i] = r1;
                dst[i + hd2] = r2;
                k_out[kvh * D + i] = r1;
                k_out[kvh * D + i + hd2] = r2;
            }
        }
    }
    for (int e = tid; e < D; e += nt) {
        const uint16_t r = f_h(h_f(v_raw[kvh * D + e]) + h_f(bv[kvh * D + e]));
        vcur[e] = r;
        if (writer) {
            vc[static_cast<size_t>(pos) * kvd + kvh * D + e] = r;
            v_out[kvh * D + e] = r;
        }
    }
    __syncthreads();
    for (int tk = tid; tk < seq_k; tk += nt) {
        // a key row is read in 8-byte pieces (rows start at multiples of 8 bytes: D % 4 == 0)
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        const u16x4* kv = reinterpret_cast<const u16x4*>(tk == pos ? kcur : kc + static_cast<size_t>(tk) * kvd + kvh * D);
        const u16x4* qq = reinterpret_cast<const u16x4*>(qv);
        float acc = 0.0f;
        for (int d4 = 0; d4 < D / 4; ++d4) {
            const u16x4 a = qq[d4], b = kv[d4];
            float t = h_f(a[0]) * h_f(b[0]);
            t = fmaf(h_f(a[1]), h_f(b[1]), t);
            t = fmaf(h_f(a[2]), h_f(b[2]), t);
            t = fmaf(h_f(a[3]), h_f(b[3]), t);
            acc = acc + t;
        }
        sc[tk] = f_h(acc * scale);
    }
    __syncthreads();
    // maximum (any order gives the same value)
    float m = -3.402823466e+38f;
    for (int c = tid; c < seq_k; c += nt) m = fmaxf(m, h_f(sc[c]));
    if (tid < 64) red[tid] = -3.402823466e+38f;
    __syncthreads();
    for (int s = 32; s > 0; s >>= 1) m = fmaxf(m, __shfl_down(m, s, 64));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    float maxv = red[0];
    for (int i = 1; i < (nt + 63) / 64; ++i) maxv = fmaxf(maxv, red[i]);
    for (int c = tid; c < seq_k; c += nt) {
        const float e = exp_poly(h_f(sc[c]) - maxv);
        ex[c] = e;
        sc[c] = f_h(e);
    }
    __syncthreads();
    if (tid == 0) {
        float sum = 0.0f;
        for (int c = 0; c < seq_k; ++c) sum = sum + ex[c];
        inv_s = rcp_rn(sum + 1e-20f);
    }
    __syncthreads();
    const float inv = inv_s;
    for (int c = tid; c < seq_k; c += nt) sc[c] = f_h(h_f(sc[c]) * inv);
    __syncthreads();
    for (int e = tid; e < D; e += nt) {
        // keys 0 .. pos - 1 from the cache, eight loads in flight at a time, then the current one
        const uint16_t* col = vc + kvh * D + e;
        float acc = 0.0f;
        int tk = 0;
        for (; tk + 8 <= pos; tk += 8) {
            uint16_t v[8];
            #pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = col[static_cast<size_t>(tk + u) * kvd];
            #pragma unroll
            for (int u = 0; u < 8; ++u) acc = fmaf(h_f(sc[tk + u]), h_f(v[u]), acc);
        }
        for (; tk < pos; ++tk) acc = fmaf(h_f(sc[tk]), h_f(col[static_cast<size_t>(tk) * kvd]), acc);
        acc = fmaf(h_f(sc[pos]), h_f(vcur[e]), acc);
        out[qh * D + e] = f_h(acc);
    }
}

// The same launch for head widths known at compile time (64 and 128), laid out for latency: a
// decode step at a short context is a chain of memory round trips, so everything that does not
// depend on an earlier result is requested at once.  256 threads; the first kTileRows rows of the
// group's key and value cache are requested in 16-byte pieces, in passes of 256 pieces (rows past
// the current position too: the caches hold max_pos rows, and what is not older than the current
// position is never used; the passes above it are neither waited for nor kept), and between the
// first pass and the others the projections, biases and the rotary row (which the step's first
// launch has set aside, so that its address does not wait for the position); keys and values wait
// in LDS tiles (rows padded by 16 bytes against bank conflicts) while q, k and v of the current
// position are prepared.  Scores: one thread per key from the tile; values: one thread per
// output element, keys in index order from the tile.  Longer contexts take further tiles the
// same way, each requested while the one before it is used.  The arithmetic and its order are those of
// rope_attention_kernel.
// The two serial chains the order of operations leaves (the sum of the exponentials by one lane, an
// output element's sum over the keys by one lane each) run in batches of kBatch positions: all LDS
// reads of a batch are asked for together and the dependent additions follow as they arrive, so a
// batch costs one LDS round trip and not one per position.  The last batch is filled up with
// zeros (exponentials past the last key, probabilities from the current position on, value rows
// from the current position on), which leaves a sum as it is: x + 0 = x and fma(0, 0, x) = x for
// every x but -0, and a sum that starts at +0 never becomes -0.  The current position's
// probability is kept aside (pc) and meets the current value row after the tiles, as before.
// Dynamic LDS: 6 D bytes, 6 bytes per position (positions rounded up to kBatch), 16 bytes, then two
// tiles of kTileRows x (2 D + 16) bytes.
constexpr int kTileRows = 128;
constexpr int kBatch = 32;
static_assert(kTileRows % kBatch == 0, "whole batches in a tile");
__host__ __device__ inline int padded_positions(int max_pos) { return (max_pos + kBatch - 1) / kBatch * kBatch; }
constexpr int kMaxPositions = 8192;                      // longest context a decoder is created for

template <int D>
// (Arguments in the order of need: the first 14 dwords arrive in registers with the wavefront, and the
//  first thing the kernel does is ask for the cache tiles and the position.)
__global__ __launch_bounds__(256) void rope_attention_tiled(uint16_t* __restrict__ kc, uint16_t* __restrict__ vc,
                                      const State* __restrict__ st, int n_heads, int n_kv_heads, int max_pos,
                                      float scale, const uint16_t* __restrict__ q_raw, const uint16_t* __restrict__ k_raw,
                                      const uint16_t* __restrict__ v_raw, const uint16_t* __restrict__ bq,
                                      const uint16_t* __restrict__ bk, const uint16_t* __restrict__ bv,
                                      const uint16_t* __restrict__ rope_now,
                                      uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out,
                                      uint16_t* __restrict__ v_out, uint16_t* __restrict__ out) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int kRowH = D + 8;                           // tile row stride in halves
    constexpr int kPieces = D / 8;                         // 16-byte pieces per row
    constexpr int kPasses = kTileRows * kPieces / 256;     // pieces per thread and tile
    static_assert(kTileRows * kPieces % 256 == 0, "whole passes");
    extern __shared__ __attribute__((aligned(16))) uint16_t qv[];
    uint16_t* kcur = qv + D;
    uint16_t* vcur = kcur + D;
    const int mp = padded_positions(max_pos);
    float* ex = reinterpret_cast<float*>(vcur + D);                        // [mp] exponentials, 16-byte aligned
    uint16_t* sc = reinterpret_cast<uint16_t*>(ex + mp);                   // [mp] scores, 16-byte aligned
    uint16_t* pc = sc + mp;                                                // the current position's probability
    uint16_t* ktile = pc + 8;                                              // 16-byte aligned
    uint16_t* vtile = ktile + kTileRows * kRowH;
    const int nrep = n_heads / n_kv_heads;
    const int qh = blockIdx.x, kvd = n_kv_heads * D, kvh = qh / nrep, hd2 = D / 2;
    const bool writer = qh % nrep == 0;
    const int tid = threadIdx.x;

    // piece p of this thread in a tile: row (tid + 256 p) / kPieces, 16-byte piece (tid + 256 p) % kPieces;
    // pass p of all threads is rows p kPassRows .. (p + 1) kPassRows - 1.  Passes are asked for in
    // row order, keys and values alternating, and loads return in the order of the requests: a
    // short context waits for its first passes only and leaves the rest to arrive unused.
    constexpr int kPassRows = 256 / kPieces;
    auto request = [&](const uint16_t* cache, int row0, int p) {
        const int idx = tid + 256 * p, row = idx / kPieces, piece = idx % kPieces;
        const int tk = row0 + row < max_pos ? row0 + row : max_pos - 1;
        return *reinterpret_cast<const u32x4*>(cache + static_cast<size_t>(tk) * kvd + kvh * D + 8 * piece);
    };
    u32x4 kreg[kPasses], vreg[kPasses];
    auto request_tiles = [&](int row0, int first_pass) {
        #pragma unroll
        for (int p = first_pass; p < kPasses; ++p) {
            kreg[p] = request(kc, row0, p);
            vreg[p] = request(vc, row0, p);
            asm volatile("" ::: "memory");                 // in this order: the compiler would sort them by cache
        }
    };
    // the passes that hold rows below `rows` (of kBatch; the value sums run in whole batches) go to
    // LDS; value rows from row `valid` of the tile on are stored as zeros
    auto keep = [&](uint16_t* tile, const u32x4 (&r)[kPasses], int rows, int valid) {
        #pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            if (p * kPassRows < rows) {
                const int idx = tid + 256 * p, row = idx / kPieces, piece = idx % kPieces;
                const u32x4 zero = {0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4*>(tile + row * kRowH + 8 * piece) = row < valid ? r[p] : zero;
            }
        }
    };
    // rows of the tile at row0 that anybody reads: the keys below the current position, in whole batches
    auto tile_rows = [&](int row0, int pos) {
        const int n = pos - row0 < kTileRows ? pos - row0 : kTileRows;
        return (n + kBatch - 1) / kBatch * kBatch;
    };
    // The tiles' first passes are asked for first: their addresses need nothing but the arguments that
    // arrive in registers.  What the current position needs (projections, biases, the rotary row: a few
    // bytes per thread, behind pointers that have to be fetched) is asked for next, ahead of the other
    // passes, and arrives ahead of them, so that q, k and v are prepared while the tiles come in.  Wavefront 0 prepares q, 1 k, 2 and 3 v; every thread loads from a valid
    // address whether it has an element or not, so the number of loads in flight is the same for all.
    int pos = st->pos;
    kreg[0] = request(kc, 0, 0);
    vreg[0] = request(vc, 0, 0);
    asm volatile("" ::: "memory");
    const int role = tid >> 6, lane = tid & 63;
    const int i = role < 2 ? (lane < hd2 ? lane : hd2 - 1) : (tid - 128 < D ? tid - 128 : D - 1);
    const int i2 = role < 2 ? i + hd2 : i;
    const uint16_t* buf = role == 0 ? q_raw + qh * D : role == 1 ? k_raw + kvh * D : v_raw + kvh * D;
    const uint16_t* bias = role == 0 ? bq + qh * D : role == 1 ? bk + kvh * D : bv + kvh * D;
    const uint16_t raw1 = buf[i], raw2 = buf[i2], bias1 = bias[i], bias2 = bias[i2];
    const uint16_t cos_i = rope_now[role < 2 ? i : 0], sin_i = rope_now[D + (role < 2 ? i : 0)];   // embed_kernel's row
    asm volatile("" ::: "memory");                             // these first
    request_tiles(0, 1);
    __builtin_amdgcn_sched_barrier(0);                         // and nothing that waits for one of them in between

    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    const int seq_k = pos + 1;
    // (computed by every thread, stored by those that have an element: a load that is only used under a
    //  condition would be moved there, behind the tiles)
    const float c = h_f(cos_i), sn = h_f(sin_i);
    const float x1 = h_f(f_h(h_f(raw1) + h_f(bias1)));
    const float x2 = h_f(f_h(h_f(raw2) + h_f(bias2)));
    const uint16_t r1 = f_h(fmaf(x1, c, -(x2 * sn))), r2 = f_h(fmaf(x2, c, x1 * sn));
    const bool has_pair = role < 2 && lane < hd2, has_v = role >= 2 && tid - 128 < D;
    const uint16_t rv = f_h(x1);                               // fp16(v + bias), rounded once
    if (has_pair) {
        uint16_t* dst = role == 0 ? qv : kcur;
        dst[i] = r1;
        dst[i + hd2] = r2;
    } else if (has_v) {
        vcur[tid - 128] = rv;
    }
    keep(ktile, kreg, tile_rows(0, pos), kTileRows);
    keep(vtile, vreg, tile_rows(0, pos), pos);
    // (the stores to memory after the tiles are in LDS: a store in flight counts like a load that has not
    //  arrived, and would make the waits above wait for later passes than they need)
    if (has_pair) {
        if (role == 0) {
            q_out[qh * D + i] = r1;
            q_out[qh * D + i + hd2] = r2;
        } else if (writer) {
            uint16_t* dst = kc + static_cast<size_t>(pos) * kvd + kvh * D;
            dst[i] = r1;
            dst[i + hd2] = r2;
            k_out[kvh * D + i] = r1;
            k_out[kvh * D + i + hd2] = r2;
        }
    } else if (has_v && writer) {
        const int e = tid - 128;
        vc[static_cast<size_t>(pos) * kvd + kvh * D + e] = rv;
        v_out[kvh * D + e] = rv;
    }
    if (pos > kTileRows) request_tiles(kTileRows, 0);          // the second tiles, one tile ahead of their use
    __syncthreads();

    // scores: tile rows by threads 0 .. kTileRows - 1, the current position by thread kTileRows
    auto score = [&](const uint16_t* krow) {
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        const u16x4* kv = reinterpret_cast<const u16x4*>(krow);
        const u16x4* qq = reinterpret_cast<const u16x4*>(qv);
        float acc = 0.0f;
        #pragma unroll
        for (int d4 = 0; d4 < D / 4; ++d4) {
            const u16x4 a = qq[d4], b = kv[d4];
            float t = h_f(a[0]) * h_f(b[0]);
            t = fmaf(h_f(a[1]), h_f(b[1]), t);
            t = fmaf(h_f(a[2]), h_f(b[2]), t);
            t = fmaf(h_f(a[3]), h_f(b[3]), t);
            acc = acc + t;
        }
        return f_h(acc * scale);
    };
    if (tid == kTileRows) sc[pos] = score(kcur);
    for (int row0 = 0; row0 < pos; row0 += kTileRows) {
        if (row0 > 0) {
            __syncthreads();                               // the previous tile's scores are done
            keep(ktile, kreg, tile_rows(row0, pos), kTileRows);
            if (row0 + kTileRows < pos) {
                #pragma unroll
                for (int p = 0; p < kPasses; ++p) kreg[p] = request(kc, row0 + kTileRows, p);
            }
            __syncthreads();
        }
        if (tid < kTileRows && row0 + tid < pos) sc[row0 + tid] = score(ktile + tid * kRowH);
    }
    __syncthreads();
    // softmax by the first wavefront alone: its LDS accesses are ordered, so the steps need no
    // barrier between them (a short context is all barrier otherwise)
    if (tid < 64) {
        float m = -3.402823466e+38f;                       // maximum: any order gives the same value
        for (int c = tid; c < seq_k; c += 64) m = fmaxf(m, h_f(sc[c]));
        const float maxv = wave_max(m);
        for (int c = tid; c < seq_k; c += 64) {
            const float e = exp_poly(h_f(sc[c]) - maxv);
            ex[c] = e;
            sc[c] = f_h(e);
        }
        const int padded = (seq_k + kBatch - 1) / kBatch * kBatch;
        if (tid < padded - seq_k) ex[seq_k + tid] = 0.0f;      // kBatch <= 64 lanes
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");  // lane 0 reads what the other lanes wrote
        __builtin_amdgcn_wave_barrier();
        float inv = 0.0f;
        if (tid == 0) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4* e4 = reinterpret_cast<const f32x4*>(ex);
            float sum = 0.0f;
            for (int c = 0; c < padded; c += kBatch) {
                f32x4 t[kBatch / 4];
                #pragma unroll
                for (int j = 0; j < kBatch / 4; ++j) t[j] = e4[c / 4 + j];
                #pragma unroll
                for (int j = 0; j < kBatch / 4; ++j) {
                    sum = sum + t[j][0];
                    sum = sum + t[j][1];
                    sum = sum + t[j][2];
                    sum = sum + t[j][3];
                }
            }
            inv = rcp_rn(sum + 1e-20f);
        }
        inv = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(inv)));
        // probabilities of the older keys; zeros from the current position to the end of its batch
        for (int c = tid; c < padded; c += 64) {
            const uint16_t pr = f_h(h_f(sc[c]) * inv);
            if (c == pos) pc[0] = pr;
            sc[c] = c < pos ? pr : static_cast<uint16_t>(0);
        }
    }
    __syncthreads();
    // output element e by thread e: older keys in index order from the tiles, then the current one
    float acc = 0.0f;
    for (int row0 = 0; row0 < pos; row0 += kTileRows) {
        if (row0 > 0) {
            __syncthreads();                               // the previous tile has been used up
            keep(vtile, vreg, tile_rows(row0, pos), pos - row0);
            if (row0 + kTileRows < pos) {
                #pragma unroll
                for (int p = 0; p < kPasses; ++p) vreg[p] = request(vc, row0 + kTileRows, p);
            }
            __syncthreads();
        }
        if (tid < D) {
            typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
            const int n = pos - row0 < kTileRows ? pos - row0 : kTileRows;
            for (int r0 = 0; r0 < n; r0 += kBatch) {
                u16x8 p[kBatch / 8];
                uint16_t v[kBatch];
                #pragma unroll
                for (int j = 0; j < kBatch / 8; ++j) p[j] = *reinterpret_cast<const u16x8*>(sc + row0 + r0 + 8 * j);
                #pragma unroll
                for (int u = 0; u < kBatch; ++u) v[u] = vtile[(r0 + u) * kRowH + tid];
                #pragma unroll
                for (int u = 0; u < kBatch; ++u) acc = fmaf(h_f(p[u / 8][u % 8]), h_f(v[u]), acc);
            }
        }
    }
    if (tid < D) {
        acc = fmaf(h_f(pc[0]), h_f(vcur[tid]), acc);
        out[qh * D + tid] = f_h(acc);
    }
}

// ---- attention with the keys of a head split over several blocks (an arithmetic mode, not the default) ----
//
// The launch above keeps the reference's order of operations, and at a long context that order is two
// chains of dependent additions as long as the context, in one wavefront per head.  Here block (head, s) takes
// run s of `splits` consecutive runs of the keys: scores as above (fp32 dot product, rounded to fp16 like
// the reference's), its own maximum m, e = exp(score - m) in fp32, their sum l and o[d] = sum e v[d]; a
// second launch merges the parts of a head: M = max m, out = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s.
// The same real numbers as softmax(q k) v, summed in another order and without the fp16 roundings of the
// probabilities: within the stated tolerance of the reference-order launch, not bit-identical.
// part: [n_heads][splits][D + 2] floats: m, l, o[D].
constexpr int kSplitThreads = 256;
constexpr int kMaxSplits = 32;

template <int D>
__global__ __launch_bounds__(kSplitThreads) void attention_split_kernel(
        uint16_t* __restrict__ kc, uint16_t* __restrict__ vc, const State* __restrict__ st, int n_heads, int n_kv_heads,
        int max_pos, float scale, const uint16_t* __restrict__ q_raw, const uint16_t* __restrict__ k_raw,
        const uint16_t* __restrict__ v_raw, const uint16_t* __restrict__ bq, const uint16_t* __restrict__ bk,
        const uint16_t* __restrict__ bv, const uint16_t* __restrict__ rope_now, uint16_t* __restrict__ q_out,
        uint16_t* __restrict__ k_out, uint16_t* __restrict__ v_out, float* __restrict__ part, int chunk_cap) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float* sc = sm;                                            // [chunk_cap] scores, then exponentials
    float* red = sc + chunk_cap;                               // [8] block reductions
    float* osum = red + 8;                                     // [kSplitThreads / D][D] partial outputs
    uint16_t* qv = reinterpret_cast<uint16_t*>(osum + kSplitThreads);   // [D] q, [D] k, [D] v of the current position
    uint16_t* kcur = qv + D;
    uint16_t* vcur = kcur + D;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qh = blockIdx.x, sp = blockIdx.y, splits = gridDim.y;
    const int nrep = n_heads / n_kv_heads, kvh = qh / nrep, kvd = n_kv_heads * D, hd2 = D / 2;
    int pos = st->pos;
    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    const int seq_k = pos + 1;
    const int chunk = (seq_k + splits - 1) / splits;           // <= chunk_cap: the host sizes it for max_pos
    const int k0 = sp * chunk, k1 = k0 + chunk < seq_k ? k0 + chunk : seq_k;
    float* mine = part + (static_cast<size_t>(qh) * splits + sp) * (D + 2);
    if (k0 >= k1) {                                            // no keys for this block at this position
        if (tid == 0) { mine[0] = -3.402823466e+38f; mine[1] = 0.0f; }
        if (tid < D) mine[2 + tid] = 0.0f;
        return;
    }
    const bool has_current = k1 == seq_k;                      // the block whose run ends with the current position
    // Everything the block reads from memory is asked for now, behind the position alone: the row of the
    // thread's first key, the first kAhead values of the thread's output element, and (below) the current
    // position's q, k and v; the arithmetic then waits for one round trip, not for four in a row.
    constexpr int kGroups = kSplitThreads / D, kAhead = 32;
    const int d = tid % D, grp = tid / D;
    const int c_first = k0 + tid;
    u32x4 kr_first[D / 8];
    // (a thread without such a key reads row 0 instead and does not use it: loads under a condition of
    //  their own were measured slower, 548 -> 576 us per step at position 2000)
    {
        const bool from_cache = c_first < k1 && c_first != pos;
        const u32x4* row = reinterpret_cast<const u32x4*>(kc + static_cast<size_t>(from_cache ? c_first : 0) * kvd + kvh * D);
        #pragma unroll
        for (int i = 0; i < D / 8; ++i) kr_first[i] = row[i];
    }
    uint16_t v_first[kAhead];
    #pragma unroll
    for (int i = 0; i < kAhead; ++i) {
        const int c = k0 + grp + i * kGroups;
        v_first[i] = vc[static_cast<size_t>(c < k1 && c != pos ? c : 0) * kvd + kvh * D + d];
    }
    // q of the head (every block), k and v of the current position (the block that needs them); the block of
    // the group's first head also writes them to the caches and to the buffers a caller may inspect
    if (tid < hd2) {
        const float c = h_f(rope_now[tid]), sn = h_f(rope_now[D + tid]);
        const float x1 = h_f(f_h(h_f(q_raw[qh * D + tid]) + h_f(bq[qh * D + tid])));
        const float x2 = h_f(f_h(h_f(q_raw[qh * D + tid + hd2]) + h_f(bq[qh * D + tid + hd2])));
        const uint16_t r1 = f_h(fmaf(x1, c, -(x2 * sn))), r2 = f_h(fmaf(x2, c, x1 * sn));
        qv[tid] = r1;
        qv[tid + hd2] = r2;
        if (sp == 0) { q_out[qh * D + tid] = r1; q_out[qh * D + tid + hd2] = r2; }
    } else if (has_current && tid >= 64 && tid < 64 + hd2) {
        const int i = tid - 64;
        const float c = h_f(rope_now[i]), sn = h_f(rope_now[D + i]);
        const float x1 = h_f(f_h(h_f(k_raw[kvh * D + i]) + h_f(bk[kvh * D + i])));
        const float x2 = h_f(f_h(h_f(k_raw[kvh * D + i + hd2]) + h_f(bk[kvh * D + i + hd2])));
        const uint16_t r1 = f_h(fmaf(x1, c, -(x2 * sn))), r2 = f_h(fmaf(x2, c, x1 * sn));
        kcur[i] = r1;
        kcur[i + hd2] = r2;
        if (qh % nrep == 0) {
            uint16_t* dst = kc + static_cast<size_t>(pos) * kvd + kvh * D;
            dst[i] = r1; dst[i + hd2] = r2;
            k_out[kvh * D + i] = r1; k_out[kvh * D + i + hd2] = r2;
        }
    } else if (has_current && tid >= 128 && tid < 128 + D) {
        const int e = tid - 128;
        const uint16_t r = f_h(h_f(v_raw[kvh * D + e]) + h_f(bv[kvh * D + e]));
        vcur[e] = r;
        if (qh % nrep == 0) {
            vc[static_cast<size_t>(pos) * kvd + kvh * D + e] = r;
            v_out[kvh * D + e] = r;
        }
    }
    __syncthreads();
    // scores, a thread per key: the key's row straight from the cache (the current position's from LDS)
    float m = -3.402823466e+38f;
    for (int c = c_first; c < k1; c += kSplitThreads) {
        u32x4 kr[D / 8];
        if (c == pos) {
            #pragma unroll
            for (int i = 0; i < D / 8; ++i) kr[i] = reinterpret_cast<const u32x4*>(kcur)[i];
        } else if (c == c_first) {
            #pragma unroll
            for (int i = 0; i < D / 8; ++i) kr[i] = kr_first[i];
        } else {
            const u32x4* row = reinterpret_cast<const u32x4*>(kc + static_cast<size_t>(c) * kvd + kvh * D);
            #pragma unroll
            for (int i = 0; i < D / 8; ++i) kr[i] = row[i];
        }
        float acc = 0.0f;
        #pragma unroll
        for (int i = 0; i < D / 8; ++i) {
            const u32x4 qq = reinterpret_cast<const u32x4*>(qv)[i];
            const uint32_t qd[4] = {qq.x, qq.y, qq.z, qq.w}, kd[4] = {kr[i].x, kr[i].y, kr[i].z, kr[i].w};
            #pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = fmaf(h_f(static_cast<uint16_t>(qd[j] & 0xffffu)), h_f(static_cast<uint16_t>(kd[j] & 0xffffu)), acc);
                acc = fmaf(h_f(static_cast<uint16_t>(qd[j] >> 16)), h_f(static_cast<uint16_t>(kd[j] >> 16)), acc);
            }
        }
        const float sco = h_f(f_h(acc * scale));
        sc[c - k0] = sco;
        m = fmaxf(m, sco);
    }
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float l = 0.0f;
    for (int c = k0 + tid; c < k1; c += kSplitThreads) {
        const float e = exp_poly(sc[c - k0] - m);
        sc[c - k0] = e;
        l += e;
    }
    for (int sft = 32; sft > 0; sft >>= 1) l += __shfl_xor(l, sft, 64);
    if (lane == 0) red[4 + wave] = l;
    __syncthreads();                                           // exponentials and the waves' sums are in LDS
    // o[d]: kSplitThreads / D groups of D threads, group g takes the keys k0 + g, k0 + g + groups, ...
    float o = 0.0f;
    #pragma unroll
    for (int i = 0; i < kAhead; ++i) {
        const int c = k0 + grp + i * kGroups;
        if (c < k1) o = fmaf(sc[c - k0], h_f(c == pos ? vcur[d] : v_first[i]), o);
    }
    #pragma unroll 8
    for (int c = k0 + grp + kAhead * kGroups; c < k1; c += kGroups) {
        const uint16_t v = c == pos ? vcur[d] : vc[static_cast<size_t>(c) * kvd + kvh * D + d];
        o = fmaf(sc[c - k0], h_f(v), o);
    }
    osum[grp * D + d] = o;
    __syncthreads();
    if (tid < D) {
        float t = osum[tid];
        #pragma unroll
        for (int g2 = 1; g2 < kGroups; ++g2) t += osum[g2 * D + tid];
        mine[2 + tid] = t;
    }
    if (tid == 0) {
        mine[0] = m;
        mine[1] = (red[4] + red[5]) + (red[6] + red[7]);
    }
}

// The parts of a head into its attention output (see attention_split_kernel).  Every load of the launch is
// asked for before the first is used: thread s takes the maximum and the sum of part s, thread d element d
// of every part.
template <int D>
__global__ __launch_bounds__(D) void attention_merge_kernel(const float* __restrict__ part, int splits,
                                                            uint16_t* __restrict__ out) {
    __shared__ float w[kMaxSplits];
    __shared__ float Ls;
    const int qh = blockIdx.x, d = threadIdx.x;
    const float* p = part + static_cast<size_t>(qh) * splits * (D + 2);
    float o_s[kMaxSplits];
    #pragma unroll
    for (int s = 0; s < kMaxSplits; ++s) o_s[s] = s < splits ? p[s * (D + 2) + 2 + d] : 0.0f;
    if (d < 64) {                                              // the first wavefront: splits <= 32 lanes of it
        const bool has = d < splits;
        const float ms = has ? p[d * (D + 2)] : -3.402823466e+38f;
        const float ls = has ? p[d * (D + 2) + 1] : 0.0f;
        const float M = wave_max(ms);
        const float ws = ls > 0.0f ? exp_poly(ms - M) : 0.0f;
        float L = ls * ws;
        for (int sft = 32; sft > 0; sft >>= 1) L += __shfl_xor(L, sft, 64);
        if (d < kMaxSplits) w[d] = ws;
        if (d == 0) Ls = L;
    }
    __syncthreads();
    float o = 0.0f;
    #pragma unroll
    for (int s = 0; s < kMaxSplits; ++s) o = fmaf(o_s[s], w[s], o);
    out[qh * D + d] = f_h(o * rcp_rn(Ls + 1e-20f));
}

inline size_t split_attention_lds(int D, int chunk_cap) {
    return static_cast<size_t>(chunk_cap + 8 + kSplitThreads) * 4 + 3 * static_cast<size_t>(D) * 2;
}

// gate[i] = fp16((g * sigmoid(g)) * up[i])   (QW/kernels/mlp.cl swiglu_inplace)
__global__ void swiglu_kernel(uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const float g = h_f(gate[i]), u = h_f(up[i]);
        const float sig = rcp_rn(1.0f + exp_poly(-g));
        gate[i] = f_h((g * sig) * u);
    }
}


// ---- a prompt of M tokens at once (Model::forward with seq_len = M, QW/src/model.cpp:243-376) ----
// Row r of every buffer belongs to position pos0 + r.  The kernels below repeat, row by row, the
// operations of the single-token kernels above in the same order, so that a prompt gives the
// same cache rows and logits as M single-token steps wherever the projections do (they do bit
// for bit when the M > 1 projections run as rows of GEMV, and within the GEMM's tolerance when
// they run on the matrix cores).

// H[r][c] = embed[tokens[r]][c]   (QW/kernels/embedding.cl)
__global__ void embed_rows_kernel(const uint16_t* __restrict__ embed, const int* __restrict__ tokens,
                                  uint16_t* __restrict__ H, int hidden, int vocab) {
    int t = tokens[blockIdx.x];
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);
    const uint16_t* src = embed + static_cast<size_t>(t) * hidden;
    uint16_t* dst = H + static_cast<size_t>(blockIdx.x) * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = src[c];
}

// One block per row: q/k/v bias, rotary embedding of q and k at position pos0 + row, k and v into
// the cache rows of that position (QW/kernels/bias_add.cl, rope.cl; rows as QW/src/layers/
// attention.cpp:560-600).
__global__ __launch_bounds__(256) void rope_rows_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ Kp,
                                                        const uint16_t* __restrict__ V, const uint16_t* __restrict__ bq,
                                                        const uint16_t* __restrict__ bk, const uint16_t* __restrict__ bv,
                                                        const uint16_t* __restrict__ cosT, const uint16_t* __restrict__ sinT,
                                                        uint16_t* __restrict__ kc, uint16_t* __restrict__ vc,
                                                        uint16_t* __restrict__ QR, int pos0, int n_heads, int n_kv_heads, int D,
                                                        int ldq, int ldkv) {
    // ldq, ldkv: halves between rows of Q and of Kp / V (the widths of the projections, or of the
    // stacked q|k|v projection they are columns of)
    const int row = blockIdx.x, pos = pos0 + row, hd2 = D / 2, qd = n_heads * D, kvd = n_kv_heads * D;
    const uint16_t* cr = cosT + static_cast<size_t>(pos) * D;
    const uint16_t* sr = sinT + static_cast<size_t>(pos) * D;
    for (int j = threadIdx.x; j < (n_heads + n_kv_heads) * hd2; j += blockDim.x) {
        const int head = j / hd2, i = j - head * hd2;
        const bool isq = head < n_heads;
        const int hh = isq ? head : head - n_heads;
        const uint16_t* buf = isq ? Q + static_cast<size_t>(row) * ldq + hh * D : Kp + static_cast<size_t>(row) * ldkv + hh * D;
        const uint16_t* bias = (isq ? bq : bk) + hh * D;
        uint16_t* dst = isq ? QR + static_cast<size_t>(row) * qd + hh * D : kc + static_cast<size_t>(pos) * kvd + hh * D;
        const float c = h_f(cr[i]), sn = h_f(sr[i]);
        const float x1 = h_f(f_h(h_f(buf[i]) + h_f(bias[i])));
        const float x2 = h_f(f_h(h_f(buf[i + hd2]) + h_f(bias[i + hd2])));
        dst[i] = f_h(fmaf(x1, c, -(x2 * sn)));
        dst[i + hd2] = f_h(fmaf(x2, c, x1 * sn));
    }
    for (int e = threadIdx.x; e < kvd; e += blockDim.x)
        vc[static_cast<size_t>(pos) * kvd + e] = f_h(h_f(V[static_cast<size_t>(row) * ldkv + e]) + h_f(bv[e]));
}

// One block per (query head, row): the query of position pos0 + row against cache rows
// 0 .. pos0 + row (causal), QW/kernels/attention.cl gqa_attn_scores, gqa_softmax, gqa_attn_out with
// the sums in the order of rope_attention_kernel.  256 threads.  Dynamic LDS: 2 D (1 + kPromptTile)
// bytes + 6 bytes per position.
constexpr int kPromptTile = 64;
__global__ __launch_bounds__(256) void attention_rows_kernel(const uint16_t* __restrict__ QR, const uint16_t* __restrict__ kc,
                                                             const uint16_t* __restrict__ vc, uint16_t* __restrict__ out,
                                                             int pos0, int seq_cap, int n_heads, int n_kv_heads, int D,
                                                             float scale) {
    extern __shared__ __attribute__((aligned(16))) uint16_t qv[];
    uint16_t* tile = qv + D;                                       // [kPromptTile][D] values
    float* ex = reinterpret_cast<float*>(tile + kPromptTile * D);
    uint16_t* sc = reinterpret_cast<uint16_t*>(ex + seq_cap);
    __shared__ float red[64];
    __shared__ float inv_s;
    const int qh = blockIdx.x, row = blockIdx.y, pos = pos0 + row, seq_k = pos + 1;
    const int nrep = n_heads / n_kv_heads, kvh = qh / nrep, kvd = n_kv_heads * D, qd = n_heads * D;
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int i = tid; i < D; i += nt) qv[i] = QR[static_cast<size_t>(row) * qd + qh * D + i];
    __syncthreads();
    for (int tk = tid; tk < seq_k; tk += nt) {
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        const u16x4* kv = reinterpret_cast<const u16x4*>(kc + static_cast<size_t>(tk) * kvd + kvh * D);
        const u16x4* qq = reinterpret_cast<const u16x4*>(qv);
        float acc = 0.0f;
        for (int d4 = 0; d4 < D / 4; ++d4) {
            const u16x4 a = qq[d4], b = kv[d4];
            float t = h_f(a[0]) * h_f(b[0]);
            t = fmaf(h_f(a[1]), h_f(b[1]), t);
            t = fmaf(h_f(a[2]), h_f(b[2]), t);
            t = fmaf(h_f(a[3]), h_f(b[3]), t);
            acc = acc + t;
        }
        sc[tk] = f_h(acc * scale);
    }
    __syncthreads();
    float m = -3.402823466e+38f;
    for (int c = tid; c < seq_k; c += nt) m = fmaxf(m, h_f(sc[c]));
    if (tid < 64) red[tid] = -3.402823466e+38f;
    __syncthreads();
    for (int s = 32; s > 0; s >>= 1) m = fmaxf(m, __shfl_down(m, s, 64));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    float maxv = red[0];
    for (int i = 1; i < (nt + 63) / 64; ++i) maxv = fmaxf(maxv, red[i]);
    for (int c = tid; c < seq_k; c += nt) {
        const float e = exp_poly(h_f(sc[c]) - maxv);
        ex[c] = e;
        sc[c] = f_h(e);
    }
    __syncthreads();
    if (tid == 0) {
        float sum = 0.0f;
        for (int c = 0; c < seq_k; ++c) sum = sum + ex[c];
        inv_s = rcp_rn(sum + 1e-20f);
    }
    __syncthreads();
    const float inv = inv_s;
    for (int c = tid; c < seq_k; c += nt) sc[c] = f_h(h_f(sc[c]) * inv);
    __syncthreads();
    // values: tiles of kPromptTile cache rows go through LDS (all threads fetch, 8 bytes each), then
    // thread e < D runs its sum over the tile's keys in index order
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    u16x4* tile4 = reinterpret_cast<u16x4*>(tile);
    const int d4n = D / 4;
    float acc = 0.0f;                                   // of output element tid (D <= 256 = threads)
    for (int t0 = 0; t0 < seq_k; t0 += kPromptTile) {
        const int rows = seq_k - t0 < kPromptTile ? seq_k - t0 : kPromptTile;
        for (int i = tid; i < rows * d4n; i += nt) {
            const int r = i / d4n, p = i - r * d4n;
            tile4[i] = *reinterpret_cast<const u16x4*>(vc + static_cast<size_t>(t0 + r) * kvd + kvh * D + 4 * p);
        }
        __syncthreads();
        if (tid < D)
            for (int r = 0; r < rows; ++r) acc = fmaf(h_f(sc[t0 + r]), h_f(tile[r * D + tid]), acc);
        __syncthreads();
    }
    if (tid < D) out[static_cast<size_t>(row) * qd + qh * D + tid] = f_h(acc);
}

// The same for head widths 64 and 128 with at most 8 query heads per key/value head: one block per
// (key/value head, row) serves all query heads of the group, so that a cache row is fetched once
// per group and position instead of once per head, and every fetch is a coalesced copy of a tile
// of kPromptTile rows into LDS (a thread of attention_rows_kernel walks a cache row of its own,
// which the memory pipeline serves one line per thread).  Per query the operations and their
// order are those of attention_rows_kernel: a score per thread from the key tile (rows padded by
// 8 bytes against bank conflicts), maximum, exponentials, the denominator summed by one thread
// in key order, the output element's sum in key order from the value tiles.  A (query, key)
// pair owns 4 bytes of LDS that hold, in turn, its fp16 score, its fp32 exponential and its fp16
// probability.  Wavefront w serves queries w and w + 4 in every phase but the last, where a thread
// owns one output element of up to 8 D / 256 queries.
// Dynamic LDS: 2 kPromptTile (D + 4) + 4 nrep seq_cap bytes; seq_cap is a multiple of 4.
template <int D>
__global__ __launch_bounds__(256) void attention_group_kernel(const uint16_t* __restrict__ QR, const uint16_t* __restrict__ kc,
                                                              const uint16_t* __restrict__ vc, uint16_t* __restrict__ out,
                                                              int pos0, int seq_cap, int n_heads, int n_kv_heads, float scale) {
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    constexpr int TK = kPromptTile, KS = D + 4, D4 = D / 4;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    uint16_t* tile = smem;                                          // [TK][KS] keys, then [TK][D] values
    uint32_t* slot = reinterpret_cast<uint32_t*>(tile + TK * KS);   // [nrep][seq_cap]
    __shared__ float inv_s[8];
    const int g = blockIdx.x, row = blockIdx.y, pos = pos0 + row, seq_k = pos + 1;
    const int nrep = n_heads / n_kv_heads, kvd = n_kv_heads * D, qd = n_heads * D;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const uint16_t* qsrc = QR + static_cast<size_t>(row) * qd + static_cast<size_t>(g) * nrep * D;   // the group's heads are adjacent
    const bool has0 = w < nrep, has1 = w + 4 < nrep;
    const int q0i = has0 ? w : 0, q1i = has1 ? w + 4 : q0i;
    // the wavefront's two query rows live in registers for the whole scores phase
    u16x4 qa[D4], qb[D4];
    #pragma unroll
    for (int d4 = 0; d4 < D4; ++d4) {
        qa[d4] = *reinterpret_cast<const u16x4*>(qsrc + q0i * D + 4 * d4);
        qb[d4] = *reinterpret_cast<const u16x4*>(qsrc + q1i * D + 4 * d4);
    }

    // A tile's rows travel global memory -> registers -> LDS; the next tile's are requested before
    // the current tile is worked on, so that their latency runs under the arithmetic.
    constexpr int kPieces = TK * D4 / 256;                          // 8-byte pieces of a tile per thread
    u16x4 pre[kPieces];
    auto fetch = [&](const uint16_t* cache, int t0) {
        #pragma unroll
        for (int u = 0; u < kPieces; ++u) {
            const int i = tid + 256 * u, r = i / D4, p = i - r * D4;
            const int tk = t0 + r < seq_k ? t0 + r : seq_k - 1;     // rows past the last key: a copy of it, never used
            pre[u] = *reinterpret_cast<const u16x4*>(cache + static_cast<size_t>(tk) * kvd + g * D + 4 * p);
        }
    };
    auto stash = [&](int stride) {
        #pragma unroll
        for (int u = 0; u < kPieces; ++u) {
            const int i = tid + 256 * u, r = i / D4, p = i - r * D4;
            *reinterpret_cast<u16x4*>(tile + r * stride + 4 * p) = pre[u];
        }
    };

    // scores: thread (key = lane, wavefront w) of a tile takes queries w and w + 4
    fetch(kc, 0);
    for (int t0 = 0; t0 < seq_k; t0 += TK) {
        const int rows = seq_k - t0 < TK ? seq_k - t0 : TK;
        __syncthreads();                                             // the last tile has been used
        stash(KS);
        __syncthreads();
        if (t0 + TK < seq_k) fetch(kc, t0 + TK);
        if (lane < rows) {
            const u16x4* kr = reinterpret_cast<const u16x4*>(tile + lane * KS);
            float acc0 = 0.0f, acc1 = 0.0f;
            #pragma unroll
            for (int d4 = 0; d4 < D4; ++d4) {
                const u16x4 b = kr[d4], a0 = qa[d4], a1 = qb[d4];
                float t = h_f(a0[0]) * h_f(b[0]);
                t = fmaf(h_f(a0[1]), h_f(b[1]), t);
                t = fmaf(h_f(a0[2]), h_f(b[2]), t);
                t = fmaf(h_f(a0[3]), h_f(b[3]), t);
                acc0 = acc0 + t;
                float u = h_f(a1[0]) * h_f(b[0]);
                u = fmaf(h_f(a1[1]), h_f(b[1]), u);
                u = fmaf(h_f(a1[2]), h_f(b[2]), u);
                u = fmaf(h_f(a1[3]), h_f(b[3]), u);
                acc1 = acc1 + u;
            }
            if (has0) slot[q0i * seq_cap + t0 + lane] = f_h(acc0 * scale);
            if (has1) slot[q1i * seq_cap + t0 + lane] = f_h(acc1 * scale);
        }
    }
    fetch(vc, 0);                                                    // the first tile of values arrives under the softmax
    __syncthreads();
    // maximum and exponentials, a wavefront per query.  A lane takes four of its entries at a time
    // (all reads ahead of the arithmetic and the writes: one LDS round trip per four entries).
    auto each4 = [&](uint32_t* sl, auto&& f) {
        for (int c0 = lane; c0 < seq_k; c0 += 256) {
            uint32_t v[4];
            #pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = sl[c0 + 64 * u < seq_k ? c0 + 64 * u : c0];
            #pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = f(v[u]);
            #pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c0 + 64 * u < seq_k) sl[c0 + 64 * u] = v[u];
        }
    };
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (j ? has1 : has0) {
            uint32_t* sl = slot + (j ? q1i : q0i) * seq_cap;
            float m = -3.402823466e+38f;
            for (int c0 = lane; c0 < seq_k; c0 += 256) {
                uint32_t v[4];
                #pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = sl[c0 + 64 * u < seq_k ? c0 + 64 * u : c0];
                #pragma unroll
                for (int u = 0; u < 4; ++u) m = fmaxf(m, h_f(static_cast<uint16_t>(v[u])));
            }
            for (int s = 32; s > 0; s >>= 1) m = fmaxf(m, __shfl_xor(m, s, 64));
            each4(sl, [m](uint32_t v) { return __float_as_uint(exp_poly(h_f(static_cast<uint16_t>(v)) - m)); });
        }
    }
    __syncthreads();
    // denominators: lanes 0 and 1 of a wavefront, one query each, keys in index order (sixteen
    // entries are read ahead of their additions; rows of slot start at multiples of 16 bytes)
    {
        const int qi = w + 4 * lane;
        if (lane < 2 && qi < nrep) {
            const uint32_t* sl = slot + qi * seq_cap;
            float sum = 0.0f;
            int c = 0;
            for (; c + 16 <= seq_k; c += 16) {
                uint4 v[4];
                #pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const uint4*>(sl + c + 4 * u);
                #pragma unroll
                for (int u = 0; u < 4; ++u) {
                    sum = sum + __uint_as_float(v[u].x);
                    sum = sum + __uint_as_float(v[u].y);
                    sum = sum + __uint_as_float(v[u].z);
                    sum = sum + __uint_as_float(v[u].w);
                }
            }
            for (; c < seq_k; ++c) sum = sum + __uint_as_float(sl[c]);
            inv_s[qi] = rcp_rn(sum + 1e-20f);
        }
    }
    __syncthreads();
    // probabilities: fp16(fp16(e) * inv), as the separate kernels store them
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (j ? has1 : has0) {
            const int qi = j ? q1i : q0i;
            const float inv = inv_s[qi];
            each4(slot + qi * seq_cap, [inv](uint32_t v) -> uint32_t { return f_h(h_f(f_h(__uint_as_float(v))) * inv); });
        }
    }
    // values: thread (e = tid % D, tid / D) owns element e of queries tid / D + j (256 / D)
    constexpr int kStep = 256 / D, kJ = 8 / kStep;
    const int e = tid % D, qfirst = tid / D;
    int qc[kJ];
    float acc[kJ];
    #pragma unroll
    for (int j = 0; j < kJ; ++j) {
        const int qi = qfirst + j * kStep;
        qc[j] = (qi < nrep ? qi : nrep - 1) * seq_cap;
        acc[j] = 0.0f;
    }
    for (int t0 = 0; t0 < seq_k; t0 += TK) {
        const int rows = seq_k - t0 < TK ? seq_k - t0 : TK;
        __syncthreads();                                             // probabilities are in place; the last tile has been used
        stash(D);
        __syncthreads();
        if (t0 + TK < seq_k) fetch(vc, t0 + TK);
        int r = 0;
        for (; r + 8 <= rows; r += 8) {                              // eight keys read ahead of their sums
            uint16_t v[8];
            uint4 pr[kJ][2];
            #pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = tile[(r + u) * D + e];
            #pragma unroll
            for (int j = 0; j < kJ; ++j) {
                pr[j][0] = *reinterpret_cast<const uint4*>(slot + qc[j] + t0 + r);
                pr[j][1] = *reinterpret_cast<const uint4*>(slot + qc[j] + t0 + r + 4);
            }
            #pragma unroll
            for (int j = 0; j < kJ; ++j) {
                const uint32_t p8[8] = {pr[j][0].x, pr[j][0].y, pr[j][0].z, pr[j][0].w, pr[j][1].x, pr[j][1].y, pr[j][1].z, pr[j][1].w};
                #pragma unroll
                for (int u = 0; u < 8; ++u) acc[j] = fmaf(h_f(static_cast<uint16_t>(p8[u])), h_f(v[u]), acc[j]);
            }
        }
        for (; r < rows; ++r) {
            const float v = h_f(tile[r * D + e]);
            #pragma unroll
            for (int j = 0; j < kJ; ++j) acc[j] = fmaf(h_f(static_cast<uint16_t>(slot[qc[j] + t0 + r])), v, acc[j]);
        }
    }
    #pragma unroll
    for (int j = 0; j < kJ; ++j) {
        const int qi = qfirst + j * kStep;
        if (qi < nrep) out[static_cast<size_t>(row) * qd + (static_cast<size_t>(g) * nrep + qi) * D + e] = f_h(acc[j]);
    }
}

inline size_t group_attention_lds(int D, int nrep, int seq_cap) {
    return 2 * static_cast<size_t>(kPromptTile) * (D + 4) + 4 * static_cast<size_t>(nrep) * seq_cap;
}

// H[i] = fp16(H[i] + T[i]): the element-wise add behind a projection (QW/kernels/utils.cl element_add)
__global__ void add_rows_kernel(uint16_t* __restrict__ H, const uint16_t* __restrict__ T, long n) {
    for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x)
        H[i] = f_h(h_f(T[i]) + h_f(H[i]));
}

// add_rows_kernel and rmsnorm_kernel in one launch, a wavefront per row: H[r] = fp16(H[r] + T[r]),
// out[r] = rmsnorm(H[r]) * w, with the operations of the two kernels in their order (the row stays
// in registers between them).  For rows of at most 2048 elements, a multiple of 4.
__global__ __launch_bounds__(64) void add_rmsnorm_rows_kernel(uint16_t* __restrict__ H, const uint16_t* __restrict__ T,
                                                              const uint16_t* __restrict__ w, uint16_t* __restrict__ out,
                                                              int cols, float eps) {
    constexpr int kGroups = 8;
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    const int lid = threadIdx.x, c4n = cols >> 2;
    H += static_cast<size_t>(blockIdx.x) * cols;
    T += static_cast<size_t>(blockIdx.x) * cols;
    out += static_cast<size_t>(blockIdx.x) * cols;
    u16x4 xv[kGroups], tv[kGroups], wv[kGroups];
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        const int c4 = lid + 64 * g;
        if (c4 < c4n) {
            xv[g] = *reinterpret_cast<const u16x4*>(H + 4 * c4);
            tv[g] = *reinterpret_cast<const u16x4*>(T + 4 * c4);
            wv[g] = *reinterpret_cast<const u16x4*>(w + 4 * c4);
        }
    }
    float acc = 0.0f;
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        const int c4 = lid + 64 * g;
        if (c4 < c4n) {
            #pragma unroll
            for (int e = 0; e < 4; ++e) xv[g][e] = f_h(h_f(tv[g][e]) + h_f(xv[g][e]));
            *reinterpret_cast<u16x4*>(H + 4 * c4) = xv[g];
            const float v0 = h_f(xv[g][0]), v1 = h_f(xv[g][1]), v2 = h_f(xv[g][2]), v3 = h_f(xv[g][3]);
            float d = v0 * v0;
            d = fmaf(v1, v1, d);
            d = fmaf(v2, v2, d);
            d = fmaf(v3, v3, d);
            acc = acc + d;
        }
    }
    #pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float o = __shfl_down(acc, s, 64);
        acc = acc + o;
    }
    const float total = __shfl(acc, 0, 64);
    const float inv = rcp_rn(sqrtf(__fdiv_rn(total, static_cast<float>(cols)) + eps));
    #pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        const int c4 = lid + 64 * g;
        if (c4 < c4n) {
            u16x4 o;
            #pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = f_h((h_f(xv[g][e]) * inv) * h_f(wv[g][e]));
            *reinterpret_cast<u16x4*>(out + 4 * c4) = o;
        }
    }
}

// gate[i] = swiglu(gate[i], up[i]) over any number of elements, four per thread and step (n is a
// multiple of 4 and both arrays start at multiples of 8 bytes; swiglu_kernel's operations per element)
__global__ void swiglu_rows_kernel(uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, long n) {
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    const long n4 = n >> 2;
    for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += static_cast<long>(gridDim.x) * blockDim.x) {
        u16x4 g4 = *reinterpret_cast<const u16x4*>(gate + 4 * i);
        const u16x4 u4 = *reinterpret_cast<const u16x4*>(up + 4 * i);
        #pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float g = h_f(g4[e]), u = h_f(u4[e]);
            const float sig = rcp_rn(1.0f + exp_poly(-g));
            g4[e] = f_h((g * sig) * u);
        }
        *reinterpret_cast<u16x4*>(gate + 4 * i) = g4;
    }
}

// out[r][c] = swiglu(GU[r][c], GU[r][inter + c]): rows of a stacked gate|up projection ([M, 2 inter]),
// four columns per thread and step (inter a multiple of 4); swiglu_kernel's operations per element
__global__ void swiglu_stacked_kernel(const uint16_t* __restrict__ GU, uint16_t* __restrict__ out, int inter, long n4) {
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    const int c4n = inter >> 2;
    for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += static_cast<long>(gridDim.x) * blockDim.x) {
        const long r = i / c4n;
        const int c = static_cast<int>(i - r * c4n) * 4;
        u16x4 g4 = *reinterpret_cast<const u16x4*>(GU + r * 2 * inter + c);
        const u16x4 u4 = *reinterpret_cast<const u16x4*>(GU + r * 2 * inter + inter + c);
        #pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float g = h_f(g4[e]), u = h_f(u4[e]);
            const float sig = rcp_rn(1.0f + exp_poly(-g));
            g4[e] = f_h((g * sig) * u);
        }
        *reinterpret_cast<u16x4*>(out + r * inter + c) = g4;
    }
}

// the state a prompt leaves behind for the launches that pick the next token: they read the
// last prompt position and advance it
__global__ void set_pos_kernel(State* st, int pos) { st->pos = pos; }

// Dynamic LDS of rope_attention_tiled<D>.
inline size_t tiled_attention_lds(int D, int max_pos) {
    const size_t head = static_cast<size_t>(3 * D + 3 * padded_positions(max_pos) + 8) * 2;
    return head + 2 * static_cast<size_t>(kTileRows) * (D + 8) * 2;
}

__global__ void advance_kernel(State* st) {
    st->token = st->next;
    st->pos = st->pos + 1;
}

struct Decoder {
    mi_decoder_config c{};
    std::vector<const void*> in_norm, post_norm, bq, bk, bv, wq, wk, wv, wo, wgate, wup, wdown;
    const void* embed = nullptr;
    const void* final_norm = nullptr;
    const void* lm_head = nullptr;
    // device memory owned by the decoder
    uint16_t *kc = nullptr, *vc = nullptr, *cosT = nullptr, *sinT = nullptr;
    uint16_t *h = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr;
    uint16_t *qr = nullptr, *kr = nullptr, *vr = nullptr;      // q, k, v after bias and rotary embedding
    uint16_t* rope_now = nullptr;                              // cosines and sines of the current position (embed_kernel)
    uint16_t *gate = nullptr, *up = nullptr, *logits = nullptr;
    State* st = nullptr;
    std::vector<void*> owned;
    // rows of a prompt (mi_decoder_prefill): one allocation, made on the first prompt and again
    // only for a longer one
    void* prompt_mem = nullptr;
    int prompt_rows = 0;
    // q|k|v and gate|up of every layer as one matrix each (rows stacked, scales stacked), copies made
    // with the first prompt: a prompt's projections of one input are then one GEMM instead of three
    // or two.  An entry stays null where a layer's matrices are not of one kind.
    std::vector<void*> wqkv, wgu, stacked_mem;
    bool stacked_built = false;
    // attention with a head's keys split over blocks (mi_decoder_set_attention_splits): 0 = the reference-order launch
    int splits = 0;
    float* split_part = nullptr;                               // [n_heads][splits][head_dim + 2]
};

template <typename T>
bool dev_alloc(Decoder* d, T** p, size_t bytes) {
    void* m = nullptr;
    if (!MI_HIP_OK(hipMalloc(&m, bytes ? bytes : 1))) return false;
    d->owned.push_back(m);
    *p = static_cast<T*>(m);
    return true;
}

uint16_t host_f16(float f) { return mi_f32_to_f16(f); }

}  // namespace
}  // namespace mi

using namespace mi;

extern "C" {

void* mi_decoder_create(const mi_decoder_config* cfg, const mi_decoder_weights* w) {
    if (!cfg || !w || !ensure_init()) return nullptr;
    const mi_decoder_config& c = *cfg;
    if (c.hidden <= 0 || c.inter <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.head_dim <= 0 || c.n_layers <= 0 ||
        c.vocab <= 0 || c.max_pos <= 0 || c.n_heads % c.n_kv_heads || c.head_dim % 4 || c.head_dim > 256 || c.max_pos > kMaxPositions) {
        MI_ERROR_FMT("mi_decoder_create: bad configuration");
        return nullptr;
    }
    auto* d = new Decoder;
    d->c = c;
    const int L = c.n_layers;
    auto take = [L](std::vector<const void*>& dst, const void* const* src) {
        dst.assign(src, src + L);
    };
    take(d->in_norm, w->in_norm); take(d->post_norm, w->post_norm);
    take(d->bq, w->bq); take(d->bk, w->bk); take(d->bv, w->bv);
    take(d->wq, w->wq); take(d->wk, w->wk); take(d->wv, w->wv); take(d->wo, w->wo);
    take(d->wgate, w->wgate); take(d->wup, w->wup); take(d->wdown, w->wdown);
    d->embed = w->embed; d->final_norm = w->final_norm; d->lm_head = w->lm_head;
    // (16 bytes: the GEMV launches that carry the norm in their prologue read it in 16-byte pieces)
    bool aligned = reinterpret_cast<uintptr_t>(w->final_norm) % 16 == 0;
    for (int l = 0; l < L; ++l)
        aligned = aligned && reinterpret_cast<uintptr_t>(w->in_norm[l]) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(w->post_norm[l]) % 16 == 0;
    if (!aligned || c.hidden % 4) {
        MI_ERROR_FMT("mi_decoder_create: norm weights must be 16-byte aligned and hidden a multiple of 4");
        delete d;
        return nullptr;
    }

    const int D = c.head_dim, kvd = c.n_kv_heads * D, qd = c.n_heads * D;
    if (D == 64 || D == 128) {
        // more than 64 KB of LDS per block has to be asked for once per kernel: the most any context length needs
        const size_t most = tiled_attention_lds(D, kMaxPositions);
        const void* kern = D == 64 ? reinterpret_cast<const void*>(rope_attention_tiled<64>)
                                   : reinterpret_cast<const void*>(rope_attention_tiled<128>);
        if (!MI_HIP_OK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(most)))) {
            delete d;
            return nullptr;
        }
    }
    const size_t cache = static_cast<size_t>(L) * c.max_pos * kvd * 2;
    bool ok = dev_alloc(d, &d->kc, cache) && dev_alloc(d, &d->vc, cache) &&
              dev_alloc(d, &d->cosT, static_cast<size_t>(c.max_pos) * D * 2) &&
              dev_alloc(d, &d->sinT, static_cast<size_t>(c.max_pos) * D * 2) &&
              dev_alloc(d, &d->h, c.hidden * 2) && dev_alloc(d, &d->xn, c.hidden * 2) && dev_alloc(d, &d->q, qd * 2) &&
              dev_alloc(d, &d->k, kvd * 2) && dev_alloc(d, &d->v, kvd * 2) && dev_alloc(d, &d->qr, qd * 2) &&
              dev_alloc(d, &d->kr, kvd * 2) && dev_alloc(d, &d->vr, kvd * 2) && dev_alloc(d, &d->attn, qd * 2) &&
              dev_alloc(d, &d->gate, c.inter * 2) &&
              dev_alloc(d, &d->up, c.inter * 2) && dev_alloc(d, &d->logits, static_cast<size_t>(c.vocab) * 2) &&
              dev_alloc(d, &d->st, sizeof(State)) && dev_alloc(d, &d->rope_now, 2 * D * 2);
    if (ok) {
        // rotary tables, QW/src/layers/attention.cpp:133-172: cos/sin(t * theta^(-2i/D)), both halves alike
        std::vector<uint16_t> ct(static_cast<size_t>(c.max_pos) * D), stb(ct.size());
        for (int t = 0; t < c.max_pos; ++t)
            for (int i = 0; i < D / 2; ++i) {
                const float exponent = (2.0f * static_cast<float>(i)) / static_cast<float>(D);
                const float inv_freq = powf(c.rope_theta, -exponent);
                const float angle = static_cast<float>(t) * inv_freq;
                const uint16_t cv = host_f16(cosf(angle)), sv = host_f16(sinf(angle));
                ct[static_cast<size_t>(t) * D + i] = cv; ct[static_cast<size_t>(t) * D + i + D / 2] = cv;
                stb[static_cast<size_t>(t) * D + i] = sv; stb[static_cast<size_t>(t) * D + i + D / 2] = sv;
            }
        const State zero{0, 0, 0};
        ok = MI_HIP_OK(hipMemcpy(d->cosT, ct.data(), ct.size() * 2, hipMemcpyHostToDevice)) &&
             MI_HIP_OK(hipMemcpy(d->sinT, stb.data(), stb.size() * 2, hipMemcpyHostToDevice)) &&
             MI_HIP_OK(hipMemset(d->kc, 0, cache)) && MI_HIP_OK(hipMemset(d->vc, 0, cache)) &&
             MI_HIP_OK(hipMemcpy(d->st, &zero, sizeof zero, hipMemcpyHostToDevice));
    }
    if (!ok) {
        mi_decoder_destroy(d);
        return nullptr;
    }
    return d;
}

int mi_decoder_destroy(void* dec) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d) return 1;
    for (void* p : d->owned) (void)hipFree(p);
    if (d->prompt_mem) (void)hipFree(d->prompt_mem);
    for (void* w : d->wqkv) if (w) mi_unregister_weight(w);
    for (void* w : d->wgu) if (w) mi_unregister_weight(w);
    for (void* p : d->stacked_mem) (void)hipFree(p);
    delete d;
    return 1;
}

int mi_decoder_reset(void* dec, void* stream, int pos, int token) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d || pos < 0 || pos >= d->c.max_pos || token < 0 || token >= d->c.vocab) {
        MI_ERROR_FMT("mi_decoder_reset: bad argument (pos=%d token=%d)", pos, token);
        return 0;
    }
    const State s{pos, token, token};
    auto st = static_cast<hipStream_t>(stream);
    return MI_HIP_OK(hipMemcpyAsync(d->st, &s, sizeof s, hipMemcpyHostToDevice, st)) && MI_HIP_OK(hipStreamSynchronize(st));
}

int mi_decoder_set_token(void* dec, void* stream, int token) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d || token < 0 || token >= d->c.vocab) {
        MI_ERROR_FMT("mi_decoder_set_token: bad argument (token=%d)", token);
        return 0;
    }
    auto st = static_cast<hipStream_t>(stream);
    return MI_HIP_OK(hipMemcpyAsync(reinterpret_cast<char*>(d->st) + offsetof(State, token), &token, sizeof token,
                                    hipMemcpyHostToDevice, st)) && MI_HIP_OK(hipStreamSynchronize(st));
}

int mi_decoder_read(void* dec, void* stream, int* pos, int* token) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d) return 0;
    State s{};
    auto st = static_cast<hipStream_t>(stream);
    if (!MI_HIP_OK(hipMemcpyAsync(&s, d->st, sizeof s, hipMemcpyDeviceToHost, st)) || !MI_HIP_OK(hipStreamSynchronize(st)))
        return 0;
    if (pos) *pos = s.pos;
    if (token) *token = s.token;
    return 1;
}

const void* mi_decoder_logits(void* dec) { return dec ? static_cast<Decoder*>(dec)->logits : nullptr; }

int mi_decoder_set_attention_splits(void* dec, int splits) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d) return 0;
    if (splits <= 1) { d->splits = 0; return 1; }
    const int D = d->c.head_dim;
    if (splits > kMaxSplits || (D != 64 && D != 128)) {
        MI_ERROR_FMT("mi_decoder_set_attention_splits: %d splits at head_dim %d (2..%d, head_dim 64 or 128)", splits, D, kMaxSplits);
        return 0;
    }
    if (!d->split_part &&
        !dev_alloc(d, &d->split_part, static_cast<size_t>(d->c.n_heads) * kMaxSplits * (D + 2) * sizeof(float))) return 0;
    d->splits = splits;
    return 1;
}

const void* mi_decoder_buffer(void* dec, int which) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d) return nullptr;
    switch (which) {
        case 0: return d->h;
        case 1: return d->qr;
        case 2: return d->kr;
        case 3: return d->vr;
        case 4: return d->attn;
        case 5: return d->gate;
        case 6: return d->cosT;
        case 7: return d->sinT;
        default: return nullptr;
    }
}

// The end of a step and of a prompt: final norm, lm_head, greedy token; the token moves into the
// device state and the position advances.  d->h holds the residual stream of the last position.
static int decoder_pick_next(Decoder* d, void* stream) {
    const mi_decoder_config& c = d->c;
    auto s = static_cast<hipStream_t>(stream);
    const int Hd = c.hidden;
    auto launched = [] { return MI_HIP_OK(hipGetLastError()); };
    // (the fused argmax's second launch also does what advance_kernel does)
    void* next = reinterpret_cast<char*>(d->st) + offsetof(State, next);
    bool fused = false;
    if (!linear_argmax(s, c.vocab, Hd, d->h, d->lm_head, d->logits, d->final_norm, c.rms_eps, 32, next, &d->st->token,
                       &d->st->pos, &fused))
        return 0;
    if (fused) return 1;
    {
        // Q4: the throughput GEMV has no norm in its prologue but takes the argmax in its epilogue, and
        // at the lm_head's size it is the faster one: norm as a launch of its own, then that kernel
        WeightKind kind = WK_F16;
        if (!fused_gemv_kind(d->lm_head, c.vocab, Hd, &kind)) return 0;
        if (kind == WK_Q4 || !gemv_takes_norm(kind, Hd)) {
            hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(64), 0, s, d->h, static_cast<const uint16_t*>(d->final_norm), d->xn,
                               Hd, c.rms_eps);
            if (!launched()) return 0;
            if (!linear_argmax(s, c.vocab, Hd, d->xn, d->lm_head, d->logits, nullptr, 0.0f, 32, next, &d->st->token,
                               &d->st->pos, &fused))
                return 0;
            if (fused) return 1;
            if (!mi_linear(stream, 1, c.vocab, Hd, d->xn, d->lm_head, d->logits)) return 0;
            if (!mi_argmax_f16(stream, d->logits, c.vocab, 32, next)) return 0;
            hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(1), 0, s, d->st);
            return launched() ? 1 : 0;
        }
    }
    {
        // the head's GEMV takes the norm in its prologue (checked above) but not the argmax in its epilogue
        const int N1[1] = {c.vocab};
        const void* const W1[1] = {d->lm_head};
        void* const y1[1] = {d->logits};
        if (!fused_gemv(s, 1, N1, Hd, d->h, W1, y1, d->final_norm, c.rms_eps, EPI_STORE)) return 0;
        if (!mi_argmax_f16(stream, d->logits, c.vocab, 32, next)) return 0;
    }
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(1), 0, s, d->st);
    return launched() ? 1 : 0;
}

int mi_decoder_step(void* dec, void* stream) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d) return 0;
    const mi_decoder_config& c = d->c;
    auto s = static_cast<hipStream_t>(stream);
    const int Hd = c.hidden, D = c.head_dim, qd = c.n_heads * D, kvd = c.n_kv_heads * D;
    const float scale = 1.0f / sqrtf(static_cast<float>(D));
    auto launched = [] { return MI_HIP_OK(hipGetLastError()); };
    // Projections of rmsnorm(h) * w.  The norm rides in the GEMV launch where the weights allow it
    // (every wavefront repeats it while its first weights are in flight); otherwise it is a
    // launch of its own into xn.
    // With swiglu set (gate and up projection), y[0] receives swiglu(gate, up) and the SwiGLU
    // rides in the same launch too where it can.
    auto norm_linear = [&](const void* w, int n, const int* N, const void* const* W, void* const* y, bool swiglu) {
        WeightKind kind = WK_F16, k0 = WK_F16;
        bool fuse = true;
        for (int i = 0; i < n; ++i) {
            if (!fused_gemv_kind(W[i], N[i], Hd, &kind)) return false;
            if (i == 0) k0 = kind;
            fuse = fuse && kind == k0 && gemv_takes_norm(kind, Hd);
        }
        if (fuse && swiglu && gemv_takes_swiglu(k0, Hd)) return fused_gemv(s, n, N, Hd, d->h, W, y, w, c.rms_eps, EPI_SWIGLU);
        if (fuse) {
            if (!fused_gemv(s, n, N, Hd, d->h, W, y, w, c.rms_eps, EPI_STORE)) return false;
        } else {
            hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(64), 0, s, d->h, static_cast<const uint16_t*>(w), d->xn, Hd,
                               c.rms_eps);
            if (!launched()) return false;
            mi_linear_call calls[kMaxSegments];
            for (int i = 0; i < n; ++i) calls[i] = mi_linear_call{1, N[i], Hd, d->xn, W[i], y[i]};
            if (mi_linear_batch(stream, calls, n) != n) return false;
        }
        if (swiglu) {
            hipLaunchKernelGGL(swiglu_kernel, dim3((N[0] + 255) / 256), dim3(256), 0, s, static_cast<uint16_t*>(y[0]),
                               static_cast<const uint16_t*>(y[1]), N[0]);
            return launched();
        }
        return true;
    };
    // h = fp16(h + fp16(W x)): the projection and the element-wise add that follows it
    // (QW/kernels/utils.cl element_add), one launch
    auto linear_into_h = [&](int K, const void* x, const void* W) {
        const int N1[1] = {Hd};
        const void* const W1[1] = {W};
        void* const y1[1] = {d->h};
        return fused_gemv(s, 1, N1, K, x, W1, y1, nullptr, 0.0f, EPI_ADD);
    };
    hipLaunchKernelGGL(embed_kernel, dim3(1), dim3(256), 0, s, static_cast<const uint16_t*>(d->embed), d->st, d->h, Hd, c.vocab,
                       d->cosT, d->sinT, d->rope_now, D, c.max_pos);
    if (!launched()) return 0;
    for (int l = 0; l < c.n_layers; ++l) {
        {
            const int N3[3] = {qd, kvd, kvd};
            const void* const W3[3] = {d->wq[l], d->wk[l], d->wv[l]};
            void* const y3[3] = {d->q, d->k, d->v};
            if (!norm_linear(d->in_norm[l], 3, N3, W3, y3, false)) return 0;
        }
        uint16_t* kc = d->kc + static_cast<size_t>(l) * c.max_pos * kvd;
        uint16_t* vc = d->vc + static_cast<size_t>(l) * c.max_pos * kvd;
        const auto *bq = static_cast<const uint16_t*>(d->bq[l]), *bk = static_cast<const uint16_t*>(d->bk[l]),
                   *bv = static_cast<const uint16_t*>(d->bv[l]);
        if (d->splits > 1) {
            const int chunk_cap = ((c.max_pos + d->splits - 1) / d->splits + 3) & ~3;
            const size_t lds = split_attention_lds(D, chunk_cap);
            const dim3 grid(c.n_heads, d->splits);
            if (D == 64) {
                hipLaunchKernelGGL(attention_split_kernel<64>, grid, dim3(kSplitThreads), lds, s, kc, vc, d->st, c.n_heads,
                                   c.n_kv_heads, c.max_pos, scale, d->q, d->k, d->v, bq, bk, bv, d->rope_now, d->qr, d->kr,
                                   d->vr, d->split_part, chunk_cap);
                hipLaunchKernelGGL(attention_merge_kernel<64>, dim3(c.n_heads), dim3(64), 0, s, d->split_part, d->splits, d->attn);
            } else {
                hipLaunchKernelGGL(attention_split_kernel<128>, grid, dim3(kSplitThreads), lds, s, kc, vc, d->st, c.n_heads,
                                   c.n_kv_heads, c.max_pos, scale, d->q, d->k, d->v, bq, bk, bv, d->rope_now, d->qr, d->kr,
                                   d->vr, d->split_part, chunk_cap);
                hipLaunchKernelGGL(attention_merge_kernel<128>, dim3(c.n_heads), dim3(128), 0, s, d->split_part, d->splits, d->attn);
            }
        } else if (D == 64 || D == 128) {
            const size_t lds = tiled_attention_lds(D, c.max_pos);
            if (D == 64)
                hipLaunchKernelGGL(rope_attention_tiled<64>, dim3(c.n_heads), dim3(256), lds, s, kc, vc, d->st, c.n_heads,
                                   c.n_kv_heads, c.max_pos, scale, d->q, d->k, d->v, bq, bk, bv, d->rope_now, d->qr, d->kr,
                                   d->vr, d->attn);
            else
                hipLaunchKernelGGL(rope_attention_tiled<128>, dim3(c.n_heads), dim3(256), lds, s, kc, vc, d->st, c.n_heads,
                                   c.n_kv_heads, c.max_pos, scale, d->q, d->k, d->v, bq, bk, bv, d->rope_now, d->qr, d->kr,
                                   d->vr, d->attn);
        } else {
            // a whole number of wavefronts: the maximum's cross-lane steps read every lane of a wavefront
            const int at = ((D > 64 ? D : 64) + 63) & ~63;
            hipLaunchKernelGGL(rope_attention_kernel, dim3(c.n_heads), dim3(at), static_cast<size_t>(c.max_pos) * 6 + D * 6, s,
                               d->q, d->k, d->v, bq, bk, bv, d->cosT, d->sinT, kc, vc, d->qr, d->kr, d->vr, d->attn,
                               d->st, c.n_heads, c.n_kv_heads, D, c.max_pos, scale);
        }
        if (!launched()) return 0;
        if (!linear_into_h(qd, d->attn, d->wo[l])) return 0;
        {
            const int N2[2] = {c.inter, c.inter};
            const void* const W2[2] = {d->wgate[l], d->wup[l]};
            void* const y2[2] = {d->gate, d->up};
            if (!norm_linear(d->post_norm[l], 2, N2, W2, y2, true)) return 0;
        }
        if (!linear_into_h(c.inter, d->gate, d->wdown[l])) return 0;
    }
    return decoder_pick_next(d, stream);
}

// Rows of n matrices of one kind and K (and their scales) copied into one matrix, registered like
// its parts.  Null when the parts are not of one kind or memory is short; *failed on a HIP error.
static void* stack_weights(Decoder* d, hipStream_t s, int n, const void* const* W, const int* N, int K, bool* failed) {
    WeightKind kind = WK_F16, k0 = WK_F16;
    const void* scale[4] = {nullptr, nullptr, nullptr, nullptr};
    int total = 0;
    for (int i = 0; i < n; ++i) {
        if (!registered_weight(W[i], N[i], K, &kind, &scale[i])) return nullptr;
        if (i == 0) k0 = kind;
        if (kind != k0) return nullptr;
        total += N[i];
    }
    const size_t row = k0 == WK_F16 ? static_cast<size_t>(K) * 2 : k0 == WK_I8 ? static_cast<size_t>(K) : static_cast<size_t>(K) / 2;
    const size_t srow = k0 == WK_I8 ? 2 : k0 == WK_Q4 ? static_cast<size_t>(K / 32) * 2 : 0;
    void *w = nullptr, *sc = nullptr;
    if (hipMalloc(&w, row * total) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    d->stacked_mem.push_back(w);
    if (srow) {
        if (hipMalloc(&sc, srow * total) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
        d->stacked_mem.push_back(sc);
    }
    size_t at = 0;
    for (int i = 0; i < n; ++i) {
        bool ok = MI_HIP_OK(hipMemcpyAsync(static_cast<char*>(w) + at * row, W[i], row * N[i], hipMemcpyDeviceToDevice, s));
        if (ok && srow)
            ok = MI_HIP_OK(hipMemcpyAsync(static_cast<char*>(sc) + at * srow, scale[i], srow * N[i], hipMemcpyDeviceToDevice, s));
        if (!ok) { *failed = true; return nullptr; }
        at += N[i];
    }
    const int reg = k0 == WK_I8 ? mi_register_int8_weight(w, sc, total, K) : k0 == WK_Q4 ? mi_register_q4_weight(w, sc, total, K) : 1;
    return reg ? w : nullptr;
}

// Device rows for a prompt of up to M tokens (H, XN, T [M, hidden]; QKV [M, qd + 2 kvd]; QR, ATT
// [M, qd]; GU [M, 2 inter]; G2 [M, inter]; the token ids).  Grows only; growing waits for the
// stream (an earlier prompt may still be running in the old rows) and reallocates.
static bool ensure_prompt_rows(Decoder* d, hipStream_t s, int M) {
    if (M <= d->prompt_rows) return true;
    const mi_decoder_config& c = d->c;
    const size_t qd = static_cast<size_t>(c.n_heads) * c.head_dim, kvd = static_cast<size_t>(c.n_kv_heads) * c.head_dim;
    const size_t row_halves = 3 * static_cast<size_t>(c.hidden) + 3 * qd + 2 * kvd + 3 * static_cast<size_t>(c.inter);
    if (d->prompt_mem) {
        if (!MI_HIP_OK(hipStreamSynchronize(s))) return false;
        (void)hipFree(d->prompt_mem);
        d->prompt_mem = nullptr;
        d->prompt_rows = 0;
    }
    // every block starts at a multiple of 16 bytes: the row counts are padded to 8 halves per block
    const size_t bytes = (row_halves * M + 10 * 8) * 2 + static_cast<size_t>(M) * 4 + 16;
    if (!MI_HIP_OK(hipMalloc(&d->prompt_mem, bytes))) {
        d->prompt_mem = nullptr;
        return false;
    }
    d->prompt_rows = M;
    return true;
}

// Every layer's q | k | v and gate | up matrices stacked into one registered matrix each, once.
static bool ensure_stacked(Decoder* d, hipStream_t s) {
    if (d->stacked_built) return true;
    const mi_decoder_config& c = d->c;
    const int Hd = c.hidden, qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim, I = c.inter;
    d->wqkv.assign(c.n_layers, nullptr);
    d->wgu.assign(c.n_layers, nullptr);
    bool failed = false;
    for (int l = 0; l < c.n_layers && !failed; ++l) {
        const void* const W3[3] = {d->wq[l], d->wk[l], d->wv[l]};
        const int N3[3] = {qd, kvd, kvd};
        d->wqkv[l] = stack_weights(d, s, 3, W3, N3, Hd, &failed);
        const void* const W2[2] = {d->wgate[l], d->wup[l]};
        const int N2[2] = {I, I};
        if (!failed && I % 4 == 0) d->wgu[l] = stack_weights(d, s, 2, W2, N2, Hd, &failed);
    }
    if (failed) {
        // nothing half-built stays behind: the next prompt starts over, and no registry entry
        // outlives the memory it names
        if (!MI_HIP_OK(hipStreamSynchronize(s))) return false;
        for (void* w : d->wqkv) if (w) mi_unregister_weight(w);
        for (void* w : d->wgu) if (w) mi_unregister_weight(w);
        for (void* p : d->stacked_mem) { mi_unregister_weight(p); (void)hipFree(p); }
        d->wqkv.clear(); d->wgu.clear(); d->stacked_mem.clear();
        return false;
    }
    d->stacked_built = true;
    return true;
}

int mi_decoder_reserve_prompt(void* dec, void* stream, int max_tokens) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d || max_tokens < 1 || max_tokens > d->c.max_pos) {
        MI_ERROR_FMT("mi_decoder_reserve_prompt: bad argument (max_tokens=%d, max_pos=%d)", max_tokens, d ? d->c.max_pos : 0);
        return 0;
    }
    auto s = static_cast<hipStream_t>(stream);
    return ensure_prompt_rows(d, s, max_tokens) && ensure_stacked(d, s) && MI_HIP_OK(hipStreamSynchronize(s)) ? 1 : 0;
}

int mi_decoder_prefill(void* dec, void* stream, const int* tokens, int n_tokens, int pos0) {
    auto* d = static_cast<Decoder*>(dec);
    if (!d || !tokens || n_tokens < 1 || pos0 < 0 || static_cast<long>(pos0) + n_tokens > d->c.max_pos) {
        MI_ERROR_FMT("mi_decoder_prefill: bad argument (n_tokens=%d pos0=%d, max_pos=%d)", n_tokens, pos0,
                     d ? d->c.max_pos : 0);
        return 0;
    }
    const mi_decoder_config& c = d->c;
    auto s = static_cast<hipStream_t>(stream);
    const int M = n_tokens, Hd = c.hidden, D = c.head_dim, qd = c.n_heads * D, kvd = c.n_kv_heads * D, I = c.inter;
    const float scale = 1.0f / sqrtf(static_cast<float>(D));
    auto launched = [] { return MI_HIP_OK(hipGetLastError()); };

    // rows of the prompt (allocated here unless mi_decoder_reserve_prompt has made room already):
    // H, XN, T [M, hidden]; QKV [M, qd + 2 kvd] (q | k | v of a row side by side from the stacked
    // projection, or three blocks of their own); QR, ATT [M, qd]; GU [M, 2 inter] likewise; G2 [M, inter]; tokens
    if (!ensure_prompt_rows(d, s, M)) return 0;
    const int cap = d->prompt_rows;
    auto* base = static_cast<uint16_t*>(d->prompt_mem);
    size_t at = 0;
    auto carve = [&](size_t halves_per_row) {
        uint16_t* p = base + at;
        at += (halves_per_row * cap + 7) & ~static_cast<size_t>(7);
        return p;
    };
    uint16_t *H = carve(Hd), *XN = carve(Hd), *T = carve(Hd), *QKV = carve(qd + 2 * kvd), *QR = carve(qd), *ATT = carve(qd);
    uint16_t *GU = carve(2 * static_cast<size_t>(I)), *G2 = carve(I);
    int* tok = reinterpret_cast<int*>(base + at);

    if (!ensure_stacked(d, s)) return 0;
    if (!MI_HIP_OK(hipMemcpyAsync(tok, tokens, static_cast<size_t>(M) * 4, hipMemcpyHostToDevice, s))) return 0;
    hipLaunchKernelGGL(embed_rows_kernel, dim3(M), dim3(256), 0, s, static_cast<const uint16_t*>(d->embed), tok, H, Hd, c.vocab);
    if (!launched()) return 0;
    const long nH = static_cast<long>(M) * Hd, nI = static_cast<long>(M) * I;
    const unsigned gH = static_cast<unsigned>(nH / 256 + 1 < 4096 ? nH / 256 + 1 : 4096);
    const unsigned gI = static_cast<unsigned>(nI / 1024 + 1 < 8192 ? nI / 1024 + 1 : 8192);
    const size_t att_lds = static_cast<size_t>(D) * 2 * (1 + kPromptTile) + static_cast<size_t>(pos0 + M) * 6;
    if (att_lds > 65536) {
        // (the most any head width and context need, so that one call serves every later shape)
        if (!MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_rows_kernel),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize,
                                                      256 * 2 * (1 + kPromptTile) + kMaxPositions * 6))))
            return 0;
    }
    // one block per key/value head and row where the group's scores fit the LDS of a CU (160 KB, less
    // the kernel's few static bytes)
    constexpr size_t kGroupLdsMost = 160 * 1024 - 256;
    const int nrep = c.n_heads / c.n_kv_heads;
    const int grp_cap = (pos0 + M + 3) & ~3;             // rows of (query, key) entries start at multiples of 16 bytes
    const size_t grp_lds = group_attention_lds(D, nrep, grp_cap);
    const bool grouped = (D == 64 || D == 128) && nrep <= 8 && grp_lds <= kGroupLdsMost;
    if (grouped && grp_lds > 65536) {
        const void* kern = D == 64 ? reinterpret_cast<const void*>(attention_group_kernel<64>)
                                   : reinterpret_cast<const void*>(attention_group_kernel<128>);
        if (!MI_HIP_OK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kGroupLdsMost)))) return 0;
    }
    // H += T, then XN = rmsnorm(H) * w: one launch where a row fits the fused kernel's registers
    const bool add_norm_fused = Hd % 4 == 0 && Hd <= 2048;
    auto add_then_norm = [&](const void* w) {
        if (add_norm_fused) {
            hipLaunchKernelGGL(add_rmsnorm_rows_kernel, dim3(M), dim3(64), 0, s, H, T, static_cast<const uint16_t*>(w), XN, Hd,
                               c.rms_eps);
            return launched();
        }
        hipLaunchKernelGGL(add_rows_kernel, dim3(gH), dim3(256), 0, s, H, T, nH);
        if (!launched()) return false;
        hipLaunchKernelGGL(rmsnorm_kernel, dim3(M), dim3(64), 0, s, H, static_cast<const uint16_t*>(w), XN, Hd, c.rms_eps);
        return launched();
    };
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(M), dim3(64), 0, s, H, static_cast<const uint16_t*>(d->in_norm[0]), XN, Hd,
                       c.rms_eps);
    if (!launched()) return 0;
    for (int l = 0; l < c.n_layers; ++l) {
        uint16_t *Q = QKV, *Kp, *V;
        int ldq, ldkv;
        if (d->wqkv[l]) {
            if (!mi_linear(stream, M, qd + 2 * kvd, Hd, XN, d->wqkv[l], QKV)) return 0;
            Kp = QKV + qd;
            V = Kp + kvd;
            ldq = ldkv = qd + 2 * kvd;
        } else {
            Kp = QKV + static_cast<size_t>(cap) * qd;
            V = Kp + static_cast<size_t>(cap) * kvd;
            ldq = qd;
            ldkv = kvd;
            if (!mi_linear(stream, M, qd, Hd, XN, d->wq[l], Q) || !mi_linear(stream, M, kvd, Hd, XN, d->wk[l], Kp) ||
                !mi_linear(stream, M, kvd, Hd, XN, d->wv[l], V))
                return 0;
        }
        uint16_t* kc = d->kc + static_cast<size_t>(l) * c.max_pos * kvd;
        uint16_t* vc = d->vc + static_cast<size_t>(l) * c.max_pos * kvd;
        hipLaunchKernelGGL(rope_rows_kernel, dim3(M), dim3(256), 0, s, Q, Kp, V, static_cast<const uint16_t*>(d->bq[l]),
                           static_cast<const uint16_t*>(d->bk[l]), static_cast<const uint16_t*>(d->bv[l]), d->cosT, d->sinT,
                           kc, vc, QR, pos0, c.n_heads, c.n_kv_heads, D, ldq, ldkv);
        if (!launched()) return 0;
        if (grouped && D == 64)
            hipLaunchKernelGGL(attention_group_kernel<64>, dim3(c.n_kv_heads, M), dim3(256), grp_lds, s, QR, kc, vc, ATT, pos0,
                               grp_cap, c.n_heads, c.n_kv_heads, scale);
        else if (grouped)
            hipLaunchKernelGGL(attention_group_kernel<128>, dim3(c.n_kv_heads, M), dim3(256), grp_lds, s, QR, kc, vc, ATT, pos0,
                               grp_cap, c.n_heads, c.n_kv_heads, scale);
        else
            hipLaunchKernelGGL(attention_rows_kernel, dim3(c.n_heads, M), dim3(256), att_lds, s, QR, kc, vc, ATT, pos0, pos0 + M,
                               c.n_heads, c.n_kv_heads, D, scale);
        if (!launched()) return 0;
        if (!mi_linear(stream, M, Hd, qd, ATT, d->wo[l], T)) return 0;
        if (!add_then_norm(d->post_norm[l])) return 0;
        const uint16_t* act;                      // swiglu(gate, up), [M, inter]
        if (d->wgu[l]) {
            if (!mi_linear(stream, M, 2 * I, Hd, XN, d->wgu[l], GU)) return 0;
            hipLaunchKernelGGL(swiglu_stacked_kernel, dim3(gI), dim3(256), 0, s, GU, G2, I, nI / 4);
            act = G2;
        } else {
            uint16_t *G = GU, *U = GU + static_cast<size_t>(cap) * I;
            if (!mi_linear(stream, M, I, Hd, XN, d->wgate[l], G) || !mi_linear(stream, M, I, Hd, XN, d->wup[l], U)) return 0;
            if (I % 4 == 0) {
                hipLaunchKernelGGL(swiglu_rows_kernel, dim3(gI), dim3(256), 0, s, G, U, nI);
            } else {
                if (nI > 2147483647L) return 0;
                hipLaunchKernelGGL(swiglu_kernel, dim3(gI), dim3(256), 0, s, G, U, static_cast<int>(nI));
            }
            act = G;
        }
        if (!launched()) return 0;
        if (!mi_linear(stream, M, Hd, I, act, d->wdown[l], T)) return 0;
        if (l + 1 < c.n_layers) {
            if (!add_then_norm(d->in_norm[l + 1])) return 0;     // the next layer's input norm rides along
        } else {
            hipLaunchKernelGGL(add_rows_kernel, dim3(gH), dim3(256), 0, s, H, T, nH);
            if (!launched()) return 0;
        }
    }
    // only the last position picks a token: its residual stream becomes the single-token state
    if (!MI_HIP_OK(hipMemcpyAsync(d->h, H + static_cast<size_t>(M - 1) * Hd, static_cast<size_t>(Hd) * 2,
                                  hipMemcpyDeviceToDevice, s)))
        return 0;
    hipLaunchKernelGGL(set_pos_kernel, dim3(1), dim3(1), 0, s, d->st, pos0 + M - 1);
    if (!launched()) return 0;
    return decoder_pick_next(d, stream);
}


}  // extern "C"
