// Prefill GEMM for gfx950: out[M,N] = x[M,K] * W[N,K]^T on the matrix cores, with the weight
// dequantisation fused into the tile load.  fp16 activations, fp16 or per-row int8 weights,
// fp32 accumulation (v_mfma_f32_32x32x16_f16), fp16 output.
//
// Semantics follow the reference's M > 1 path: row i of out is the GEMV of row i of x
// (LF/src/model.cpp:243-250); for int8 the per-row scale multiplies the fp32 sum once, in the
// epilogue, as the int8 GEMV does (LF/kernels/gemv_m1_int8.cl:69-77).  int8 weights convert
// exactly to fp16, so every product is exact in fp32; only the order of the fp32 additions
// differs from the GEMV kernels (results agree to fp32 rounding, not bit for bit).
//
// Both operands are K-contiguous, so a block stages a BM x 64 tile of x and a BN x 64 tile of W
// through LDS (rows padded to 72 halves: 16-byte reads of 8 consecutive rows then fall in
// 8 different bank groups; two LDS stages) while the loads of the next three K-tiles are
// already in flight in registers.  Four wavefronts per block, each owning a WM x WN sub-tile as (WM/32) x (WN/32)
// accumulators of 32 x 32.
#include "common.h"
#include <hip/hip_fp16.h>
#include <type_traits>
#include <utility>

namespace mi {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kKT = 64;            // K-tile, elements
constexpr int kLd = kKT + 8;       // LDS row stride, halves
constexpr int kThreads = 256;

__device__ __forceinline__ uint16_t to_half_bits(float f) {
    asm volatile("" : "+v"(f));    // round the fp32 value first, then convert (two roundings, as the GEMV path)
    return __half_as_ushort(__float2half_rn(f));
}

// Four int8 in one dword -> four fp16 (two dwords), exact: byte ^ 0x80 is q + 128, the byte
// permute builds the halves 1024 + (q + 128), and subtracting 1152 leaves q.
__device__ __forceinline__ void i8x4_to_h4(uint32_t v, uint32_t& lo, uint32_t& hi) {
    const uint32_t u = v ^ 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
    const __half2 k = __builtin_bit_cast(__half2, 0x64806480u);               // 1152, 1152
    lo = __builtin_bit_cast(uint32_t, __hsub2(__builtin_bit_cast(__half2, a), k));
    hi = __builtin_bit_cast(uint32_t, __hsub2(__builtin_bit_cast(__half2, b), k));
}

// Byte B of v holds two Q4 values, low nibble first.  Returns them as a pair of fp16 times the
// pair s2: the nibbles are placed into the mantissas of 1024 (unit 1) and of 64 (unit 1/16, which
// is where a high nibble sits), 1032 and 72 are subtracted (exact), and the product with the
// scale is rounded to fp16 once.
template <int B>
__device__ __forceinline__ uint32_t q4x2_to_h2(uint32_t v, __half2 s2) {
    const uint32_t t = __builtin_amdgcn_perm(0u, v, 0x0C000C00u | (B << 16) | B);
    const uint32_t h = (t & 0x00F0000Fu) | 0x54006400u;
    const __half2 k = __builtin_bit_cast(__half2, 0xD480E408u);               // -1032, -72
    return __builtin_bit_cast(uint32_t, __hmul2(__hadd2(__builtin_bit_cast(__half2, h), k), s2));
}

template <int BM, int BN, int WM, int WN, int KIND>
__global__ __launch_bounds__(kThreads) void gemm_kernel(const uint16_t* __restrict__ X,
                                                        const uint8_t* __restrict__ W,
                                                        const uint16_t* __restrict__ scale,
                                                        uint16_t* __restrict__ out, int M, int N, int K) {
    static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_CHUNKS = BM * (kKT / 8) / kThreads;                      // 16-byte chunks of x per thread
    constexpr int B_BYTES = KIND == WK_I8 ? 1 : 2;
    constexpr int B_CPR = kKT * B_BYTES / 16;                                // 16-byte chunks per W row and K-tile
    constexpr int B_CHUNKS = BN * B_CPR / kThreads;
    static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");

    // Two LDS stages (x tile then W tile in each) and kStages register stages: the global
    // loads of K-tile i + kStages are issued while tile i is multiplied, which is what hides
    // the HBM / L2 latency (one tile ahead is far too short for it).
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    constexpr int kStageHalves = (BM + BN) * kLd;

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int gk = lane / 32, li = lane % 32;

    floatx16 acc[TM][TN];
    #pragma unroll
    for (int t = 0; t < TM; ++t)
        #pragma unroll
        for (int u = 0; u < TN; ++u)
            #pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][u][r] = 0.0f;

    struct Regs { u32x4 a[A_CHUNKS]; u32x4 b[B_CHUNKS]; };
    auto load_tile = [&](Regs& R, int k0) {
        #pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * kThreads, row = c / (kKT / 8), kc = c % (kKT / 8);
            const int m = m0 + row < M ? m0 + row : M - 1;          // rows past M are never stored
            R.a[i] = *reinterpret_cast<const u32x4*>(X + static_cast<size_t>(m) * K + k0 + kc * 8);
        }
        #pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            const int c = tid + i * kThreads, row = c / B_CPR, kc = c % B_CPR;
            const int n = n0 + row < N ? n0 + row : N - 1;
            R.b[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                W + (static_cast<size_t>(n) * K + k0) * B_BYTES + kc * 16));
        }
    };
    auto store_tile = [&](const Regs& R, uint16_t* As, uint16_t* Bs) {
        #pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * kThreads, row = c / (kKT / 8), kc = c % (kKT / 8);
            *reinterpret_cast<u32x4*>(&As[row * kLd + kc * 8]) = R.a[i];
        }
        #pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            const int c = tid + i * kThreads, row = c / B_CPR, kc = c % B_CPR;
            if constexpr (KIND == WK_I8) {
                uint32_t h[8];
                i8x4_to_h4(R.b[i].x, h[0], h[1]);
                i8x4_to_h4(R.b[i].y, h[2], h[3]);
                i8x4_to_h4(R.b[i].z, h[4], h[5]);
                i8x4_to_h4(R.b[i].w, h[6], h[7]);
                *reinterpret_cast<u32x4*>(&Bs[row * kLd + kc * 16]) = u32x4{h[0], h[1], h[2], h[3]};
                *reinterpret_cast<u32x4*>(&Bs[row * kLd + kc * 16 + 8]) = u32x4{h[4], h[5], h[6], h[7]};
            } else {
                *reinterpret_cast<u32x4*>(&Bs[row * kLd + kc * 8]) = R.b[i];
            }
        }
    };
    auto multiply = [&](const uint16_t* As, const uint16_t* Bs) {
        #pragma unroll
        for (int kk = 0; kk < kKT / 16; ++kk) {
            // lane group gk supplies k = 32 gk + 8 kk .. +7 of the tile, for both operands
            const int kcol = 32 * gk + 8 * kk;
            half8 a[TM], b[TN];
            #pragma unroll
            for (int t = 0; t < TM; ++t)
                a[t] = *reinterpret_cast<const half8*>(&As[(wm * WM + t * 32 + li) * kLd + kcol]);
            #pragma unroll
            for (int u = 0; u < TN; ++u)
                b[u] = *reinterpret_cast<const half8*>(&Bs[(wn * WN + u * 32 + li) * kLd + kcol]);
            #pragma unroll
            for (int t = 0; t < TM; ++t)
                #pragma unroll
                for (int u = 0; u < TN; ++u)
                    acc[t][u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[t], b[u], acc[t][u], 0, 0, 0);
        }
    };

    const int nk = K / kKT;
    Regs R0, R1, R2;
    load_tile(R0, 0);
    load_tile(R1, (1 < nk ? 1 : nk - 1) * kKT);
    load_tile(R2, (2 < nk ? 2 : nk - 1) * kKT);
    // One step: tile i goes registers -> LDS stage i % 2; one barrier publishes it (and, being
    // the second barrier since stage i % 2 was last read, also guards the overwrite); the
    // freed registers take tile i + 3; the matrix cores run on tile i.
#define MI_GEMM_STEP(R)                                                        \
    {                                                                          \
        uint16_t* As = lds + (i & 1) * kStageHalves;                           \
        uint16_t* Bs = As + BM * kLd;                                          \
        store_tile(R, As, Bs);                                                 \
        __syncthreads();                                                       \
        load_tile(R, (i + 3 < nk ? i + 3 : nk - 1) * kKT);                     \
        multiply(As, Bs);                                                      \
        if (++i >= nk) break;                                                  \
    }
    for (int i = 0;;) {
        MI_GEMM_STEP(R0)
        MI_GEMM_STEP(R1)
        MI_GEMM_STEP(R2)
    }
#undef MI_GEMM_STEP

    // D[i][j]: j = lane % 32 (a W row, i.e. an output column), i = 8 (r / 4) + 4 (lane / 32) + r % 4.
    #pragma unroll
    for (int u = 0; u < TN; ++u) {
        const int n = n0 + wn * WN + u * 32 + li;
        if (n >= N) continue;
        float s = 1.0f;
        if constexpr (KIND == WK_I8) s = __half2float(__ushort_as_half(scale[n]));
        #pragma unroll
        for (int t = 0; t < TM; ++t) {
            #pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WM + t * 32 + 8 * (r / 4) + 4 * gk + r % 4;
                if (m < M) {
                    const float v = KIND == WK_I8 ? acc[t][u][r] * s : acc[t][u][r];
                    out[static_cast<size_t>(m) * N + n] = to_half_bits(v);
                }
            }
        }
    }
}

// ---- wide tiles fed by direct global -> LDS loads (int8, Q4 and fp16 weights) ----------
//
// What bounds the kernel above is the rate at which a CU can fill LDS (about 150 bytes/ns,
// against 530 bytes/ns for reads and one 32x32x16 MFMA per 15.6 ns per SIMD) and the fragment
// reads that are not overlapped with the MFMAs of the same wavefront.  This kernel therefore
//  * keeps quantised W as it is stored (int8, or Q4 nibbles with their block scales) in LDS
//    (a half or a quarter of the fill bytes) and converts a fragment to fp16 in registers after
//    reading it; the four wavefronts of a block own disjoint rows of W (64 each, so the block
//    covers 256 rows of W) and share the 32*TM rows of x, so no fragment of W is converted twice;
//  * fills LDS with global_load_lds_dwordx4 (no registers, no ds_write), three to eight stages of
//    K = 64; 16-byte chunks are XOR-swizzled inside a row so that fragment reads are conflict-free
//    without padding (a wavefront's load always fills 1 KB of consecutive LDS);
//  * reads the fragments of the next 32 values of K before issuing the MFMAs of the current
//    ones, with one barrier per stage placed in the middle of a stage, where the data of the
//    next stage is known to have landed;
//  * orders K inside a group of 32 so that a lane's 16 consecutive weights feed two MFMAs: lanes
//    0-31 supply k = 0..7 then 8..15, lanes 32-63 supply 16..23 then 24..31, for W and x alike.
// W is the MFMA "A" operand and x the "B" operand, so a lane ends up with four consecutive
// output columns of one output row and stores them as 8 bytes.
namespace wide {

constexpr int kBN = 256;                    // rows of W per block
// LDS stages (K = 64 each) for 32 * tm rows of x.  A stage is requested stages - 2 stage times
// before it is needed, which is what covers the load latency.  Tall tiles (tm >= 3) take as many
// stages as 160 KB hold.  Low tiles of quantised weights take half of the LDS (3 or 4 stages), so
// that two blocks share a CU: they belong to shapes with many small tiles, where one block's
// prologue and epilogue then overlap the other's main loop (lm_head at M = 16: 37 -> 29 us).
constexpr int stages_for(int kind, int tm) {
    return kind == WK_Q4 ? (tm >= 5 ? 5 : tm == 4 ? 6 : tm == 3 ? 7 : 4)
         : kind == WK_F16 ? (tm >= 3 ? 3 : 4)
                          : (tm >= 4 ? 4 : tm == 3 ? 5 : tm == 2 ? 3 : 4);
}
// blocks of such a tile that fit one CU
constexpr int blocks_per_cu(int kind, int tm) { return kind != WK_F16 && tm <= 2 ? 2 : 1; }
// bytes of W per stage: int8 rows of 64 bytes; fp16 rows of 128 bytes; Q4 rows of 32 bytes of
// packed nibbles followed by the 256 rows' two block scales (fp16) each
constexpr int w_stage_bytes(int kind) {
    return kind == WK_Q4 ? kBN * 32 + kBN * 4 : kind == WK_F16 ? kBN * 128 : kBN * 64;
}
typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef __attribute__((address_space(1))) const uint8_t glb_u8;

__device__ __forceinline__ void lds_fill16(const uint8_t* g, uint8_t* l) {
    __builtin_amdgcn_global_load_lds((glb_u8*)g, (lds_u8*)l, 16, 0, 0);   // address-space casts
}
__device__ __forceinline__ void lds_fill4(const uint8_t* g, uint8_t* l) {
    __builtin_amdgcn_global_load_lds((glb_u8*)g, (lds_u8*)l, 4, 0, 0);
}
#define MI_LDS_READ8(dst, addr, imm) \
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(imm))
#define MI_LDS_READ4(dst, addr, imm) \
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(imm))
#define MI_LDS_READ16(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(imm))
#define MI_WAIT_LGKM(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n) : "memory")
#define MI_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
#define MI_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): indices are compile-time
// constants inside f (immediate operands, register array subscripts)
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

typedef float float2v __attribute__((ext_vector_type(2)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
// two fp32 values, already rounded to fp32, to a pair of fp16 (round to nearest even): one
// v_cvt_pk_f16_f32
__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    float2v v = {a, b};
    asm volatile("" : "+v"(v));    // keep the fp32 rounding of the products: no fused multiply-convert
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, half2v));
}

template <int TM>
struct Frags {
    u32x4 w[2];          // int8: 16 weights of two 32-row fragments of W, as read from LDS
    uint2 w4[2];         // Q4: the same, 8 bytes
    uint32_t ws[2];      // Q4: the two block scales of the stage, of the lane's row in either fragment
    uint32_t wf[2][2][4];  // the same as fp16: [fragment][MFMA of the pair][4 dwords = 8 halves]
    uint32_t wg[2][2][4];  // Q4 in two terms: the second term
    u32x4 wh[2][2];        // fp16 weights: read from LDS as they are used
    u32x4 x[2][TM];      // [MFMA of the pair][32-row fragment of x], 8 halves each
};

template <int TM, int KIND, int TERMS>
__global__ __launch_bounds__(256) void gemm_wide(const uint16_t* __restrict__ X,
                                                   const uint8_t* __restrict__ W,
                                                   const uint16_t* __restrict__ scale,
                                                   uint16_t* __restrict__ out, int M, int N, int K,
                                                   float* __restrict__ partial, int splits) {
    constexpr int BM = 32 * TM;
    constexpr int kXStage = BM * 128;                    // bytes of x (fp16) per stage
    constexpr bool Q4 = KIND == WK_Q4, F16 = KIND == WK_F16;
    constexpr int kWRow = Q4 ? 32 : F16 ? 128 : 64;      // bytes of one row of W per stage
    constexpr int kWLoads = Q4 ? 3 : F16 ? 8 : 4;        // Q4: two loads of nibbles, one of scales
    constexpr int kWReads = Q4 || F16 ? 4 : 2;           // Q4: two fragments, two scale pairs; fp16: two fragments for two MFMAs
    constexpr int kConv = F16 ? 0 : 8;                   // conversions per set of fragments
    constexpr int kScaleAt = kXStage + kBN * 32;         // Q4: the scales of a stage, 4 bytes per row of W
    constexpr int kStage = kXStage + w_stage_bytes(KIND);
    constexpr int kLoads = TM + kWLoads;                 // global -> LDS loads per wavefront and stage
    constexpr int kStages = stages_for(KIND, TM);
    constexpr int kReads = kWReads + 2 * TM;             // LDS reads per set of fragments
    constexpr int kMfmas = 4 * TM * TERMS;               // MFMAs per half stage (K = 32)
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, li = lane & 31;
    // Block -> tile.  Blocks go to the 8 XCDs round-robin and every XCD has its own L2, so XCD x
    // takes the x-th contiguous eighth of the tile list, and the list runs through bands of 4
    // tiles along N, down M inside a band: the tiles that are in flight on one XCD at the same
    // time then share rows of x and of W and fetch them into that L2 once.
    // With splits > 1 the list holds every tile once per slice of K (slice-major); a block then
    // sums its slice only and leaves fp32 partial sums for reduce_partials.
    int tile_m, tile_n, split;
    {
        const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + kBN - 1) / kBN, tiles = tiles_m * tiles_n;
        const int total = tiles * splits;
        const int per_xcd = (total + 7) / 8;
        int l = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (blockIdx.x >= 8 * per_xcd || l >= total) return;          // whole block, before any barrier
        split = l / tiles;
        l -= split * tiles;
        constexpr int kBand = 4;
        const int band = l / (kBand * tiles_m);
        const int width = tiles_n - band * kBand < kBand ? tiles_n - band * kBand : kBand;
        const int in_band = l - band * kBand * tiles_m;
        tile_m = in_band / width;
        tile_n = band * kBand + in_band % width;
    }
    const int m0 = tile_m * BM, n0 = tile_n * kBN;
    const uint32_t lbase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_u8*)lds));

    // per-row scales of this lane's output columns, requested before anything else so that they
    // are in registers long before the epilogue: sc[u][rq] = 4 fp16 scales of columns nq .. nq + 3
    // (Q4 has no per-row scale: the block scales travel with the weights)
    const bool cols4 = (N % 4) == 0 && reinterpret_cast<uintptr_t>(scale) % 8 == 0;
    uint2 sc[2][4];
    #pragma unroll
    for (int u = 0; u < 2; ++u) {
        #pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            const int nq = n0 + 64 * w + 32 * u + 8 * rq + 4 * g;
            if constexpr (Q4 || F16) {
                sc[u][rq] = uint2{0u, 0u};
            } else if (cols4 && nq + 3 < N) {
                sc[u][rq] = *reinterpret_cast<const uint2*>(scale + nq);
            } else {
                uint32_t h[4];
                #pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = scale[nq + e < N ? nq + e : N - 1];
                sc[u][rq] = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
            }
        }
    }

    // --- fill side: lane i of load j writes LDS bytes [1024 j + 16 i, +16) of its region --------
    // x: load j covers rows 8j..8j+7 (128 bytes each, 8 chunks); slot p of row r holds chunk p ^ ((r >> 1) & 7)
    // W: load j covers rows 16j..16j+15 (64 bytes each, 4 chunks); slot p of row r holds chunk p ^ ((r >> 2) & 3)
    // W, Q4: load j covers rows 32j..32j+31 (32 bytes each, 2 chunks); slot p of row r holds chunk
    //        p ^ ((r >> 3) & 1); a third load of 4 bytes per lane brings the two block scales of
    //        the wavefront's own 64 rows
    // W, fp16: as x, load j covers rows 8j..8j+7, eight loads for the wavefront's own 64 rows
    uint32_t xsrc[TM], wsrc[F16 ? 8 : 4];
    #pragma unroll
    for (int jj = 0; jj < TM; ++jj) {
        const int r = 8 * (w + 4 * jj) + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        const int m = m0 + r < M ? m0 + r : M - 1;
        xsrc[jj] = static_cast<uint32_t>(m) * K * 2u + c * 16u;
    }
    if constexpr (Q4) {
        #pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int r = 32 * (2 * w + jj) + (lane >> 1);
            const int c = (lane & 1) ^ ((r >> 3) & 1);
            const int n = n0 + r < N ? n0 + r : N - 1;
            wsrc[jj] = static_cast<uint32_t>(n) * (K / 2) + c * 16u;
        }
        const int r = 64 * w + lane;
        const int n = n0 + r < N ? n0 + r : N - 1;
        wsrc[2] = static_cast<uint32_t>(n) * (K / 32) * 2u;
        wsrc[3] = 0u;
    } else if constexpr (F16) {
        #pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
            const int r = 8 * (8 * w + jj) + (lane >> 3);
            const int c = (lane & 7) ^ ((r >> 1) & 7);
            const int n = n0 + r < N ? n0 + r : N - 1;
            wsrc[jj] = static_cast<uint32_t>(n) * K * 2u + c * 16u;
        }
    } else {
        #pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int r = 16 * (4 * w + jj) + (lane >> 2);
            const int c = (lane & 3) ^ ((r >> 2) & 3);
            const int n = n0 + r < N ? n0 + r : N - 1;
            wsrc[jj] = static_cast<uint32_t>(n) * K + c * 16u;
        }
    }
    const uint8_t* Sb = reinterpret_cast<const uint8_t*>(scale);  // Q4: advanced like W below
    const uint8_t* Xb = reinterpret_cast<const uint8_t*>(X);     // both advanced to the block's first K-stage below
    // load j (0 .. kLoads - 1) of this wavefront for K-stage stage_k into LDS slot `slot`
    auto fill_one = [&](int stage_k, int slot, auto jc) {
        constexpr int j = decltype(jc)::value;
        uint8_t* xs = lds + slot * kStage;
        if constexpr (j < TM)
            lds_fill16(Xb + static_cast<size_t>(stage_k) * 128 + xsrc[j], xs + 1024 * (w + 4 * j));
        else if constexpr (F16)
            lds_fill16(W + static_cast<size_t>(stage_k) * 128 + wsrc[j - TM], xs + kXStage + 1024 * (8 * w + (j - TM)));
        else if constexpr (!Q4)
            lds_fill16(W + static_cast<size_t>(stage_k) * 64 + wsrc[j - TM], xs + kXStage + 1024 * (4 * w + (j - TM)));
        else if constexpr (j - TM < 2)
            lds_fill16(W + static_cast<size_t>(stage_k) * 32 + wsrc[j - TM], xs + kXStage + 1024 * (2 * w + (j - TM)));
        else
            lds_fill4(Sb + static_cast<size_t>(stage_k) * 4 + wsrc[2], xs + kScaleAt + 256 * w);
    };
    auto fill_stage = [&](int stage_k, int slot) {
        static_for<kLoads>([&](auto jc) { fill_one(stage_k, slot, jc); });
    };

    // --- read side -------------------------------------------------------------------------------
    // pair S (0, 1) of a stage, MFMA e (0, 1) of the pair: x chunk 4S + 2g + e, W chunk 2S + g
    const uint32_t xrow = lbase + li * 128u, xq = (2u * g) ^ ((li >> 1) & 7u);
    // Q4: bytes 16 S + 8 g .. + 7 of the row: chunk S, its lower or upper half
    // fp16: as x (the swizzle of rows li and li + 32 is the same)
    const uint32_t wrow = lbase + kXStage + (64u * w + li) * kWRow, wq = Q4 ? (li >> 3) & 1u : g ^ ((li >> 2) & 3u);
    const uint32_t soff = lbase + kScaleAt + (64u * w + li) * 4u;
    uint32_t xoff[2][2], woff[2], whoff[2][2];
    #pragma unroll
    for (int S = 0; S < 2; ++S) {
        #pragma unroll
        for (int e = 0; e < 2; ++e) {
            xoff[S][e] = xrow + (((4u * S + e) ^ xq) << 4);
            whoff[S][e] = wrow + (((4u * S + e) ^ xq) << 4);
        }
        woff[S] = Q4 ? wrow + ((S ^ wq) << 4) + 8u * g : wrow + (((2u * S) ^ wq) << 4);
    }
    // LDS read j (0 .. kReads - 1) of a set: the two W fragments first, then x for the first and
    // the second MFMA of the pair
    auto read_one = [&](Frags<TM>& F, uint32_t slot_bytes, auto Sc, auto jc) {
        constexpr int S = decltype(Sc)::value, j = decltype(jc)::value;
        if constexpr (F16 && j < kWReads) {
            const uint32_t a = whoff[S][j % 2] + slot_bytes;
            MI_LDS_READ16(F.wh[j / 2][j % 2], a, (j / 2) * 32 * kWRow);
        } else if constexpr (j < 2) {
            const uint32_t a = woff[S] + slot_bytes;
            if constexpr (Q4) {
                MI_LDS_READ8(F.w4[j], a, j * 32 * kWRow);
            } else {
                MI_LDS_READ16(F.w[j], a, j * 32 * kWRow);
            }
        } else if constexpr (j < kWReads) {
            const uint32_t a = soff + slot_bytes;
            MI_LDS_READ4(F.ws[j - 2], a, (j - 2) * 32 * 4);
        } else {
            constexpr int e = (j - kWReads) / TM, t = (j - kWReads) % TM;
            const uint32_t a = xoff[S][e] + slot_bytes;
            MI_LDS_READ16(F.x[e][t], a, t * 4096);
        }
    };
    // conversion j (0 .. 7) of a set: dword j % 4 of W fragment j / 4 becomes four halves
    // Q4 (S = pair of the stage, which selects the block scale): bytes 2 (d % 2), 2 (d % 2) + 1 of
    // dword d / 2 of fragment j / 4 become four halves, scaled
    auto convert_one = [&](Frags<TM>& F, auto Sc, auto jc) {
        constexpr int j = decltype(jc)::value, u = j / 4, d = j % 4;
        if constexpr (Q4) {
            constexpr int S = decltype(Sc)::value;
            const uint32_t sb = __builtin_amdgcn_perm(0u, F.ws[u], S ? 0x03020302u : 0x01000100u);
            const uint32_t v = d / 2 ? F.w4[u].y : F.w4[u].x;
            if constexpr (TERMS == 2) {
                // scale = hi + lo with 7 and 4 significant bits: q * hi and q * lo are exact in
                // fp16 and add up to q * scale in the fp32 accumulator
                const uint32_t hi = sb & 0xFFF0FFF0u;
                const __half2 s2 = __builtin_bit_cast(__half2, hi);
                const __half2 r2 = __hsub2(__builtin_bit_cast(__half2, sb), s2);
                F.wf[u][d / 2][2 * (d % 2)] = q4x2_to_h2<2 * (d % 2)>(v, s2);
                F.wf[u][d / 2][2 * (d % 2) + 1] = q4x2_to_h2<2 * (d % 2) + 1>(v, s2);
                F.wg[u][d / 2][2 * (d % 2)] = q4x2_to_h2<2 * (d % 2)>(v, r2);
                F.wg[u][d / 2][2 * (d % 2) + 1] = q4x2_to_h2<2 * (d % 2) + 1>(v, r2);
            } else {
                const __half2 s2 = __builtin_bit_cast(__half2, sb);
                F.wf[u][d / 2][2 * (d % 2)] = q4x2_to_h2<2 * (d % 2)>(v, s2);
                F.wf[u][d / 2][2 * (d % 2) + 1] = q4x2_to_h2<2 * (d % 2) + 1>(v, s2);
            }
        } else {
            i8x4_to_h4(F.w[u][d], F.wf[u][d / 2][2 * (d % 2)], F.wf[u][d / 2][2 * (d % 2) + 1]);
        }
    };

    floatx16 acc[2][TM];
    #pragma unroll
    for (int u = 0; u < 2; ++u)
        #pragma unroll
        for (int t = 0; t < TM; ++t)
            #pragma unroll
            for (int r = 0; r < 16; ++r) acc[u][t][r] = 0.0f;

    // MFMA n (0 .. kMfmas - 1) of a half stage; consecutive n use different accumulators
    auto mfma_one = [&](const Frags<TM>& F, auto nc) {
        constexpr int n = decltype(nc)::value, c = n / (2 * TM), e = c % 2, u = (n / TM) % 2, t = n % TM;
        const u32x4 wv = F16 ? F.wh[u][e]
                       : c / 2 ? u32x4{F.wg[u][e][0], F.wg[u][e][1], F.wg[u][e][2], F.wg[u][e][3]}
                               : u32x4{F.wf[u][e][0], F.wf[u][e][1], F.wf[u][e][2], F.wf[u][e][3]};
        acc[u][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, wv),
                                                          __builtin_bit_cast(half8, F.x[e][t]), acc[u][t], 0, 0, 0);
    };

    // One half stage.  An MFMA keeps the matrix pipe busy for 32 cycles but issues in 4, and a
    // wavefront issues in order: whatever else has to happen (LDS fills for a later stage, the
    // LDS reads of the next fragments, their int8 -> fp16 conversion) is dealt out between the
    // MFMAs, so that it runs in their shadow instead of draining the pipe.
    //   C  = fragments being multiplied; Nx = fragments being prepared (LDS slot at next_bytes,
    //   pair NS of that stage); FILL: also issue this wavefront's fills of stage fill_k.
    auto half_stage = [&](Frags<TM>& C, Frags<TM>& Nx, uint32_t next_bytes, auto NSc, auto fillc,
                          int fill_k, int fill_slot) {
        constexpr bool FILL = decltype(fillc)::value;
        constexpr int nF = FILL ? kLoads : 0;
        constexpr int A = nF + kReads + (kConv ? 1 + kConv : 0);   // fills, reads, wait for W, conversions
        static_for<kMfmas>([&](auto nc) {
            constexpr int n = decltype(nc)::value;
            mfma_one(C, nc);
            MI_SCHED_FENCE();
            constexpr int a0 = n * A / kMfmas, a1 = (n + 1) * A / kMfmas;
            static_for<a1 - a0>([&](auto kc) {
                constexpr int a = a0 + decltype(kc)::value;
                if constexpr (a < nF) {
                    fill_one(fill_k, fill_slot, std::integral_constant<int, a>{});
                } else if constexpr (a < nF + kReads) {
                    read_one(Nx, next_bytes, NSc, std::integral_constant<int, a - nF>{});
                } else if constexpr (a == nF + kReads) {
                    // LDS returns in order: the two W reads are back.  The registers are operands
                    // of the wait so that the conversions that read them cannot be moved above it.
                    if constexpr (F16)
                        ;
                    else if constexpr (Q4)
                        asm volatile("s_waitcnt lgkmcnt(%4)"
                                     : "+v"(Nx.w4[0]), "+v"(Nx.w4[1]), "+v"(Nx.ws[0]), "+v"(Nx.ws[1])
                                     : "n"(kReads - kWReads) : "memory");
                    else
                        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(Nx.w[0]), "+v"(Nx.w[1]) : "n"(kReads - kWReads) : "memory");
                    MI_SCHED_FENCE();
                } else {
                    convert_one(Nx, NSc, std::integral_constant<int, a - nF - kReads - 1>{});
                }
            });
            MI_SCHED_FENCE();
        });
        // The reads into Nx complete before this straight-line block ends: the compiler takes the
        // asm outputs for ready values, so they must be, wherever it may place a register copy.
        MI_WAIT_LGKM(0);
        MI_SCHED_FENCE();
    };

    // waits until at most `stages` of this wavefront's stage fills are still in flight
    auto wait_fills = [&](int stages) {
        bool done = false;
        #pragma unroll
        for (int d = kStages - 2; d >= 1; --d) {
            if (!done && stages >= d) {
                MI_WAIT_VM(d * kLoads);
                done = true;
            }
        }
        if (!done) MI_WAIT_VM(0);
    };

    // this block's K-stages: [k_first, k_first + nk) of the K / 64 stages
    const int k_first = static_cast<int>(static_cast<long>(K / 64) * split / splits);
    const int nk = static_cast<int>(static_cast<long>(K / 64) * (split + 1) / splits) - k_first;
    Xb += static_cast<size_t>(k_first) * 128;
    W += static_cast<size_t>(k_first) * kWRow;
    Sb += static_cast<size_t>(k_first) * 4;
    Frags<TM> FA, FB;
    #pragma unroll
    for (int st = 0; st < kStages - 1; ++st)
        if (st < nk) fill_stage(st, st);
    wait_fills((nk < kStages - 1 ? nk : kStages - 1) - 1);          // stage 0 has landed
    __builtin_amdgcn_s_barrier();
    MI_SCHED_FENCE();
    static_for<kReads>([&](auto jc) { read_one(FA, 0u, std::integral_constant<int, 0>{}, jc); });
    if constexpr (Q4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(FA.w4[0]), "+v"(FA.w4[1]), "+v"(FA.ws[0]), "+v"(FA.ws[1]) : : "memory");
    else if constexpr (F16)
        MI_WAIT_LGKM(0);
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(FA.w[0]), "+v"(FA.w[1]) : : "memory");
    MI_SCHED_FENCE();
    static_for<kConv>([&](auto jc) { convert_one(FA, std::integral_constant<int, 0>{}, jc); });

    // Stage i lives in slot i % kStages.  In the middle of stage i every wavefront waits for its
    // own fills of stage i + 1 and meets the others at the barrier; behind it stage i + 1 is
    // complete and stage i - 1 is no longer read, so its slot takes stage i + kStages - 1.
    auto stage = [&](int i, int slot, auto fillc) {
        const int next = slot + 1 == kStages ? 0 : slot + 1;
        const int prev = slot == 0 ? kStages - 1 : slot - 1;
        half_stage(FA, FB, static_cast<uint32_t>(slot) * kStage, std::integral_constant<int, 1>{},
                   std::false_type{}, 0, 0);
        MI_SCHED_FENCE();
        const int last = i + kStages - 2 < nk - 1 ? i + kStages - 2 : nk - 1;   // newest stage requested so far
        wait_fills(last - (i + 1));
        __builtin_amdgcn_s_barrier();
        MI_SCHED_FENCE();
        // (after the last stage the fragments read here are not used)
        half_stage(FB, FA, static_cast<uint32_t>(next) * kStage, std::integral_constant<int, 0>{},
                   fillc, i + kStages - 1, prev);
        MI_SCHED_FENCE();
    };
    int slot = 0, i = 0;
    for (; i + kStages - 1 < nk; ++i) {
        stage(i, slot, std::true_type{});
        slot = slot + 1 == kStages ? 0 : slot + 1;
    }
    for (; i < nk; ++i) {
        stage(i, slot, std::false_type{});
        slot = slot + 1 == kStages ? 0 : slot + 1;
    }

    // --- epilogue ----------------------------------------------------------------------------------
    // D[i][j]: i = 8 (r / 4) + 4 (lane / 32) + r % 4 is a row of W (an output column), j = lane % 32
    // a row of x (an output row): a lane holds 4 consecutive output columns per r / 4.  The
    // scaled fp16 values go through LDS (rows of 64 columns, padded to 144 bytes) so that the
    // stores to out are 16 bytes per lane and 128 consecutive bytes per 8 lanes.
    if (partial) {
        // slice of K: the raw fp32 sums, 16 bytes per lane, into partial[split][M][N]
        float* pout = partial + static_cast<size_t>(split) * M * N;
        const bool vec4 = (N % 4) == 0;
        #pragma unroll
        for (int u = 0; u < 2; ++u) {
            #pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                const int nq = n0 + 64 * w + 32 * u + 8 * rq + 4 * g;
                #pragma unroll
                for (int t = 0; t < TM; ++t) {
                    const int m = m0 + 32 * t + li;
                    if (m >= M) continue;
                    float* dst = pout + static_cast<size_t>(m) * N + nq;
                    if (vec4 && nq + 3 < N) {
                        *reinterpret_cast<float4*>(dst) = float4{acc[u][t][4 * rq], acc[u][t][4 * rq + 1],
                                                                 acc[u][t][4 * rq + 2], acc[u][t][4 * rq + 3]};
                    } else {
                        #pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (nq + e < N) dst[e] = acc[u][t][4 * rq + e];
                    }
                }
            }
        }
        return;
    }
    MI_WAIT_LGKM(0);
    __builtin_amdgcn_s_barrier();                        // nobody reads operands from LDS any more
    MI_SCHED_FENCE();
    constexpr int kERow = 144;
    uint8_t* ebase = lds + w * (BM * kERow);
    #pragma unroll
    for (int u = 0; u < 2; ++u) {
        #pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            float s4[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if constexpr (!Q4 && !F16) {
                s4[0] = __half2float(__ushort_as_half(static_cast<uint16_t>(sc[u][rq].x & 0xFFFFu)));
                s4[1] = __half2float(__ushort_as_half(static_cast<uint16_t>(sc[u][rq].x >> 16)));
                s4[2] = __half2float(__ushort_as_half(static_cast<uint16_t>(sc[u][rq].y & 0xFFFFu)));
                s4[3] = __half2float(__ushort_as_half(static_cast<uint16_t>(sc[u][rq].y >> 16)));
            }
            #pragma unroll
            for (int t = 0; t < TM; ++t) {
                const uint32_t lo = pack_half2(acc[u][t][4 * rq] * s4[0], acc[u][t][4 * rq + 1] * s4[1]);
                const uint32_t hi = pack_half2(acc[u][t][4 * rq + 2] * s4[2], acc[u][t][4 * rq + 3] * s4[3]);
                *reinterpret_cast<uint2*>(ebase + (32 * t + li) * kERow + (32 * u + 8 * rq + 4 * g) * 2) = uint2{lo, hi};
            }
        }
    }
    // each wavefront reads back only what it wrote itself
    const int ncol = n0 + 64 * w + 8 * (lane & 7);       // first of this lane's 8 output columns
    const bool cols8 = (N % 8) == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    #pragma unroll
    for (int j = 0; j < BM / 8; ++j) {
        const int row = 8 * j + (lane >> 3);
        const u32x4 v = *reinterpret_cast<const u32x4*>(ebase + row * kERow + (lane & 7) * 16);
        const int m = m0 + row;
        if (m >= M) continue;
        uint16_t* dst = out + static_cast<size_t>(m) * N + ncol;
        if (cols8 && ncol + 7 < N) {
            // streaming store: all blocks of a round write their tiles at about the same time, 20 MB at
            // M = 2048, N = 4864, and nothing reads them back soon (measured: 25.8 -> 24.2 us there)
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        } else {
            #pragma unroll
            for (int e = 0; e < 8; ++e)
                if (ncol + e < N) dst[e] = static_cast<uint16_t>(v[e / 2] >> (16 * (e % 2)));
        }
    }
}

// out[m][n] = fp16((sum over slices of partial[slice][m][n]) * scale[n]) (no factor when scale is
// null); slices are added in index order, so the result does not depend on how the blocks were
// scheduled.
__global__ __launch_bounds__(256) void reduce_partials(const float* __restrict__ partial, int splits,
                                                       const uint16_t* __restrict__ scale,
                                                       uint16_t* __restrict__ out, long MN, int N) {
    const long i4 = (static_cast<long>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i4 >= MN) return;
    const bool vec = (N % 4) == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0;
    if (vec) {
        // eight, four, two slices are requested at a time and then added in index order: a few trips
        // to memory instead of one per slice (16 slices of 64 x 896: 5.4 -> 3.5 us)
        float4 a = *reinterpret_cast<const float4*>(partial + i4);
        int z = 1;
        auto add_batch = [&](auto nc) {
            constexpr int n = decltype(nc)::value;
            float4 b[n];
            #pragma unroll
            for (int u = 0; u < n; ++u) b[u] = *reinterpret_cast<const float4*>(partial + (z + u) * MN + i4);
            #pragma unroll
            for (int u = 0; u < n; ++u) { a.x += b[u].x; a.y += b[u].y; a.z += b[u].z; a.w += b[u].w; }
            z += n;
        };
        while (splits - z >= 8) add_batch(std::integral_constant<int, 8>{});
        if (splits - z >= 4) add_batch(std::integral_constant<int, 4>{});
        if (splits - z >= 2) add_batch(std::integral_constant<int, 2>{});
        if (splits - z >= 1) add_batch(std::integral_constant<int, 1>{});
        const int n = static_cast<int>(i4 % N);
        float s0 = 1.0f, s1 = 1.0f, s2 = 1.0f, s3 = 1.0f;
        if (scale) {
            s0 = __half2float(__ushort_as_half(scale[n])), s1 = __half2float(__ushort_as_half(scale[n + 1]));
            s2 = __half2float(__ushort_as_half(scale[n + 2])), s3 = __half2float(__ushort_as_half(scale[n + 3]));
        }
        __builtin_nontemporal_store(u32x2{pack_half2(a.x * s0, a.y * s1), pack_half2(a.z * s2, a.w * s3)},
                                    reinterpret_cast<u32x2*>(out + i4));
    } else {
        for (int e = 0; e < 4 && i4 + e < MN; ++e) {
            float a = partial[i4 + e];
            for (int z = 1; z < splits; ++z) a += partial[z * MN + i4 + e];
            out[i4 + e] = to_half_bits(scale ? a * __half2float(__ushort_as_half(scale[(i4 + e) % N])) : a);
        }
    }
}

template <int TM, int KIND, int TERMS>
bool launch(hipStream_t s, int M, int N, int K, const void* x, const void* W, const void* scale, void* out,
            float* partial, size_t partial_bytes, int splits) {
    // the kernel writes splits x M x N fp32 partial sums and gives every slice at least two K-stages
    if (splits < 1 || (splits > 1 && (!partial || K / 64 < 2 * splits ||
                                      static_cast<double>(splits) * M * N * 4 > static_cast<double>(partial_bytes)))) {
        MI_ERROR_FMT("gemm: %d slices of K do not fit (M=%d N=%d K=%d, %zu bytes of workspace)", splits, M, N, K,
                     partial_bytes);
        return false;
    }
    constexpr size_t lds_bytes = static_cast<size_t>(stages_for(KIND, TM)) * (32 * TM * 128 + w_stage_bytes(KIND));
    auto* kern = gemm_wide<TM, KIND, TERMS>;
    if (lds_bytes > 65536 &&
        !MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))))
        return false;
    const long total = static_cast<long>((N + kBN - 1) / kBN) * ((M + 32 * TM - 1) / (32 * TM)) * splits;
    const dim3 grid(static_cast<unsigned>(8 * ((total + 7) / 8)), 1, 1);      // see the block -> tile map in the kernel
    hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, s, static_cast<const uint16_t*>(x),
                       static_cast<const uint8_t*>(W), static_cast<const uint16_t*>(scale),
                       static_cast<uint16_t*>(out), M, N, K, splits > 1 ? partial : nullptr, splits);
    if (!MI_HIP_OK(hipGetLastError())) return false;
    if (splits > 1) {
        const long MN = static_cast<long>(M) * N;
        hipLaunchKernelGGL(reduce_partials, dim3(static_cast<unsigned>((MN / 4 + 256) / 256)), dim3(256), 0, s,
                           partial, splits, KIND == WK_I8 ? static_cast<const uint16_t*>(scale) : nullptr,
                           static_cast<uint16_t*>(out), MN, N);
        if (!MI_HIP_OK(hipGetLastError())) return false;
    }
    return true;
}

// Estimated time (us) of the wide kernel with 32 * tm rows of x per block and K cut into
// `splits` slices.  Fitted to measurements on MI355X: a block takes about 2.6 + 0.5 tm us of
// prologue and epilogue plus, per K-stage of 64, 0.27 + 0.10 tm us for int8 weights, 0.56 + 0.10 tm
// for Q4 weights rounded to fp16 once and 0.49 + 0.22 tm for Q4 weights in two terms; a fully
// occupied chip runs the same cycles about 1.56 times slower (clock under load, shared L2 and
// fabric) than a nearly empty one.  Slices cost a second launch and the partial sums' trip
// through memory.
inline double estimate_us(int kind, int terms, int tm, int splits, int M, int N, int K, int cus) {
    const long blocks = static_cast<long>((M + 32 * tm - 1) / (32 * tm)) * ((N + kBN - 1) / kBN) * splits;
    const int stages = (K / 64 + splits - 1) / splits;
    const double stage_us = kind == WK_Q4 ? (terms == 2 ? 0.49 + 0.22 * tm : 0.56 + 0.10 * tm)
                          : kind == WK_F16 ? 0.35 + 0.10 * tm : 0.27 + 0.10 * tm;
    // two blocks on one CU take about 1.4 times as long each as one alone (the dispatcher puts a
    // second block on a CU only when every CU has one)
    const int per_cu = blocks > cus ? blocks_per_cu(kind, tm) : 1;
    const double block_us = (2.6 + 0.5 * tm + stages * stage_us) * (per_cu == 2 ? 1.4 : 1.0);
    const long slots = static_cast<long>(cus) * per_cu;
    const long full = (blocks - 1) / slots, rem = blocks - full * slots;     // the last round, full or not, is `rem`
    // (64-row tiles of int8 / fp16 weights, unsliced, on more than half of the CUs and at most one per CU,
    //  run nearly as on an empty chip: 512 x 4864 x 896 in 11.2 us where the general factor says 13.6 and the
    //  64 x 64 tiles, estimated at 13.5, take 13.2; 2048 x 1152 x 896 13.2 against 15.9, 512 x 4608 x 1024 12.1
    //  against 14.5, 4096 x 576 x 1536 18.9 against 33.5.  With fewer blocks the long serial K of such
    //  shapes decides and the general factor holds: 2048 x 896 x 4864 unsliced 47 against 37 us in two slices.
    //  32-row tiles likewise at a K of 1280 to 3072, where the 64 x 64 tiles slow down as soon as a CU holds
    //  two of them: 1536 x 576 x 1536 19.2 -> 14.6 us, 1024 x 2048 x 2048 23.2 -> 18.4, 192 x 8192 x 2048 21.6 ->
    //  17.3, fp16 1536 x 1024 x 2560 29.6 -> 22.7, and from K = 1024 on (2048 x 1024 x 1024: 12.2 against 14.5 us);
    //  at a shorter K the 64 x 64 tiles stay ahead (1536 x 1152 x 896 10.2 against 11.2), at a longer one
    //  slices do (1536 x 896 x 4864 32.6 against 37.7).
    //  Q4 weights in two terms behave the same there (1024 x 2048 x 2048 in 32-row tiles 29.1 us against 34.0
    //  in two slices, 256 x 8192 x 2048 29.2 against 35.0, 2048 x 576 x 1536 21.7 against 24.2), and their tall
    //  tiles, one block per CU and twice the matrix work per byte, lose less to a full chip than the general
    //  factors say: 2048 x 4864 x 896 in 160-row tiles 34.8 us (a block alone: 27.4), 4096 x 8192 x 2048 in
    //  128-row tiles 231 us for four rounds of 48.4, against 258 us for the 64-row tiles the factors preferred.)
    const bool roomy = splits == 1 && blocks > cus / 2 && blocks <= cus &&
                       (tm == 2 || (tm == 1 && stages >= 16 && stages <= 48));
    const bool q4_tall = kind == WK_Q4 && terms == 2 && tm >= 3 && splits == 1;
    const double crowd = roomy ? 0.2 : q4_tall ? 0.3 : 0.56;
    const double round = q4_tall ? 1.25 : 1.56;
    double t = full * round * block_us + (rem ? (1.0 + crowd * rem / slots) * block_us : 0.0);
    // every row of tiles streams W again: not faster than that many bytes at about 6.8 TB/s, or,
    // for a W that stays in the memory-side cache (40 MB taken as the limit: fp16 8192 x 2048, 33.5 MB, still
    // runs eight rows of tiles in 25.9 us, and the choices at 50 MB and more are right as they are), 2.2 times that for
    // the reads after the first
    const double w_once = static_cast<double>(N) * K * (kind == WK_F16 ? 2.0 : kind == WK_I8 ? 1.0 : 0.5625);
    const int tiles_m = (M + 32 * tm - 1) / (32 * tm);
    const double w_bytes = w_once <= 40.0e6 ? w_once * (1.0 + (tiles_m - 1) / 2.2) : w_once * tiles_m;
    if (t < 2.5 + w_bytes / 6.8e6) t = 2.5 + w_bytes / 6.8e6;
    if (splits > 1) t += 2.5 + 2.0 * splits * M * static_cast<double>(N) * 4 / 4.0e6;   // ~4 TB/s there and back
    return t;
}

// Rows of x per block (in units of 32) and slices of K with the smallest estimated time; slices
// only as far as their fp32 partial sums fit the workspace.
inline void pick_shape(int kind, int terms, int M, int N, int K, int cus, size_t workspace_bytes, int* tm_out,
                       int* splits_out, double* best_us) {
    static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24};
    double best_t = 1e30;
    for (int tm = 1; tm <= 5; ++tm) {
        if (32 * (tm - 1) >= M) break;                   // no tile taller than x needs (16 x 49 152 x 576: 7.8 against 8.7 us)
        for (int sp : kSplits) {
            if (sp > 1 && (K / 64 < 2 * sp || static_cast<double>(sp) * M * N * 4 > static_cast<double>(workspace_bytes)))
                continue;
            const double t = estimate_us(kind, terms, tm, sp, M, N, K, cus);
            if (t < best_t) { best_t = t; *tm_out = tm; *splits_out = sp; }
        }
    }
    if (best_us) *best_us = best_t;
}

template <int KIND, int TERMS>
bool launch_any(int tm, hipStream_t s, int M, int N, int K, const void* x, const void* W,
                const void* scale, void* out, float* partial, size_t partial_bytes, int splits) {
    switch (tm) {
        case 1: return launch<1, KIND, TERMS>(s, M, N, K, x, W, scale, out, partial, partial_bytes, splits);
        case 2: return launch<2, KIND, TERMS>(s, M, N, K, x, W, scale, out, partial, partial_bytes, splits);
        case 3: return launch<3, KIND, TERMS>(s, M, N, K, x, W, scale, out, partial, partial_bytes, splits);
        case 4: return launch<4, KIND, TERMS>(s, M, N, K, x, W, scale, out, partial, partial_bytes, splits);
        default: return launch<5, KIND, TERMS>(s, M, N, K, x, W, scale, out, partial, partial_bytes, splits);
    }
}

}  // namespace wide

// ---- 256 x 256 blocks, 128 x 128 per wavefront (int8 weights) --------------------------------------
//
// The wide kernel above gives a wavefront 64 rows of W against up to 160 rows of x: per MFMA it reads
// (2 + 2 TM) / (4 TM) fragments from LDS, and at 160 rows that traffic (133 KB per stage of K = 64) takes
// the LDS four fifths as long as the MFMAs take the matrix cores, overlapped by less than half.  Here the
// four wavefronts sit two along x by two along W and each owns 128 x 128 of the block's 256 x 256 outputs:
// sixteen 32 x 32 accumulators (all 256 AGPRs), four fragments of W and four of x per 16 MFMAs, 37 % less
// LDS read traffic and 19 % less fill traffic per MFMA.  Same LDS layout, swizzles, K permutation, fills
// and barrier scheme as the wide kernel; three stages of 48 KB.  It needs whole rounds of 256-row tiles to
// pay: a few hundred tiles at least, and a long K (each block's prologue and epilogue stand alone on its CU).
namespace quad {

constexpr int kBM = 256, kBN = 256, kStages = 3;
constexpr int kXStage = kBM * 128, kWStage = kBN * 64, kStage = kXStage + kWStage;
constexpr int kXLoads = 8, kWLoads = 4, kLoads = kXLoads + kWLoads;   // 1 KB loads per wavefront and stage
constexpr int kReads = 12, kConv = 16, kMfmas = 32;                   // per half stage (K = 32)
constexpr int kERow = 272;                                            // epilogue: 128 columns of fp16 + 16 bytes

struct Frags {
    u32x4 w[4];                // 16 int8 weights of four 32-row fragments of W
    uint32_t wf[4][2][4];      // the same as fp16: [fragment][MFMA of the pair][4 dwords = 8 halves]
    u32x4 x[2][4];             // [MFMA of the pair][32-row fragment of x]
};

using wide::lds_fill16;
using wide::static_for;
using wide::pack_half2;

__global__ __launch_bounds__(256) void gemm_quad(const uint16_t* __restrict__ X, const uint8_t* __restrict__ W,
                                                 const uint16_t* __restrict__ scale, uint16_t* __restrict__ out,
                                                 int M, int N, int K) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = w >> 1, wc = w & 1;                  // this wavefront's 128 rows of x, 128 rows of W
    const int g = lane >> 5, li = lane & 31;
    // block -> tile: as in the wide kernel (an XCD takes a contiguous eighth of the list, bands of 4 tiles along N)
    int tile_m, tile_n;
    {
        const int tiles_m = (M + kBM - 1) / kBM, tiles_n = (N + kBN - 1) / kBN, total = tiles_m * tiles_n;
        const int per_xcd = (total + 7) / 8;
        const int l = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (blockIdx.x >= 8 * per_xcd || l >= total) return;          // whole block, before any barrier
        constexpr int kBand = 4;
        const int band = l / (kBand * tiles_m);
        const int width = tiles_n - band * kBand < kBand ? tiles_n - band * kBand : kBand;
        const int in_band = l - band * kBand * tiles_m;
        tile_m = in_band / width;
        tile_n = band * kBand + in_band % width;
    }
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;
    const uint32_t lbase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((wide::lds_u8*)lds));

    // fill side: x load j covers rows 8 (w + 4 j) .. + 7 of the tile (128 bytes each, chunk p of row r in slot
    // p ^ ((r >> 1) & 7)); W load j rows 16 (4 w + j) .. + 15 (64 bytes each, slot p ^ ((r >> 2) & 3))
    uint32_t xsrc[kXLoads], wsrc[kWLoads];
    #pragma unroll
    for (int j = 0; j < kXLoads; ++j) {
        const int r = 8 * (w + 4 * j) + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        const int m = m0 + r < M ? m0 + r : M - 1;
        xsrc[j] = static_cast<uint32_t>(m) * K * 2u + c * 16u;
    }
    #pragma unroll
    for (int j = 0; j < kWLoads; ++j) {
        const int r = 16 * (4 * w + j) + (lane >> 2);
        const int c = (lane & 3) ^ ((r >> 2) & 3);
        const int n = n0 + r < N ? n0 + r : N - 1;
        wsrc[j] = static_cast<uint32_t>(n) * K + c * 16u;
    }
    const uint8_t* Xb = reinterpret_cast<const uint8_t*>(X);
    auto fill_one = [&](int stage_k, int slot, auto jc) {
        constexpr int j = decltype(jc)::value;
        uint8_t* xs = lds + slot * kStage;
        if constexpr (j < kXLoads)
            lds_fill16(Xb + static_cast<size_t>(stage_k) * 128 + xsrc[j], xs + 1024 * (w + 4 * j));
        else
            lds_fill16(W + static_cast<size_t>(stage_k) * 64 + wsrc[j - kXLoads], xs + kXStage + 1024 * (4 * w + (j - kXLoads)));
    };
    auto fill_stage = [&](int stage_k, int slot) {
        static_for<kLoads>([&](auto jc) { fill_one(stage_k, slot, jc); });
    };

    // read side: pair S of a stage, MFMA e of the pair: x chunk 4 S + 2 g + e, W chunk 2 S + g
    const uint32_t xrow = lbase + (128u * wr + li) * 128u, xq = (2u * g) ^ ((li >> 1) & 7u);
    const uint32_t wrow = lbase + kXStage + (128u * wc + li) * 64u, wq = g ^ ((li >> 2) & 3u);
    uint32_t xoff[2][2], woff[2];
    #pragma unroll
    for (int S = 0; S < 2; ++S) {
        #pragma unroll
        for (int e = 0; e < 2; ++e) xoff[S][e] = xrow + (((4u * S + e) ^ xq) << 4);
        woff[S] = wrow + (((2u * S) ^ wq) << 4);
    }
    // read j of a set: the four W fragments first, then x for the first and the second MFMA of the pair
    auto read_one = [&](Frags& F, uint32_t slot_bytes, auto Sc, auto jc) {
        constexpr int S = decltype(Sc)::value, j = decltype(jc)::value;
        if constexpr (j < 4) {
            const uint32_t a = woff[S] + slot_bytes;
            MI_LDS_READ16(F.w[j], a, j * 32 * 64);
        } else {
            constexpr int e = (j - 4) / 4, t = (j - 4) % 4;
            const uint32_t a = xoff[S][e] + slot_bytes;
            MI_LDS_READ16(F.x[e][t], a, t * 4096);
        }
    };
    auto convert_one = [&](Frags& F, auto jc) {
        constexpr int j = decltype(jc)::value, u = j / 4, d = j % 4;
        i8x4_to_h4(F.w[u][d], F.wf[u][d / 2][2 * (d % 2)], F.wf[u][d / 2][2 * (d % 2) + 1]);
    };

    floatx16 acc[4][4];
    #pragma unroll
    for (int u = 0; u < 4; ++u)
        #pragma unroll
        for (int t = 0; t < 4; ++t)
            #pragma unroll
            for (int r = 0; r < 16; ++r) acc[u][t][r] = 0.0f;

    auto mfma_one = [&](const Frags& F, auto nc) {
        constexpr int n = decltype(nc)::value, e = n / 16, u = (n / 4) % 4, t = n % 4;
        const u32x4 wv = u32x4{F.wf[u][e][0], F.wf[u][e][1], F.wf[u][e][2], F.wf[u][e][3]};
        acc[u][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, wv),
                                                          __builtin_bit_cast(half8, F.x[e][t]), acc[u][t], 0, 0, 0);
    };

    // one half stage: the fills of a later stage, the reads and conversions of the next fragments, dealt out
    // between the MFMAs of the current ones
    auto half_stage = [&](Frags& C, Frags& Nx, uint32_t next_bytes, auto NSc, auto fillc, int fill_k, int fill_slot) {
        constexpr bool FILL = decltype(fillc)::value;
        constexpr int nF = FILL ? kLoads : 0;
        constexpr int A = nF + kReads + 1 + kConv;
        static_for<kMfmas>([&](auto nc) {
            constexpr int n = decltype(nc)::value;
            mfma_one(C, nc);
            MI_SCHED_FENCE();
            constexpr int a0 = n * A / kMfmas, a1 = (n + 1) * A / kMfmas;
            static_for<a1 - a0>([&](auto kc) {
                constexpr int a = a0 + decltype(kc)::value;
                if constexpr (a < nF) {
                    fill_one(fill_k, fill_slot, std::integral_constant<int, a>{});
                } else if constexpr (a < nF + kReads) {
                    read_one(Nx, next_bytes, NSc, std::integral_constant<int, a - nF>{});
                } else if constexpr (a == nF + kReads) {
                    // LDS returns in order: with the eight x reads outstanding, the four W reads are back
                    asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(Nx.w[0]), "+v"(Nx.w[1]), "+v"(Nx.w[2]), "+v"(Nx.w[3]) : : "memory");
                    MI_SCHED_FENCE();
                } else {
                    convert_one(Nx, std::integral_constant<int, a - nF - kReads - 1>{});
                }
            });
            MI_SCHED_FENCE();
        });
        MI_WAIT_LGKM(0);
        MI_SCHED_FENCE();
    };
    // at most `stages` (0 or 1) of this wavefront's stage fills still in flight
    auto wait_fills = [&](int stages) {
        if (stages >= 1) MI_WAIT_VM(kLoads); else MI_WAIT_VM(0);
    };

    const int nk = K / 64;
    Frags FA, FB;
    #pragma unroll
    for (int st = 0; st < kStages - 1; ++st)
        if (st < nk) fill_stage(st, st);
    wait_fills((nk < kStages - 1 ? nk : kStages - 1) - 1);          // stage 0 has landed
    __builtin_amdgcn_s_barrier();
    MI_SCHED_FENCE();
    static_for<kReads>([&](auto jc) { read_one(FA, 0u, std::integral_constant<int, 0>{}, jc); });
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(FA.w[0]), "+v"(FA.w[1]), "+v"(FA.w[2]), "+v"(FA.w[3]) : : "memory");
    MI_SCHED_FENCE();
    static_for<kConv>([&](auto jc) { convert_one(FA, jc); });

    auto stage = [&](int i, int slot, auto fillc) {
        const int next = slot + 1 == kStages ? 0 : slot + 1;
        const int prev = slot == 0 ? kStages - 1 : slot - 1;
        half_stage(FA, FB, static_cast<uint32_t>(slot) * kStage, std::integral_constant<int, 1>{}, std::false_type{}, 0, 0);
        MI_SCHED_FENCE();
        const int last = i + kStages - 2 < nk - 1 ? i + kStages - 2 : nk - 1;   // newest stage requested so far
        wait_fills(last - (i + 1));
        __builtin_amdgcn_s_barrier();
        MI_SCHED_FENCE();
        half_stage(FB, FA, static_cast<uint32_t>(next) * kStage, std::integral_constant<int, 0>{}, fillc, i + kStages - 1, prev);
        MI_SCHED_FENCE();
    };
    int slot = 0, i = 0;
    for (; i + kStages - 1 < nk; ++i) {
        stage(i, slot, std::true_type{});
        slot = slot + 1 == kStages ? 0 : slot + 1;
    }
    for (; i < nk; ++i) {
        stage(i, slot, std::false_type{});
        slot = slot + 1 == kStages ? 0 : slot + 1;
    }

    // epilogue: D[i][j], i = 8 (r / 4) + 4 g + r % 4 a row of W (an output column), j = li a row of x.  The scaled
    // fp16 values go through LDS (this wavefront's own 128 x 128 patch, rows padded to 272 bytes) so that the
    // stores are 16 bytes per lane, 256 consecutive bytes per 16 lanes.
    MI_WAIT_LGKM(0);
    __builtin_amdgcn_s_barrier();                        // nobody reads operands from LDS any more
    MI_SCHED_FENCE();
    uint8_t* ebase = lds + w * (128 * kERow);
    const bool cols4 = (N % 4) == 0 && reinterpret_cast<uintptr_t>(scale) % 8 == 0;
    #pragma unroll
    for (int u = 0; u < 4; ++u) {
        #pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            const int nq = n0 + 128 * wc + 32 * u + 8 * rq + 4 * g;
            uint32_t h[4];
            if (cols4 && nq + 3 < N) {
                const uint2 v = *reinterpret_cast<const uint2*>(scale + nq);
                h[0] = v.x & 0xFFFFu; h[1] = v.x >> 16; h[2] = v.y & 0xFFFFu; h[3] = v.y >> 16;
            } else {
                #pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = scale[nq + e < N ? nq + e : N - 1];
            }
            float s4[4];
            #pragma unroll
            for (int e = 0; e < 4; ++e) s4[e] = __half2float(__ushort_as_half(static_cast<uint16_t>(h[e])));
            #pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t lo = pack_half2(acc[u][t][4 * rq] * s4[0], acc[u][t][4 * rq + 1] * s4[1]);
                const uint32_t hi = pack_half2(acc[u][t][4 * rq + 2] * s4[2], acc[u][t][4 * rq + 3] * s4[3]);
                *reinterpret_cast<uint2*>(ebase + (32 * t + li) * kERow + (32 * u + 8 * rq + 4 * g) * 2) = uint2{lo, hi};
            }
        }
    }
    // each wavefront reads back only what it wrote itself
    const int ncol = n0 + 128 * wc + 8 * (lane & 15);    // first of this lane's 8 output columns
    const bool cols8 = (N % 8) == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    #pragma unroll 4
    for (int j = 0; j < 32; ++j) {
        const int row = 4 * j + (lane >> 4);
        const u32x4 v = *reinterpret_cast<const u32x4*>(ebase + row * kERow + (lane & 15) * 16);
        const int m = m0 + 128 * wr + row;
        if (m >= M) continue;
        uint16_t* dst = out + static_cast<size_t>(m) * N + ncol;
        if (cols8 && ncol + 7 < N) {
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        } else {
            #pragma unroll
            for (int e = 0; e < 8; ++e)
                if (ncol + e < N) dst[e] = static_cast<uint16_t>(v[e / 2] >> (16 * (e % 2)));
        }
    }
}

bool launch(hipStream_t s, int M, int N, int K, const void* x, const void* W, const void* scale, void* out) {
    constexpr size_t lds_bytes = static_cast<size_t>(kStages) * kStage;
    static_assert(4 * 128 * kERow <= kStages * kStage, "the epilogue's patches fit the operand stages");
    if (!MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_quad),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))))
        return false;
    const long total = static_cast<long>((N + kBN - 1) / kBN) * ((M + kBM - 1) / kBM);
    hipLaunchKernelGGL(gemm_quad, dim3(static_cast<unsigned>(8 * ((total + 7) / 8))), dim3(256), lds_bytes, s,
                       static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(W),
                       static_cast<const uint16_t*>(scale), static_cast<uint16_t*>(out), M, N, K);
    return MI_HIP_OK(hipGetLastError());
}

}  // namespace quad

// ---- a few rows of x (M <= 64): the weights stream once, as in the GEMV ------------------------
//
// With up to 64 rows of x the contraction is bound by the weights' bytes, like the GEMV, not by
// the matrix cores, and the tiles above leave most of the chip idle (19 tiles at N = 4864).  Here a
// wavefront takes a strip of 16 rows of W and streams it through v_mfma_f32_16x16x32_f16 against
// the 16 MT rows of x:
//   A = W strip: lane l supplies row l % 16, 8 values of K starting at 16 (l / 16) + 8 s of the
//       iteration's 64 (s = 0, 1: the two MFMAs of an iteration), i.e. one 16-byte load of int8
//       weights per lane and iteration, 64 contiguous bytes per row;
//   B = x^T: lane l supplies row l % 16 of the x tile at the same 16 values of K, 32 contiguous
//       bytes (x is small and comes from the caches);
//   D[i][j] (lane l: i = 4 (l / 16) + r, j = l % 16) = out[row j of the x tile][row i of the strip]:
//       four consecutive output columns per lane.
// K is cut into ks slices over the wavefronts of a block where N alone gives too few strips to
// fill the chip; their sums meet in LDS and are added in slice order.  Iterations go through two
// register buffers, one in flight while the other is multiplied.
namespace skinny {

typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int kMaxM = 64;
constexpr int kWaves = 8;                // wavefronts per block

// SW strips of W per wavefront: the fragments of x a lane holds are multiplied with SW strips.
// XL: the block first copies its rows of x into LDS (rows padded by 16 bytes, which spreads the 16
// rows a 16-byte read touches over all banks) and every wavefront reads its fragments from there;
// blocks then live long and walk over the strips.  Without XL (x too large for LDS) the fragments
// come from the caches with the weights, 2 MT / SW bytes per byte of W, and the L1's few requests
// in flight bound the rate: that form only pays for a few rows of x at a long K.
// Q4 weights: an iteration is 128 values of K, of which a lane holds 32, exactly one scale block (16
// bytes of nibbles and one scale per lane and iteration); the weights enter the matrix cores as
// q * scale, exactly, in TERMS = 2 fp16 terms (scale = hi + lo with 7 and 4 significant bits, as in
// the wide kernel), or rounded to fp16 once with TERMS = 1.
template <int KIND, int MT, int SW, bool XL, int TERMS>
__global__ __launch_bounds__(64 * kWaves) void gemm_skinny(const uint16_t* __restrict__ X,
                                                           const uint8_t* __restrict__ W,
                                                           const uint16_t* __restrict__ scale,
                                                           uint16_t* __restrict__ out, int M, int N, int K, int ks,
                                                           int logical_blocks, float* __restrict__ partial) {
    constexpr bool F16 = KIND == WK_F16, Q4 = KIND == WK_Q4;
    constexpr int WV = F16 ? 2 : 1;                       // 16-byte loads of W per lane, strip and iteration
    constexpr int kWB = F16 ? 2 : 1;                      // bytes of a row of W per 64 bytes of an iteration's weights / 64
    constexpr int kItK = Q4 ? 128 : 64;                   // values of K per iteration
    constexpr int XE = kItK / 32;                         // 16-byte pieces of x per lane and iteration = MFMAs per x tile and term
    constexpr int kPerIt = (4 * WV + (Q4 ? 1 : 0)) * SW + (XL ? 0 : 4 * XE * MT);   // registers one iteration's operands take in a buffer
    constexpr int kBudget = F16 ? 40 : 48;                // registers per buffer (with 64 the fp16 instances spill)
    constexpr int kChunk = kBudget / kPerIt < 1 ? 1 : kBudget / kPerIt > 8 ? 8 : kBudget / kPerIt;   // iterations per buffer
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t xrow = XL ? static_cast<uint32_t>(K) * 2u + 16u : 0u;              // bytes per row of x in LDS
    float* red = reinterpret_cast<float*>(lds + 16u * MT * xrow);                     // [kWaves][MT][4][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, c = lane >> 4;
    const int slice = wave % ks;
    const int nit = (K + kItK - 1) / kItK;               // (Q4 at K = 64 mod 128: the upper half of the lanes sits out the last one)
    const size_t wrowb = Q4 ? static_cast<size_t>(K) / 2 : static_cast<size_t>(K) * kWB;   // bytes of a row of W
    // K is cut over the blocks of the grid's y (then `partial` takes raw sums, one M x N matrix per y,
    // for reduce_partials) and, inside a block, over ks wavefronts
    const int b0 = nit * static_cast<int>(blockIdx.y) / static_cast<int>(gridDim.y);
    const int b1 = nit * (static_cast<int>(blockIdx.y) + 1) / static_cast<int>(gridDim.y);
    const int it0 = b0 + (b1 - b0) * slice / ks, it1 = b0 + (b1 - b0) * (slice + 1) / ks;

    if constexpr (XL) {
        // Wavefront w copies rows w, w + 8, ...: a lane requests its 16-byte piece of each of the wavefront's
        // 2 MT rows before it stores the first, so the copy is one trip to memory per 64 pieces of a row
        // (before: a trip per 512 pieces of the tile, and a division per piece; 4864 x 896 at 16 / 32 / 48
        // rows 4.65 / 5.8 / 6.8 -> 4.35 / 4.95 / 5.7 us).  Rows past M are read as the last row and never
        // stored from.  Asking for the first weights ahead of this copy was measured as well: slower
        // (4.7 / 5.4 / 6.05 us), x then arrives behind them.
        const int per_row = K / 8;                       // 16-byte pieces per row
        const uint8_t* Xb = reinterpret_cast<const uint8_t*>(X);
        for (int piece = threadIdx.x & 63; piece < per_row; piece += 64) {
            u32x4 t[2 * MT];
            #pragma unroll
            for (int rr = 0; rr < 2 * MT; ++rr) {
                const int row = wave + kWaves * rr;
                const int m = row < M ? row : M - 1;
                t[rr] = *reinterpret_cast<const u32x4*>(Xb + static_cast<size_t>(m) * K * 2 + piece * 16);
            }
            #pragma unroll
            for (int rr = 0; rr < 2 * MT; ++rr)
                *reinterpret_cast<u32x4*>(lds + (wave + kWaves * rr) * xrow + piece * 16) = t[rr];
        }
        __syncthreads();
    }
    const uint8_t* xp[MT];                               // without XL: this lane's rows of x in memory
    #pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + i < M ? 16 * t + i : M - 1;
        xp[t] = reinterpret_cast<const uint8_t*>(X) + static_cast<size_t>(m) * K * 2 + c * (16 * XE);
    }
    const uint32_t xl = (16u * 0 + i) * xrow + c * (16u * XE);  // with XL: this lane's row of the first x tile in LDS
    const bool cols4 = (N % 4) == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0;

    for (int lb = blockIdx.x; lb < logical_blocks; lb += gridDim.x) {     // (the same trips for the whole block)
        const int group = lb * (kWaves / ks) + wave / ks;                 // group: SW consecutive strips
        const uint8_t* wp[SW];
        [[maybe_unused]] const uint16_t* sp[SW];                          // Q4: the row's block scales, this lane's first
        #pragma unroll
        for (int q = 0; q < SW; ++q) {
            const int row = 16 * (group * SW + q) + i;                    // rows past N are read as the last row
            wp[q] = W + static_cast<size_t>(row < N ? row : N - 1) * wrowb + c * 16 * WV;
            if constexpr (Q4) sp[q] = scale + static_cast<size_t>(row < N ? row : N - 1) * (K / 32) + c;
        }
        floatx4 acc[SW][MT];
        #pragma unroll
        for (int q = 0; q < SW; ++q)
            #pragma unroll
            for (int t = 0; t < MT; ++t) acc[q][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

        u32x4 wb[2][kChunk][SW][WV];
        [[maybe_unused]] uint16_t sb[2][kChunk][SW];
        [[maybe_unused]] u32x4 xb[2][XL ? 1 : kChunk][XL ? 1 : MT][XE];
        // `full`: kChunk iterations whatever the slice's end (the caller knows they exist); the number
        // of requests is then a constant, and only then can the wait before a buffer is multiplied
        // leave the other buffer's requests in flight
        auto fetch = [&](auto fullc, int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int it = j0 + u;
                if constexpr (!decltype(fullc)::value) {
                    if (it >= it1) break;
                }
                // (Q4, K = 64 mod 128: a lane without weights in the last iteration asks for the start of its rows)
                [[maybe_unused]] const bool mine = !Q4 || kItK * it + 32 * c < K;
                if constexpr (!XL) {
                    #pragma unroll
                    for (int t = 0; t < MT; ++t)
                        #pragma unroll
                        for (int e = 0; e < XE; ++e)
                            xb[b][u][t][e] = reinterpret_cast<const u32x4*>(
                                xp[t] + (mine ? static_cast<ptrdiff_t>(it) * (2 * kItK) : -static_cast<ptrdiff_t>(c) * (16 * XE)))[e];
                }
                #pragma unroll
                for (int q = 0; q < SW; ++q) {
                    #pragma unroll
                    for (int v = 0; v < WV; ++v)
                        wb[b][u][q][v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                            wp[q] + (mine ? static_cast<ptrdiff_t>(it) * 64 * kWB : -static_cast<ptrdiff_t>(c) * 16 * WV)) + v);
                    if constexpr (Q4) sb[b][u][q] = sp[q][mine ? 4 * it : -c];
                }
            }
        };
        auto multiply = [&](int b, int j0) {
            #pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int it = j0 + u;
                if (it < it1) {
                    [[maybe_unused]] const bool mine = !Q4 || kItK * it + 32 * c < K;
                    half8 xf[MT][XE];
                    #pragma unroll
                    for (int t = 0; t < MT; ++t)
                        #pragma unroll
                        for (int e = 0; e < XE; ++e) {
                            if constexpr (XL)
                                xf[t][e] = *reinterpret_cast<const half8*>(
                                    lds + xl + 16u * t * xrow + (mine ? it * (2 * kItK) : -c * (16 * XE)) + 16 * e);
                            else
                                xf[t][e] = __builtin_bit_cast(half8, xb[b][u][t][e]);
                        }
                    #pragma unroll
                    for (int q = 0; q < SW; ++q) {
                        half8 a[TERMS][XE];
                        if constexpr (F16) {
                            a[0][0] = __builtin_bit_cast(half8, wb[b][u][q][0]);
                            a[0][1] = __builtin_bit_cast(half8, wb[b][u][q][1]);
                        } else if constexpr (Q4) {
                            // a lane that sits the iteration out multiplies by a scale of zero
                            const uint32_t s1 = mine ? sb[b][u][q] : 0u;
                            const uint32_t sboth = s1 | (s1 << 16);
                            __half2 st[TERMS];
                            if constexpr (TERMS == 2) {
                                st[0] = __builtin_bit_cast(__half2, sboth & 0xFFF0FFF0u);
                                st[1] = __hsub2(__builtin_bit_cast(__half2, sboth), st[0]);
                            } else {
                                st[0] = __builtin_bit_cast(__half2, sboth);
                            }
                            #pragma unroll
                            for (int e = 0; e < XE; ++e) {
                                const uint32_t v = wb[b][u][q][0][e];
                                #pragma unroll
                                for (int z = 0; z < TERMS; ++z)
                                    a[z][e] = __builtin_bit_cast(half8, u32x4{q4x2_to_h2<0>(v, st[z]), q4x2_to_h2<1>(v, st[z]),
                                                                              q4x2_to_h2<2>(v, st[z]), q4x2_to_h2<3>(v, st[z])});
                            }
                        } else {
                            uint32_t h[8];
                            i8x4_to_h4(wb[b][u][q][0].x, h[0], h[1]);
                            i8x4_to_h4(wb[b][u][q][0].y, h[2], h[3]);
                            i8x4_to_h4(wb[b][u][q][0].z, h[4], h[5]);
                            i8x4_to_h4(wb[b][u][q][0].w, h[6], h[7]);
                            a[0][0] = __builtin_bit_cast(half8, u32x4{h[0], h[1], h[2], h[3]});
                            a[0][1] = __builtin_bit_cast(half8, u32x4{h[4], h[5], h[6], h[7]});
                        }
                        #pragma unroll
                        for (int t = 0; t < MT; ++t)
                            #pragma unroll
                            for (int z = 0; z < TERMS; ++z)
                                #pragma unroll
                                for (int e = 0; e < XE; ++e)
                                    acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[z][e], xf[t][e], acc[q][t], 0, 0, 0);
                    }
                }
            }
        };
        // buffers 0 and 1 in turn while two more whole chunks lie ahead; then what is left (one
        // buffer that may be on its way already, and at most one more chunk)
        int j0 = it0, cur = 0;
        if (it1 - j0 >= 2 * kChunk) {
            fetch(std::true_type{}, 0, j0);
            while (true) {
                fetch(std::true_type{}, 1, j0 + kChunk);
                multiply(0, j0);
                j0 += kChunk;
                if (it1 - j0 < 2 * kChunk) { cur = 1; break; }
                fetch(std::true_type{}, 0, j0 + kChunk);
                multiply(1, j0);
                j0 += kChunk;
                if (it1 - j0 < 2 * kChunk) { cur = 0; break; }
            }
        } else {
            fetch(std::false_type{}, 0, j0);
        }
        if (cur == 0) {
            fetch(std::false_type{}, 1, j0 + kChunk);
            multiply(0, j0);
            multiply(1, j0 + kChunk);
        } else {
            fetch(std::false_type{}, 0, j0 + kChunk);
            multiply(1, j0);
            multiply(0, j0 + kChunk);
        }

        if (ks > 1) {                                    // (the same for every wavefront of the grid)
            #pragma unroll
            for (int q = 0; q < SW; ++q) {               // one strip at a time through the same 4 MT KB per wavefront
                __syncthreads();                         // the last round's sums have been read
                if (slice > 0) {
                    #pragma unroll
                    for (int t = 0; t < MT; ++t)
                        #pragma unroll
                        for (int r = 0; r < 4; ++r) red[((wave * MT + t) * 4 + r) * 64 + lane] = acc[q][t][r];
                }
                __syncthreads();
                if (slice == 0) {
                    for (int z = 1; z < ks; ++z) {       // slice 0 + slice 1 + ..., in this order
                        #pragma unroll
                        for (int t = 0; t < MT; ++t)
                            #pragma unroll
                            for (int r = 0; r < 4; ++r) acc[q][t][r] += red[(((wave + z) * MT + t) * 4 + r) * 64 + lane];
                    }
                }
            }
            if (slice > 0) continue;
        }

        #pragma unroll
        for (int q = 0; q < SW; ++q) {
            const int nq = 16 * (group * SW + q) + 4 * c;    // first of this lane's 4 output columns
            if (nq >= N) continue;
            float s4[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if constexpr (KIND == WK_I8) {
                #pragma unroll
                for (int r = 0; r < 4; ++r) s4[r] = __half2float(__ushort_as_half(scale[nq + r < N ? nq + r : N - 1]));
            }
            if (partial) {
                float* pout = partial + static_cast<size_t>(blockIdx.y) * M * N;
                #pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const int m = 16 * t + i;
                    if (m >= M) continue;
                    float* dst = pout + static_cast<size_t>(m) * N + nq;
                    if ((N % 4) == 0 && nq + 3 < N) {
                        *reinterpret_cast<float4*>(dst) = float4{acc[q][t][0], acc[q][t][1], acc[q][t][2], acc[q][t][3]};
                    } else {
                        #pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (nq + r < N) dst[r] = acc[q][t][r];
                    }
                }
                continue;
            }
            #pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int m = 16 * t + i;
                if (m >= M) continue;
                const uint32_t lo = wide::pack_half2(acc[q][t][0] * s4[0], acc[q][t][1] * s4[1]);
                const uint32_t hi = wide::pack_half2(acc[q][t][2] * s4[2], acc[q][t][3] * s4[3]);
                uint16_t* dst = out + static_cast<size_t>(m) * N + nq;
                if (cols4 && nq + 3 < N) {
                    *reinterpret_cast<uint2*>(dst) = uint2{lo, hi};
                } else {
                    #pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (nq + r < N) dst[r] = static_cast<uint16_t>((r / 2 ? hi : lo) >> (16 * (r % 2)));
                }
            }
        }
    }
}

constexpr size_t kLdsLimit = 160 * 1024;
// bytes of LDS a block takes: the rows of x (XL) and the buffer in which K-slices meet
inline size_t lds_bytes(int mt, int K, bool xl, int ks) {
    return (xl ? static_cast<size_t>(16) * mt * (2 * static_cast<size_t>(K) + 16) : 0) +
           (ks > 1 ? static_cast<size_t>(kWaves) * mt * 4 * 64 * 4 : 0);
}

struct Shape { int ks; bool xl; int kb; };
// Slices of K per strip inside a block (1, 2, 4, 8: the fewest that give the chip four wavefronts
// per CU; measured at 4864 x 896: 4 slices 4.5 us, 8 slices 6.7 us), x in LDS where it fits, and
// slices of K over blocks (kb) where one block per strip still leaves most CUs idle and what a
// single CU can pull bounds the launch (896 x 4864: 56 strips): their sums go through the
// workspace and a second launch adds them in order.  One strip per wavefront: two and four (the
// kernel's SW) were measured slower at every shape tried (fewer wavefronts; the reads of x they
// save are not the bound).
inline Shape pick_shape(int kind, int M, int N, int K, int cus, size_t workspace_bytes) {
    const int mt = (M + 15) / 16;
    const long strips = (N + 15) / 16;
    const int its = kind == WK_Q4 ? (K + 127) / 128 : K / 64;        // iterations over K
    Shape sh{1, false, 1};
    while (sh.ks < kWaves && strips * sh.ks < 4L * cus && its >= 2 * sh.ks) sh.ks *= 2;
    // (a block whose eight wavefronts share one strip reads every byte of x once either way: no LDS then)
    sh.xl = sh.ks < kWaves && lds_bytes(mt, K, true, sh.ks) <= kLdsLimit;
    if (sh.ks == kWaves) {
        while (sh.kb < 8 && strips * sh.kb * 2 <= cus && its >= 2 * sh.ks * sh.kb * 2 &&
               static_cast<double>(sh.kb) * 2 * M * N * 4 <= static_cast<double>(workspace_bytes))
            sh.kb *= 2;
    }
    return sh;
}

// Where the streaming kernel is the library's own choice (measured against the tiles above, warm
// weights, us).
//  - With x in LDS, or one strip per block: up to 48 rows (int8 4864 x 896: 4.4 / 5.0 / 5.7 at 16 / 32 / 48
//    rows against 6.3 to 6.5 for the 64 x 64 tiles, 6.65 against 6.5 at 64; 2560 x 1024: 4.4 / 5.4 / 6.5
//    against 8.2 to 9.1); up to 64 where K is cut over blocks as well (896 x 4864: 6.9 / 8.0 / 10.5 at 16 /
//    32 / 64 rows against 25 and more unsliced, 12 to 14 as the wide kernel was chosen in slices).
//  - x in LDS, Q4 or fp16 weights of a few MB: up to 64 rows (Q4 4864 x 896 at 64 rows 8.55 against
//    11.8 for the wide kernel, 9728 x 896 10.5 against 12.4; fp16 4864 x 896 7.5 against 8.0).
//  - x from the caches and shared by several strips per block: only up to 16 rows (8192 x 2048 at 48
//    rows: 28 us against 17).  Q4 then holds twice the x per iteration in registers: one strip per
//    block is good for 48 rows (2560 x 1024: 7.5 against 10.7, 3072 x 1024: 7.6 against 10.9), K over
//    blocks as well for 32 (896 x 4864: 10.3 / 14.0 / 26.5 at 32 / 48 / 64 rows against 12.7 to 12.9).
//  - No more than 13.5 MB of weights: beyond that the launch is long enough for the wide kernel's
//    higher streaming rate to win (a wavefront here loads a strip, waits, multiplies).  int8 14 592 x
//    896 (13.1 MB) 6.4 / 7.0 / 7.9 at 16 / 32 / 48 rows against 8.5, but 19 456 x 896 8.8 / 9.6 / 10.5 against
//    8.6 / 8.7 / 9.0, 49 152 x 576 11.2 against 7.3 and fp16 49 152 x 576 16.7 against 10.8; an lm_head of
//    151 936 rows streams at 4.0 TB/s here against 4.8 TB/s there.
inline bool preferred(int kind, int M, int N, int K, int cus, size_t workspace_bytes) {
    const Shape sh = pick_shape(kind, M, N, K, cus, workspace_bytes);
    const double w_bytes = static_cast<double>(N) * K * (kind == WK_F16 ? 2.0 : kind == WK_Q4 ? 0.5625 : 1.0);
    int rows = sh.xl || sh.ks == kWaves ? (sh.kb > 1 ? 64 : 48) : 16;
    if (kind == WK_Q4 && !sh.xl) rows = sh.ks == kWaves && sh.kb == 1 ? 48 : rows > 32 ? 32 : rows;
    if (kind == WK_F16 && rows == 48) rows = 56;         // (fp16 2560 x 1024 at 49 / 56 rows: 7.45 / 7.7 against 9.4 / 8.8 us)
    if (kind != WK_I8 && sh.xl && w_bytes <= (kind == WK_Q4 ? 6.0e6 : 9.0e6)) rows = 64;
    return M <= rows && w_bytes <= 13.5e6 && (N + 15) / 16 <= 16L * cus;
}

// Estimated time (us), fitted to the same measurements.
inline double estimate_us(int kind, int M, int N, int K, int cus, size_t workspace_bytes) {
    const Shape sh = pick_shape(kind, M, N, K, cus, workspace_bytes);
    const double w_bytes = static_cast<double>(N) * K * (kind == WK_F16 ? 2.0 : kind == WK_Q4 ? 0.5625 : 1.0);
    // (Q4 weights: the two-term feed costs 0.6 us more, 1.1 with K over blocks)
    const double q4_us = kind == WK_Q4 ? (sh.kb > 1 ? 1.1 : 0.6) : 0.0;
    // (x from the caches: 0.07 us per row where several strips of a block read it, 0.03 where the block's
    //  eight wavefronts share one strip, 0.06 with K over blocks as well)
    const double xg_us = sh.kb > 1 ? 5.4 + 0.06 * M : sh.ks == kWaves ? 3.6 + 0.03 * M : 3.6 + 0.07 * M;
    return q4_us + (sh.xl ? 3.75 + 0.035 * M : xg_us) + w_bytes / 8.0e6;
}

template <int KIND, int MT, int SW, bool XL, int TERMS>
bool launch_one(hipStream_t s, int M, int N, int K, const void* x, const void* W, const void* scale, void* out, Shape sh,
                float* partial) {
    const int ks = sh.ks;
    const long groups = ((N + 15) / 16 + SW - 1) / SW, per_block = kWaves / ks;
    const long logical = (groups + per_block - 1) / per_block;
    const size_t lds = lds_bytes(MT, K, XL, ks);
    auto* kern = gemm_skinny<KIND, MT, SW, XL, TERMS>;
    if (lds > 65536 &&
        !MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsLimit)))))
        return false;
    // with x in LDS a block is worth keeping: as many as fit a CU at once (by LDS; at most 4), each walking over the strips
    long grid = logical;
    if (XL) {
        const long per_cu = lds == 0 ? 4 : static_cast<long>(kLdsLimit / lds) < 4 ? static_cast<long>(kLdsLimit / lds) : 4;
        const long resident = static_cast<long>(device_info().cus) * (per_cu < 1 ? 1 : per_cu);
        if (grid > resident) grid = resident;
    }
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid), static_cast<unsigned>(sh.kb)), dim3(64 * kWaves), lds, s,
                       static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(W), static_cast<const uint16_t*>(scale),
                       static_cast<uint16_t*>(out), M, N, K, ks, static_cast<int>(logical), sh.kb > 1 ? partial : nullptr);
    if (!MI_HIP_OK(hipGetLastError())) return false;
    if (sh.kb > 1) {
        const long MN = static_cast<long>(M) * N;
        hipLaunchKernelGGL(wide::reduce_partials, dim3(static_cast<unsigned>((MN / 4 + 256) / 256)), dim3(256), 0, s, partial,
                           sh.kb, KIND == WK_I8 ? static_cast<const uint16_t*>(scale) : nullptr, static_cast<uint16_t*>(out),
                           MN, N);
        if (!MI_HIP_OK(hipGetLastError())) return false;
    }
    return true;
}

template <int KIND, int MT, int TERMS>
bool launch_mt(hipStream_t s, int M, int N, int K, const void* x, const void* W, const void* scale, void* out, Shape sh,
               float* partial) {
    return sh.xl ? launch_one<KIND, MT, 1, true, TERMS>(s, M, N, K, x, W, scale, out, sh, partial)
                 : launch_one<KIND, MT, 1, false, TERMS>(s, M, N, K, x, W, scale, out, sh, partial);
}

template <int KIND, int TERMS>
bool launch(hipStream_t s, int M, int N, int K, const void* x, const void* W, const void* scale, void* out, Shape sh,
            void* workspace, size_t workspace_bytes) {
    if (M < 1 || M > kMaxM || !(sh.ks == 1 || sh.ks == 2 || sh.ks == 4 || sh.ks == 8) ||
        lds_bytes((M + 15) / 16, K, sh.xl, sh.ks) > kLdsLimit || sh.kb < 1 || (sh.kb > 1 && sh.xl) ||
        (sh.kb > 1 && (!workspace || static_cast<double>(sh.kb) * M * N * 4 > static_cast<double>(workspace_bytes)))) {
        MI_ERROR_FMT("gemm: the streaming kernel takes up to %d rows of x, 1, 2, 4 or 8 slices of K per block, %zu bytes of LDS "
                     "and a workspace for slices over blocks (M=%d K=%d, %d slices, x in LDS %d, %d slices over blocks, %zu bytes)",
                     kMaxM, kLdsLimit, M, K, sh.ks, static_cast<int>(sh.xl), sh.kb, workspace_bytes);
        return false;
    }
    auto* partial = static_cast<float*>(workspace);
    switch ((M + 15) / 16) {
        case 1: return launch_mt<KIND, 1, TERMS>(s, M, N, K, x, W, scale, out, sh, partial);
        case 2: return launch_mt<KIND, 2, TERMS>(s, M, N, K, x, W, scale, out, sh, partial);
        case 3: return launch_mt<KIND, 3, TERMS>(s, M, N, K, x, W, scale, out, sh, partial);
        default: return launch_mt<KIND, 4, TERMS>(s, M, N, K, x, W, scale, out, sh, partial);
    }
}

}  // namespace skinny

template <int BM, int BN, int WM, int WN>
bool launch_tile(hipStream_t s, WeightKind kind, int M, int N, int K, const void* x, const void* W,
                 const void* scale, void* out) {
    const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, 1);
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* wp = static_cast<const uint8_t*>(W);
    const auto* sp = static_cast<const uint16_t*>(scale);
    auto* op = static_cast<uint16_t*>(out);
    constexpr size_t lds_bytes = 2u * (BM + BN) * kLd * sizeof(uint16_t);
    // more than 64 KB of LDS per block has to be asked for once per kernel
    if (kind == WK_I8) {
        auto* kern = gemm_kernel<BM, BN, WM, WN, WK_I8>;
        if (lds_bytes > 65536 &&
            !MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))))
            return false;
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, s, xp, wp, sp, op, M, N, K);
    } else {
        auto* kern = gemm_kernel<BM, BN, WM, WN, WK_F16>;
        if (lds_bytes > 65536 &&
            !MI_ONCE_OK(MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))))
            return false;
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, s, xp, wp, sp, op, M, N, K);
    }
    return MI_HIP_OK(hipGetLastError());
}

inline long tiles(int M, int N, int bm, int bn) {
    return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}

}  // namespace

bool gemm_supported(WeightKind kind, int M, int N, int K, const void* x, const void* W, const void* scale) {
    if (!(kind == WK_I8 || kind == WK_F16 || kind == WK_Q4) || M < 2 || N < 1 || K < kKT || K % kKT != 0) return false;
    if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(W) % 16) return false;
    if (kind != WK_F16 && !scale) return false;
    return kind != WK_Q4 || reinterpret_cast<uintptr_t>(scale) % 4 == 0;
}

namespace {

bool wide_reaches(WeightKind kind, int M, int N, int K) {     // 32-bit byte offsets
    return static_cast<double>(M) * K * 2 < 4294967296.0 &&
           static_cast<double>(N) * K * (kind == WK_F16 ? 2 : 1) < 4294967296.0;
}

// The 64 x 64 tiles are bound either by one tile's serial K loop (about 0.4 us per K-tile, up to
// 1.3 times that as the chip fills) or by throughput (1.2 to 1.55 ns per tile and K-tile);
// fitted to measurements.
double tiled_estimate_us(int M, int N, int K) {
    const int nk = K / kKT;
    const long t64 = tiles(M, N, 64, 64);
    const double serial = (0.9 + nk * 0.4) * (1.0 + 0.3 * (t64 < 128 ? t64 / 128.0 : 1.0));
    // (the CUs that hold a second tile set the time: 192 x 8192 x 2048, 384 tiles, takes the 22 us of 512
    //  tiles; whole rounds of CUs at such a K, halfway there at a short one: 16 x 19 456 x 896, 304 tiles,
    //  10.6 us, 1024 x 1152 x 896, 288 tiles, 9.5 us)
    const int cus = device_info().cus;
    const long rounds = (t64 + cus - 1) / cus * cus;
    const long counted = t64 <= cus ? t64 : nk >= 20 ? rounds : (t64 + rounds) / 2;
    const double bulk = 3.3 + counted * nk * (nk > 32 ? 0.00155 : 0.0012);
    return serial > bulk ? serial : bulk;
}

}  // namespace

double gemm_estimate_us(WeightKind kind, int M, int N, int K, size_t workspace_bytes) {
    const int terms = kind == WK_Q4 ? 2 : 1;
    double wide_us = 1e30;
    int tm = 1, splits = 1;
    if (wide_reaches(kind, M, N, K))
        wide::pick_shape(kind, terms, M, N, K, device_info().cus, workspace_bytes, &tm, &splits, &wide_us);
    if (M <= skinny::kMaxM && skinny::preferred(kind, M, N, K, device_info().cus, workspace_bytes))
        return skinny::estimate_us(kind, M, N, K, device_info().cus, workspace_bytes);
    if (kind == WK_Q4) return wide_us;
    const double tiled_us = tiled_estimate_us(M, N, K);
    return wide_us < tiled_us ? wide_us : tiled_us;
}

GemmPlan plan_gemm(hipStream_t s, WeightKind kind, int M, int N, int K, size_t workspace_bytes) {
    GemmPlan p;
    int mode = gemm_mode(s) == 4 && kind != WK_Q4 ? 0 : gemm_mode(s);   // mode 4 only concerns Q4 weights
    // 100 s + 10 + t: the wide kernel pinned to 32 t rows of x per block and s slices of K
    int pin_splits = 0;
    if (mode >= 111) { pin_splits = mode / 100; mode %= 100; }
    const int cus = device_info().cus;
    const bool wide_fits = wide_reaches(kind, M, N, K);
    int tm = 1, splits = 1;
    if (kind == WK_Q4) {
        // Q4 weights have the streaming kernel (a few rows of x; mode 5 asks for it by name) and the
        // wide kernel; modes 3 and 11..15 pin the latter to one slice of K.
        // Mode 4 feeds every weight as the single fp16 number nearest to q * scale (half the
        // MFMAs, an error of up to 2^-12 sum |w x|); all other modes feed q * scale exactly, as
        // two fp16 terms.
        if (mode == 2) return p;
        p.terms = mode == 4 ? 1 : 2;
        if (M <= skinny::kMaxM && (mode == 5 || ((mode == 0 || mode == 4) && skinny::preferred(WK_Q4, M, N, K, cus, workspace_bytes)))) {
            const skinny::Shape sh = skinny::pick_shape(WK_Q4, M, N, K, cus, workspace_bytes);
            p.kernel = 4; p.tile_rows = 16 * ((M + 15) / 16); p.k_slices = sh.ks * sh.kb;
            return p;
        }
        if (!wide_fits || mode == 5) return p;
        const bool may_slice = mode == 0 || mode == 4;
        wide::pick_shape(WK_Q4, p.terms, M, N, K, cus, may_slice ? workspace_bytes : 0, &tm, &splits, nullptr);
        if (mode >= 11 && mode <= 15) tm = mode - 10;
        if (pin_splits) splits = pin_splits;
        p.kernel = 1; p.tile_rows = 32 * tm; p.k_slices = splits;
        return p;
    }
    // The 256 x 256 blocks (int8 weights): by name (mode 30), or by themselves where they pay, which takes
    // several full rounds of such tiles and a long K.  Measured against the 160-row wide tiles: 8192 x 8192 x
    // 8192 884 against 968 us, 8192 x 8192 x 2048 247 against 264 us; but 4096 x 4864 x 4864 (304 tiles, 1.2
    // rounds) 229 against 177 us and 4096 x 9728 x 896 (K of 14 stages) 89 against 78 us.
    if (kind == WK_I8 && wide_fits && (mode == 30 || mode == 0)) {
        const long t256 = static_cast<long>((M + 255) / 256) * ((N + 255) / 256);
        const long rounds = (t256 + cus - 1) / cus;
        if (mode == 30 || (K >= 2048 && rounds >= 4 && t256 * 10 >= rounds * cus * 9)) {
            p.kernel = 5; p.tile_rows = 256;
            return p;
        }
    }
    if (mode == 30) return p;
    // int8 and fp16, a few rows of x: the streaming kernel (mode 5 asks for it by name, up to 64 rows)
    if (M <= skinny::kMaxM && (mode == 5 || (mode == 0 && skinny::preferred(kind, M, N, K, cus, workspace_bytes)))) {
        const skinny::Shape sh = skinny::pick_shape(kind, M, N, K, cus, workspace_bytes);
        p.kernel = 4; p.tile_rows = 16 * ((M + 15) / 16); p.k_slices = sh.ks * sh.kb;
        return p;
    }
    if (mode == 5) return p;
    // the wide kernel where its estimated time beats that of the 64 x 64 tiles
    if (wide_fits && (mode == 0 || mode == 3 || (mode >= 11 && mode <= 15))) {
        double wide_us = 0.0;
        // modes 3 and 11..15 pin the plain kernel; slices of K are the library's own choice (mode 0)
        wide::pick_shape(kind, 1, M, N, K, cus, mode == 0 ? workspace_bytes : 0, &tm, &splits, &wide_us);
        if (mode >= 11) tm = mode - 10;
        if (pin_splits) splits = pin_splits;
        if (mode != 0 || wide_us < tiled_estimate_us(M, N, K)) {
            p.kernel = 1; p.tile_rows = 32 * tm; p.k_slices = splits;
            return p;
        }
    } else if (mode == 3 || mode >= 11) {
        return p;
    }
    // 128 x 128 tiles once they fill every CU twice over (two blocks are resident per CU);
    // below that the 64 x 64 tile spreads the work over more CUs and wins (measured).
    const bool big = mode != 2 && M > 64 && tiles(M, N, 128, 128) >= 2L * cus;
    p.kernel = big ? 3 : 2; p.tile_rows = big ? 128 : 64;
    return p;
}

bool launch_gemm(hipStream_t s, WeightKind kind, int M, int N, int K, const void* x, const void* W,
                 const void* scale, void* out, void* workspace, size_t workspace_bytes) {
    if (!gemm_supported(kind, M, N, K, x, W, scale)) {
        MI_ERROR_FMT("gemm: unsupported kind=%d M=%d N=%d K=%d, or x / W not 16-byte aligned, or int8 / Q4 "
                     "without a (4-byte aligned) scale", static_cast<int>(kind), M, N, K);
        return false;
    }
    const size_t ws_bytes = workspace ? workspace_bytes : 0;
    const GemmPlan p = plan_gemm(s, kind, M, N, K, ws_bytes);
    auto* partial = static_cast<float*>(workspace);
    switch (p.kernel) {
        case 1: {
            const int tm = p.tile_rows / 32;
            if (kind == WK_Q4)
                return p.terms == 1 ? wide::launch_any<WK_Q4, 1>(tm, s, M, N, K, x, W, scale, out, partial, ws_bytes, p.k_slices)
                                    : wide::launch_any<WK_Q4, 2>(tm, s, M, N, K, x, W, scale, out, partial, ws_bytes, p.k_slices);
            if (kind == WK_F16) return wide::launch_any<WK_F16, 1>(tm, s, M, N, K, x, W, scale, out, partial, ws_bytes, p.k_slices);
            return wide::launch_any<WK_I8, 1>(tm, s, M, N, K, x, W, scale, out, partial, ws_bytes, p.k_slices);
        }
        case 4:
        {
            const skinny::Shape sh = skinny::pick_shape(kind, M, N, K, device_info().cus, ws_bytes);
            if (kind == WK_Q4)
                return p.terms == 1 ? skinny::launch<WK_Q4, 1>(s, M, N, K, x, W, scale, out, sh, workspace, ws_bytes)
                                    : skinny::launch<WK_Q4, 2>(s, M, N, K, x, W, scale, out, sh, workspace, ws_bytes);
            return kind == WK_F16 ? skinny::launch<WK_F16, 1>(s, M, N, K, x, W, scale, out, sh, workspace, ws_bytes)
                                  : skinny::launch<WK_I8, 1>(s, M, N, K, x, W, scale, out, sh, workspace, ws_bytes);
        }
        case 5: return quad::launch(s, M, N, K, x, W, scale, out);
        case 2: return launch_tile<64, 64, 32, 32>(s, kind, M, N, K, x, W, scale, out);
        case 3: return launch_tile<128, 128, 64, 64>(s, kind, M, N, K, x, W, scale, out);
        default:
            MI_ERROR_FMT("gemm: mode %d has no kernel for kind=%d M=%d N=%d K=%d (Q4 weights have no tile kernel; the "
                         "streaming kernel takes up to 64 rows of x; the wide kernel's 32-bit offsets reach 4 GiB of x and "
                         "of W)", gemm_mode(s), static_cast<int>(kind), M, N, K);
            return false;
    }
}

}  // namespace mi
