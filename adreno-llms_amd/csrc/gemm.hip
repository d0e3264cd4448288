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

namespace mi {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// ---- 128 x 128 tile, two wavefronts ------------------------------------------------
//
// The kernel above spends more LDS bandwidth than matrix-core time: a wavefront that owns
// 64 x 64 outputs reads four operand fragments for four MFMAs.  Here a block is 128 (rows of
// x) x 128 (rows of W) with only two wavefronts, each owning all 128 rows of x against 64
// rows of W: six fragments for eight MFMAs, and accumulators of 128 registers per lane.
// Four such blocks share a CU (K-tile 32, two LDS stages of 20 KB each), i.e. two wavefronts
// per SIMD.  W is the MFMA "A" operand and x the "B" operand, so a lane ends up with four
// consecutive output columns of one output row: the epilogue scales them and writes 8 bytes
// per lane instead of four 2-byte stores.
constexpr int kKT2 = 32;
constexpr int kLd2 = kKT2 + 8;     // 40 halves = 80 bytes: 8 consecutive rows, 8 different 16-byte slots

template <int KIND>
__global__ __launch_bounds__(128) void gemm_kernel_128x128(const uint16_t* __restrict__ X,
                                                          const uint8_t* __restrict__ W,
                                                          const uint16_t* __restrict__ scale,
                                                          uint16_t* __restrict__ out, int M, int N, int K) {
    constexpr int BM = 128, BN = 128, NT = 128;
    constexpr int TM = 4, TN = 2;                                       // 32-wide tiles per wavefront
    constexpr int A_CHUNKS = BM * (kKT2 / 8) / NT;                      // 4: 16-byte chunks of x per thread
    constexpr int B_BYTES = KIND == WK_I8 ? 1 : 2;
    constexpr int B_CPR = kKT2 * B_BYTES / 16;                          // chunks per W row: 2 (int8) or 4
    constexpr int B_CHUNKS = BN * B_CPR / NT;                           // 2 or 4
    constexpr int kStage = (BM + BN) * kLd2;                            // halves per LDS stage

    __shared__ __attribute__((aligned(16))) uint16_t lds[2 * kStage];

    const int tid = threadIdx.x, lane = tid % 64, wn = tid / 64;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int gk = lane / 32, li = lane % 32;

    floatx16 acc[TN][TM];
    #pragma unroll
    for (int u = 0; u < TN; ++u)
        #pragma unroll
        for (int t = 0; t < TM; ++t)
            #pragma unroll
            for (int r = 0; r < 16; ++r) acc[u][t][r] = 0.0f;

    struct Regs { u32x4 a[A_CHUNKS]; u32x4 b[B_CHUNKS]; };
    auto load_tile = [&](Regs& R, int k0) {
        #pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / (kKT2 / 8), kc = c % (kKT2 / 8);
            const int m = m0 + row < M ? m0 + row : M - 1;
            R.a[i] = *reinterpret_cast<const u32x4*>(X + static_cast<size_t>(m) * K + k0 + kc * 8);
        }
        #pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / B_CPR, kc = c % B_CPR;
            const int n = n0 + row < N ? n0 + row : N - 1;
            R.b[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                W + (static_cast<size_t>(n) * K + k0) * B_BYTES + kc * 16));
        }
    };
    auto store_tile = [&](const Regs& R, uint16_t* Xs, uint16_t* Ws) {
        #pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / (kKT2 / 8), kc = c % (kKT2 / 8);
            *reinterpret_cast<u32x4*>(&Xs[row * kLd2 + kc * 8]) = R.a[i];
        }
        #pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / B_CPR, kc = c % B_CPR;
            if constexpr (KIND == WK_I8) {
                uint32_t h[8];
                i8x4_to_h4(R.b[i].x, h[0], h[1]);
                i8x4_to_h4(R.b[i].y, h[2], h[3]);
                i8x4_to_h4(R.b[i].z, h[4], h[5]);
                i8x4_to_h4(R.b[i].w, h[6], h[7]);
                *reinterpret_cast<u32x4*>(&Ws[row * kLd2 + kc * 16]) = u32x4{h[0], h[1], h[2], h[3]};
                *reinterpret_cast<u32x4*>(&Ws[row * kLd2 + kc * 16 + 8]) = u32x4{h[4], h[5], h[6], h[7]};
            } else {
                *reinterpret_cast<u32x4*>(&Ws[row * kLd2 + kc * 8]) = R.b[i];
            }
        }
    };
    auto multiply = [&](const uint16_t* Xs, const uint16_t* Ws) {
        #pragma unroll
        for (int kk = 0; kk < kKT2 / 16; ++kk) {
            const int kcol = 16 * gk + 8 * kk;      // lane group gk supplies k = 16 gk + 8 kk .. +7
            half8 w[TN], xf[TM];
            #pragma unroll
            for (int u = 0; u < TN; ++u)
                w[u] = *reinterpret_cast<const half8*>(&Ws[(wn * 64 + u * 32 + li) * kLd2 + kcol]);
            #pragma unroll
            for (int t = 0; t < TM; ++t)
                xf[t] = *reinterpret_cast<const half8*>(&Xs[(t * 32 + li) * kLd2 + kcol]);
            #pragma unroll
            for (int u = 0; u < TN; ++u)
                #pragma unroll
                for (int t = 0; t < TM; ++t)
                    acc[u][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[u], xf[t], acc[u][t], 0, 0, 0);
        }
    };

    const int nk = K / kKT2;
    Regs R0, R1, R2;
    load_tile(R0, 0);
    load_tile(R1, (1 < nk ? 1 : nk - 1) * kKT2);
    load_tile(R2, (2 < nk ? 2 : nk - 1) * kKT2);
#define MI_GEMM2_STEP(R)                                                       \
    {                                                                          \
        uint16_t* Xs = lds + (i & 1) * kStage;                                 \
        uint16_t* Ws = Xs + BM * kLd2;                                         \
        store_tile(R, Xs, Ws);                                                 \
        __syncthreads();                                                       \
        load_tile(R, (i + 3 < nk ? i + 3 : nk - 1) * kKT2);                    \
        multiply(Xs, Ws);                                                      \
        if (++i >= nk) break;                                                  \
    }
    for (int i = 0;;) {
        MI_GEMM2_STEP(R0)
        MI_GEMM2_STEP(R1)
        MI_GEMM2_STEP(R2)
    }
#undef MI_GEMM2_STEP

    // D[i][j]: i = 8 (r / 4) + 4 (lane / 32) + r % 4 is a W row (an output column), j = lane % 32
    // is a row of x (an output row): a lane holds 4 consecutive output columns per r / 4.
    const bool vec_ok = (N % 4) == 0;
    #pragma unroll
    for (int u = 0; u < TN; ++u) {
        #pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            const int n = n0 + wn * 64 + u * 32 + 8 * rq + 4 * gk;      // first of 4 columns
            float s4[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if constexpr (KIND == WK_I8) {
                #pragma unroll
                for (int e = 0; e < 4; ++e)
                    s4[e] = __half2float(__ushort_as_half(scale[n + e < N ? n + e : N - 1]));
            }
            #pragma unroll
            for (int t = 0; t < TM; ++t) {
                const int m = m0 + t * 32 + li;
                if (m >= M) continue;
                uint16_t h[4];
                #pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = KIND == WK_I8 ? acc[u][t][4 * rq + e] * s4[e] : acc[u][t][4 * rq + e];
                    h[e] = to_half_bits(v);
                }
                uint16_t* dst = out + static_cast<size_t>(m) * N + n;
                if (vec_ok && n + 3 < N) {
                    uint2 pk;
                    pk.x = static_cast<uint32_t>(h[0]) | (static_cast<uint32_t>(h[1]) << 16);
                    pk.y = static_cast<uint32_t>(h[2]) | (static_cast<uint32_t>(h[3]) << 16);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
                    #pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) dst[e] = h[e];
                }
            }
        }
    }
}

template <int KIND_UNUSED = 0>
bool launch_128x128(hipStream_t s, WeightKind kind, int M, int N, int K, const void* x, const void* W,
                    const void* scale, void* out) {
    const dim3 grid((N + 127) / 128, (M + 127) / 128, 1);
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* wp = static_cast<const uint8_t*>(W);
    const auto* sp = static_cast<const uint16_t*>(scale);
    auto* op = static_cast<uint16_t*>(out);
    if (kind == WK_I8)
        hipLaunchKernelGGL(gemm_kernel_128x128<WK_I8>, grid, dim3(128), 0, s, xp, wp, sp, op, M, N, K);
    else
        hipLaunchKernelGGL(gemm_kernel_128x128<WK_F16>, grid, dim3(128), 0, s, xp, wp, sp, op, M, N, K);
    return MI_HIP_OK(hipGetLastError());
}

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
    static bool raised_i8 = false, raised_f16 = false;
    if (kind == WK_I8) {
        auto* kern = gemm_kernel<BM, BN, WM, WN, WK_I8>;
        if (lds_bytes > 65536 && !raised_i8) {
            if (!MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))) return false;
            raised_i8 = true;
        }
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, s, xp, wp, sp, op, M, N, K);
    } else {
        auto* kern = gemm_kernel<BM, BN, WM, WN, WK_F16>;
        if (lds_bytes > 65536 && !raised_f16) {
            if (!MI_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes))) return false;
            raised_f16 = true;
        }
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, s, xp, wp, sp, op, M, N, K);
    }
    return MI_HIP_OK(hipGetLastError());
}

inline long tiles(int M, int N, int bm, int bn) {
    return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}

}  // namespace

bool gemm_supported(WeightKind kind, int M, int N, int K) {
    return (kind == WK_I8 || kind == WK_F16) && M >= 16 && N >= 1 && K >= kKT && K % kKT == 0;
}

bool launch_gemm(hipStream_t s, WeightKind kind, int M, int N, int K, const void* x, const void* W,
                 const void* scale, void* out) {
    if (!gemm_supported(kind, M, N, K)) {
        MI_ERROR_FMT("gemm: unsupported kind=%d M=%d N=%d K=%d", static_cast<int>(kind), M, N, K);
        return false;
    }
    if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(W) % 16 ||
        (kind == WK_I8 && !scale)) {
        MI_ERROR_FMT("gemm: x and W must be 16-byte aligned, int8 needs a scale");
        return false;
    }
    // 128 x 128 tiles once they fill every CU twice over (two blocks are resident per CU);
    // below that the 64 x 64 tile spreads the work over more CUs and wins (measured).
    const int mode = gemm_mode();
    if (mode == 3) return launch_128x128<>(s, kind, M, N, K, x, W, scale, out);
    if (mode != 2 && M > 64 && tiles(M, N, 128, 128) >= 2L * device_info().cus)
        return launch_tile<128, 128, 64, 64>(s, kind, M, N, K, x, W, scale, out);
    return launch_tile<64, 64, 32, 32>(s, kind, M, N, K, x, W, scale, out);
}

}  // namespace mi
