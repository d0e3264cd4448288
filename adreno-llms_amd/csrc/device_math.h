// Device-side scalar helpers shared by the kernels: the fp16 codec as the kernels use it and the
// exponential that every kernel (and the CPU oracle) evaluates with the same operations.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdint>

namespace mi {

__device__ __forceinline__ float h_f(uint16_t h) { return __half2float(__ushort_as_half(h)); }

// fp32 -> fp16, round to nearest even.  The empty asm pins the fp32 value in a register
// first: without it the compiler folds a preceding multiply or fma into v_fma_mixlo_f16,
// which rounds once to fp16, while the reference rounds the product to fp32 and then
// stores it as half (two roundings; they differ on about one value in 8000).
__device__ __forceinline__ uint16_t f_h(float f) {
    asm volatile("" : "+v"(f));
    return __half_as_ushort(__float2half_rn(f));
}

// The value lane g + 32 (resp. g + 16) holds, for the lanes that have such a partner in the tree
// reductions (g < 32; g % 32 < 16); the other lanes receive a value that no tree uses.  These are
// v_permlane32_swap / v_permlane16_swap, register-to-register moves of gfx950, in place of a trip
// through the LDS crossbar (ds_bpermute): with both operands the same register the "swapped-in"
// half of the second result is the upper half (resp. the odd rows of 16) of the input.
__device__ __forceinline__ float lane_plus32(float a) {
    const unsigned u = __float_as_uint(a);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[1]);
}
__device__ __forceinline__ float lane_plus16(float a) {
    const unsigned u = __float_as_uint(a);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __uint_as_float(r[1]);
}

// The greatest of a wavefront's 64 values, in every lane (register moves and DPP row shifts; a
// lane without a partner in a step compares with itself).
template <int SH> __device__ __forceinline__ float max_from_above(float a) {
    const int t = __builtin_amdgcn_update_dpp(__float_as_int(a), __float_as_int(a), 0x100 + SH, 0xf, 0xf, false);
    return fmaxf(a, __int_as_float(t));
}
__device__ __forceinline__ float wave_max(float m) {
    m = fmaxf(m, lane_plus32(m));
    m = fmaxf(m, lane_plus16(m));
    m = max_from_above<8>(m);
    m = max_from_above<4>(m);
    m = max_from_above<2>(m);
    m = max_from_above<1>(m);
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(m)));
}

// exp() of the SwiGLU epilogue: range reduction by ln2 in two parts and a degree-7 Horner
// polynomial, built from fma/rint/ldexp only so that a host evaluation of the same
// formula gives the same bits (the reference's native_exp has no defined precision,
// SM/kernels/block_fused_int8.cl:229).
__device__ __forceinline__ float exp_poly(float x) {
    if (x > 88.0f) return __builtin_huge_valf();
    if (x < -87.0f) return 0.0f;
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);
    r = fmaf(n, -1.42860682030941723212e-6f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    return ldexpf(p, static_cast<int>(n));
}

}  // namespace mi
