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
