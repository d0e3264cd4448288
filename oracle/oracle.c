/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY (see oracle.h for scope, the canonical
 * evaluation order and the pinning status of every function).
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp (see Makefile).  -ffp-contract=off
 * matters: every fused multiply-add below is an explicit fmaf(), every other
 * `a*b` and `a+b` must stay a separately rounded operation.
 */
#include "oracle.h"
#include <math.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 codec
 * Follows QW/src/utils.cpp:497-564: IEEE-754 binary16, round-to-nearest-even,
 * subnormals kept, overflow saturates to +-Inf, NaN stays NaN. */
float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, o;
    if (e == 0) {
        if (m == 0) o = sign;
        else {
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; ++sh; }
            o = sign | ((uint32_t)(127 - 15 + 1 - sh) << 23) | ((m & 0x3FFu) << 13);
        }
    } else if (e == 0x1F) o = sign | 0x7F800000u | (m << 13);
    else o = sign | ((e + 112u) << 23) | (m << 13);
    float f; memcpy(&f, &o, 4); return f;
}

/* One rounding from a 64-bit significand view: works for float and double input. */
static uint16_t round_to_f16(int sign, int is_nan, int is_inf, int exp2, uint64_t sig53)
{
    /* value = sig53 * 2^(exp2-52), sig53 in [2^52, 2^53) for finite non-zero */
    uint16_t s = (uint16_t)(sign << 15);
    if (is_nan) return (uint16_t)(s | 0x7E00u);
    if (is_inf) return (uint16_t)(s | 0x7C00u);
    if (sig53 == 0) return s;
    int e = exp2 + 15;                 /* biased half exponent if normal */
    int shift;                         /* bits dropped from the 53-bit significand */
    if (e >= 0x1F) return (uint16_t)(s | 0x7C00u);
    if (e <= 0) {                      /* subnormal result: value / 2^-24 */
        shift = 42 + (1 - e);
        if (shift > 54) return s;      /* below half of the smallest subnormal */
        e = 0;
    } else shift = 42;
    uint64_t keep = (shift >= 64) ? 0 : (sig53 >> shift);
    uint64_t rem  = sig53 & ((1ull << shift) - 1ull);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (keep & 1ull))) ++keep;
    /* keep carries the implicit bit for normals: (e<<10) + keep - 0x400 folds it in,
       and a mantissa carry rolls the exponent (up to Inf) by plain addition. */
    uint32_t out = (e == 0) ? (uint32_t)keep : (uint32_t)(((uint32_t)e << 10) + (uint32_t)keep - 0x400u);
    return (uint16_t)(s | (uint16_t)out);
}

uint16_t orc_f64_to_f16(double d)
{
    uint64_t b; memcpy(&b, &d, 8);
    int sign = (int)(b >> 63);
    int eb = (int)((b >> 52) & 0x7FF);
    uint64_t m = b & 0xFFFFFFFFFFFFFull;
    if (eb == 0x7FF) return round_to_f16(sign, m != 0, m == 0, 0, 0);
    if (eb == 0) return (uint16_t)(sign << 15);            /* double subnormals are << 2^-25 */
    return round_to_f16(sign, 0, 0, eb - 1023, m | (1ull << 52));
}

uint16_t orc_f32_to_f16(float f)
{
    /* float -> double is exact, so a single rounding from the double is the
       float's own RNE rounding. */
    return orc_f64_to_f16((double)f);
}

/* --------------------------------------------------------------- quantizers */

/* LF/scripts/quantize_weights.py:53-57 (== SM/scripts/quantize_weights.py:71-75):
 *   abs_max = float(max|w|) ; scale = abs_max/127.0 (Python double) or 1.0
 *   q = clip(round(w_f32 / scale), -127, 127)   -- the division is float32 / float32(scale)
 *        because a Python float is a weak scalar against a float32 array
 *   stored scale = float16(scale)                -- one rounding from the double */
void orc_quantize_int8(const uint16_t* w, int N, int K, int8_t* q, uint16_t* sc)
{
    for (int n = 0; n < N; ++n) {
        const uint16_t* row = w + (size_t)n * K;
        float amax = 0.0f;
        int has_nan = 0;
        for (int k = 0; k < K; ++k) {
            float a = fabsf(orc_f16_to_f32(row[k]));
            if (a != a) has_nan = 1;
            if (a > amax) amax = a;
        }
        (void)has_nan;
        double scale = (amax > 0.0f) ? (double)amax / 127.0 : 1.0;
        float sf = (float)scale;
        for (int k = 0; k < K; ++k) {
            float r = rintf(orc_f16_to_f32(row[k]) / sf);   /* rintf: half-to-even, as np.round */
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            q[(size_t)n * K + k] = (int8_t)r;
        }
        sc[n] = orc_f64_to_f16(scale);
    }
}

/* LF/scripts/quantize_q4.py:62-82: per block of 32 along K,
 *   absmax (f32); s = absmax/7.0 in float32, or 1.0 ; inv = 1.0f/s (float32)
 *   q = clip(round(w*inv), -7, 7) ; stored = q+8 ; byte i = stored[2i] | stored[2i+1]<<4
 *   scale out = float16(s). Returns 0 on success, -1 if K % 32 != 0 (the script raises). */
int orc_quantize_q4(const uint16_t* w, int N, int K, uint8_t* packed, uint16_t* sc)
{
    if (K % 32 != 0) return -1;
    int nb = K / 32;
    for (int n = 0; n < N; ++n) {
        for (int b = 0; b < nb; ++b) {
            const uint16_t* blk = w + (size_t)n * K + (size_t)b * 32;
            float amax = 0.0f;
            for (int i = 0; i < 32; ++i) {
                float a = fabsf(orc_f16_to_f32(blk[i]));
                if (a > amax) amax = a;
            }
            float s = (amax > 0.0f) ? amax / 7.0f : 1.0f;
            float inv = 1.0f / s;
            uint8_t st[32];
            for (int i = 0; i < 32; ++i) {
                float r = rintf(orc_f16_to_f32(blk[i]) * inv);
                if (r < -7.0f) r = -7.0f;
                if (r > 7.0f) r = 7.0f;
                st[i] = (uint8_t)((int)r + 8);
            }
            uint8_t* out = packed + (size_t)n * (K / 2) + (size_t)b * 16;
            for (int i = 0; i < 16; ++i)
                out[i] = (uint8_t)((st[2 * i] & 0x0F) | ((st[2 * i + 1] & 0x0F) << 4));
            sc[(size_t)n * nb + b] = orc_f32_to_f16(s);
        }
    }
    return 0;
}

/* ------------------------------------------------------------- dequant views */

/* LV/kernels/lfm2_ops.cl:731-743: w16[i] = fp16((float)q[i] * scale[i / K]). */
void orc_dequant_int8_to_f16(const int8_t* q, const uint16_t* s, int N, int K, uint16_t* w16)
{
    for (int n = 0; n < N; ++n) {
        float sf = orc_f16_to_f32(s[n]);
        for (int k = 0; k < K; ++k)
            w16[(size_t)n * K + k] = orc_f32_to_f16((float)q[(size_t)n * K + k] * sf);
    }
}

/* UNPACK8_FROM_PIXEL, LF/kernels/gemv_m1_q4.cl:31-40: byte b of a row holds
 * element 2b in bits 0-3 and element 2b+1 in bits 4-7; value = nibble - 8. */
static inline int q4_at(const uint8_t* row, int k)
{
    uint8_t b = row[k >> 1];
    return (int)((k & 1) ? (b >> 4) & 0xF : b & 0xF) - 8;
}

void orc_unpack_q4(const uint8_t* p, int N, int K, int8_t* w)
{
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
            w[(size_t)n * K + k] = (int8_t)q4_at(p + (size_t)n * (K / 2), k);
}

void orc_dequant_q4_to_f32(const uint8_t* p, const uint16_t* sc, int N, int K, float* w)
{
    int nb = K / 32;
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
            w[(size_t)n * K + k] = (float)q4_at(p + (size_t)n * (K / 2), k)
                                   * orc_f16_to_f32(sc[(size_t)n * nb + k / 32]);
}

/* ------------------------------------------------------------------- GEMV core */

/* 64-lane tree, QW/kernels/gemv_m1.cl:415-424. */
static inline float tree64(float* p)
{
    for (int s = 32; s > 0; s >>= 1)
        for (int t = 0; t < s; ++t) p[t] = p[t] + p[t + s];
    return p[0];
}

/* OpenCL dot(float4,float4) with mad contraction, elements in x,y,z,w order. */
static inline float dot4(const float* x, const float* w)
{
    float d = x[0] * w[0];
    d = fmaf(x[1], w[1], d);
    d = fmaf(x[2], w[2], d);
    d = fmaf(x[3], w[3], d);
    return d;
}

/* fp16 weights: QW/kernels/gemv_m1.cl:366-462, 580-690; SM/kernels/block_fused.cl:407-465.
 * Lane t, iteration j: elements 256j+4t .. +3; a partial last iteration runs the
 * lanes whose 4 elements lie below K (K % 4 == 0). */
static float row_f16(const float* xf, const uint16_t* wrow, int K)
{
    float part[64];
    for (int t = 0; t < 64; ++t) part[t] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += 256)
        for (int t = 0; t < 64; ++t) {
            int k = k0 + 4 * t;
            if (k + 4 > K) break;
            float w[4];
            for (int e = 0; e < 4; ++e) w[e] = orc_f16_to_f32(wrow[k + e]);
            part[t] = part[t] + dot4(xf + k, w);
        }
    return tree64(part);
}

/* int8 weights: LF/kernels/gemv_m1_int8.cl:32-79; SM/kernels/block_fused_int8.cl:37-103.
 * Same lane ownership; the per-row scale multiplies the reduced sum once. */
static float row_i8(const float* xf, const int8_t* qrow, int K)
{
    float part[64];
    for (int t = 0; t < 64; ++t) part[t] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += 256)
        for (int t = 0; t < 64; ++t) {
            int k = k0 + 4 * t;
            if (k + 4 > K) break;
            float w[4];
            for (int e = 0; e < 4; ++e) w[e] = (float)qrow[k + e];
            part[t] = part[t] + dot4(xf + k, w);
        }
    return tree64(part);
}

/* Q4 weights: LF/kernels/gemv_m1_q4.cl:45-123.  Lane t, iteration j owns packed
 * pixel p = 64j+t = 4 bytes = elements 8p..8p+7, scale block p>>2. */
static float row_q4(const float* xf, const uint8_t* prow, const uint16_t* srow, int K)
{
    float part[64];
    for (int t = 0; t < 64; ++t) part[t] = 0.0f;
    int npix = K / 8;
    for (int p0 = 0; p0 < npix; p0 += 64)
        for (int t = 0; t < 64; ++t) {
            int p = p0 + t;
            if (p >= npix) break;
            const float* xv = xf + 8 * p;
            float d = xv[0] * (float)q4_at(prow, 8 * p);
            for (int e = 1; e < 8; ++e) d = fmaf(xv[e], (float)q4_at(prow, 8 * p + e), d);
            part[t] = fmaf(d, orc_f16_to_f32(srow[p >> 2]), part[t]);
        }
    return tree64(part);
}

static float* x_to_f32(const uint16_t* x, int K)
{
    float* xf = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
    for (int k = 0; k < K; ++k) xf[k] = orc_f16_to_f32(x[k]);
    return xf;
}

int orc_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* The flags this library was compiled with (oracle/Makefile passes them in), for the benchmark's
 * CPU-baseline record. */
#ifndef ORC_BUILD_FLAGS
#define ORC_BUILD_FLAGS "unknown"
#endif
const char* orc_build_flags(void) { return ORC_BUILD_FLAGS; }

static int clamp_threads(int n)
{
    if (n < 1) n = 1;
    int m = orc_max_threads();
    return n > m ? m : n;
}

void orc_gemv_f16(const uint16_t* x, const uint16_t* W, uint16_t* y, int N, int K, int nt)
{
    float* xf = x_to_f32(x, K);
    nt = clamp_threads(nt);
    #pragma omp parallel for num_threads(nt) schedule(static)
    for (int n = 0; n < N; ++n)
        y[n] = orc_f32_to_f16(row_f16(xf, W + (size_t)n * K, K));
    free(xf);
}

void orc_gemv_i8_f32(const uint16_t* x, const int8_t* q, const uint16_t* s, float* y, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        y[n] = row_i8(xf, q + (size_t)n * K, K) * orc_f16_to_f32(s[n]);
    free(xf);
}

void orc_gemv_i8(const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* y, int N, int K, int nt)
{
    float* xf = x_to_f32(x, K);
    nt = clamp_threads(nt);
    #pragma omp parallel for num_threads(nt) schedule(static)
    for (int n = 0; n < N; ++n)
        y[n] = orc_f32_to_f16(row_i8(xf, q + (size_t)n * K, K) * orc_f16_to_f32(s[n]));
    free(xf);
}

void orc_gemv_q4(const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* y, int N, int K, int nt)
{
    float* xf = x_to_f32(x, K);
    nt = clamp_threads(nt);
    #pragma omp parallel for num_threads(nt) schedule(static)
    for (int n = 0; n < N; ++n)
        y[n] = orc_f32_to_f16(row_q4(xf, p + (size_t)n * (K / 2), sc + (size_t)n * (K / 32), K));
    free(xf);
}

/* ------------------------------------------------------------ fused epilogues */

/* QW/kernels/gemv_m1.cl:756-765: out[n] = fp16(sum + f32(out[n])). */
void orc_gemv_f16_add(const uint16_t* x, const uint16_t* W, uint16_t* res, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        res[n] = orc_f32_to_f16(row_f16(xf, W + (size_t)n * K, K) + orc_f16_to_f32(res[n]));
    free(xf);
}

/* SM/kernels/block_fused_int8.cl:154-167: res[n] = fp16(r + partial*s), contracted to fma. */
void orc_gemv_i8_add(const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* res, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        res[n] = orc_f32_to_f16(fmaf(row_i8(xf, q + (size_t)n * K, K), orc_f16_to_f32(s[n]),
                                     orc_f16_to_f32(res[n])));
    free(xf);
}

/* No Q4 residual kernel exists in the reference; this follows the int8/fp16
 * forms: one fp32 add of the residual before the single fp16 rounding. */
void orc_gemv_q4_add(const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* res, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        res[n] = orc_f32_to_f16(row_q4(xf, p + (size_t)n * (K / 2), sc + (size_t)n * (K / 32), K)
                                + orc_f16_to_f32(res[n]));
    free(xf);
}

/* exp() for the SwiGLU epilogue.  The reference calls native_exp, whose
 * precision is implementation-defined, so the oracle fixes one fp32 evaluation
 * built only from fmaf/rintf/ldexp that a GPU can repeat bit for bit:
 * range reduction by ln2 (Cody-Waite, two constants) and a degree-7 Horner
 * polynomial on [-ln2/2, ln2/2].  Tested against libm expf to <= 2 ulp. */
static float orc_expf(float x)
{
    if (x > 88.0f) return INFINITY;
    if (x < -87.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);          /* ln2 high part, 11 bits */
    r = fmaf(n, -1.42860682030941723212e-6f, r);        /* ln2 low part */
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    return ldexpf(p, (int)n);
}

float orc_expf_export(float x) { return orc_expf(x); }

static inline float silu_mul(float g, float u)
{
    return (g / (1.0f + orc_expf(-g))) * u;
}

/* SM/kernels/block_fused_int8.cl:176-236. */
void orc_gate_up_silu_i8(const uint16_t* x, const int8_t* qg, const int8_t* qu,
                         const uint16_t* sg, const uint16_t* su, uint16_t* out, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n) {
        float g = row_i8(xf, qg + (size_t)n * K, K) * orc_f16_to_f32(sg[n]);
        float u = row_i8(xf, qu + (size_t)n * K, K) * orc_f16_to_f32(su[n]);
        out[n] = orc_f32_to_f16(silu_mul(g, u));
    }
    free(xf);
}

/* SM/kernels/block_fused.cl:473-526. */
void orc_gate_up_silu_f16(const uint16_t* x, const uint16_t* Wg, const uint16_t* Wu,
                          uint16_t* out, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n) {
        float g = row_f16(xf, Wg + (size_t)n * K, K);
        float u = row_f16(xf, Wu + (size_t)n * K, K);
        out[n] = orc_f32_to_f16(silu_mul(g, u));
    }
    free(xf);
}

/* LF/kernels/mlp_fused.cl:19-79 (gemv_m1_k1024_no8_silufused_img): the fp32 row sum w3x, then
 * gate[n] = fp16(gate * sig * w3x) with sig = 1 / (1 + exp(-gate)), gate read as fp16.  The
 * reference has the fp16 form only; int8 and Q4 take the scaled row sum of their GEMV. */
static inline float silu_gate(float gate, float w3x)
{
    float sig = 1.0f / (1.0f + orc_expf(-gate));
    return (gate * sig) * w3x;
}

void orc_gemv_f16_silu_gate(const uint16_t* x, const uint16_t* W, uint16_t* gate, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        gate[n] = orc_f32_to_f16(silu_gate(orc_f16_to_f32(gate[n]), row_f16(xf, W + (size_t)n * K, K)));
    free(xf);
}

void orc_gemv_i8_silu_gate(const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* gate, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        gate[n] = orc_f32_to_f16(silu_gate(orc_f16_to_f32(gate[n]),
                                           row_i8(xf, q + (size_t)n * K, K) * orc_f16_to_f32(s[n])));
    free(xf);
}

void orc_gemv_q4_silu_gate(const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* gate, int N, int K)
{
    float* xf = x_to_f32(x, K);
    for (int n = 0; n < N; ++n)
        gate[n] = orc_f32_to_f16(silu_gate(orc_f16_to_f32(gate[n]),
                                           row_q4(xf, p + (size_t)n * (K / 2), sc + (size_t)n * (K / 32), K)));
    free(xf);
}

/* ------------------------------------------------------------------- M > 1 */

void orc_gemm_f16(const uint16_t* X, const uint16_t* W, uint16_t* out, int M, int N, int K, int nt)
{
    for (int m = 0; m < M; ++m) orc_gemv_f16(X + (size_t)m * K, W, out + (size_t)m * N, N, K, nt);
}

void orc_gemm_i8(const uint16_t* X, const int8_t* q, const uint16_t* s, uint16_t* out, int M, int N, int K, int nt)
{
    for (int m = 0; m < M; ++m) orc_gemv_i8(X + (size_t)m * K, q, s, out + (size_t)m * N, N, K, nt);
}

void orc_gemm_q4(const uint16_t* X, const uint8_t* p, const uint16_t* sc, uint16_t* out, int M, int N, int K, int nt)
{
    for (int m = 0; m < M; ++m) orc_gemv_q4(X + (size_t)m * K, p, sc, out + (size_t)m * N, N, K, nt);
}
