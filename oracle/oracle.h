/*
 * CPU oracle for the weight-only quantized matmul path of a8nova/adreno-llms.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C, the
 * arithmetic of the reference's OpenCL GEMV kernels, of its two offline
 * quantizers and of its fp16 host codec, so that the HIP path can be checked
 * against it.  Only the test-suite, the smoke check and the benchmark's
 * CPU-baseline leg may link or load this library; nothing in the shipped
 * library calls into it.
 *
 * All paths below are relative to the reference tree
 *   QW/ = src/models/qwen2-5-0-5b/      LF/ = src/models/lfm2-5-350m/
 *   SM/ = src/models/smollm2-135m-instruct/   LV/ = src/models/lfm2-5-vl-450m/
 *
 * Canonical evaluation order.  The reference compiles its kernels with
 * -cl-fast-relaxed-math (QW/src/opencl_context.cpp make_effective_options),
 * which implies -cl-mad-enable, so `a*b + c` is a fused multiply-add on the
 * device and no single bit pattern is "the" reference result.  The oracle
 * fixes one evaluation, the one the kernel source spells out, with every
 * `a*b + c` contracted to fmaf and nothing re-associated:
 *   - lane `t` of 64 owns, in K-iteration `j`, the 4 consecutive elements at
 *     k = 256*j + 4*t (fp16, int8) or the 8 consecutive elements of packed
 *     pixel p = 64*j + t (Q4);
 *   - dot(x4, w4) = fma(x3,w3, fma(x2,w2, fma(x1,w1, x0*w0)));  acc = acc + dot;
 *   - Q4: d = fma chain over the 8 elements left to right, acc = fma(d, scale, acc);
 *   - 64-lane tree: for s = 32,16,..,1: partial[t] += partial[t+s] (t < s);
 *   - epilogue in fp32, one RNE rounding to fp16 at the store.
 *
 * Pinning status (what checks each function against something other than
 * itself is listed in tests/test_oracle_*.py):
 *   orc_f16_to_f32 / orc_f32_to_f16 / orc_f64_to_f16 : exhaustive vs numpy.float16
 *   orc_quantize_int8 / orc_quantize_q4 : golden vectors written by the
 *        reference's own quantize_row_symmetric / quantize_row_q4
 *        (tests/golden/), closed-form invariants
 *   orc_unpack_q4 : brute force over all 256 byte values vs the macro's formula
 *   orc_gemv_* : unit-vector / identity / all-ones closed forms, fp64 dot
 *        product within tolerance, lane-ownership probes that fail on a wrong
 *        index, a dropped tail or a wrong scale block: pinned to the bar
 *        stated for floating point (max-abs / rel 1e-3, cosine >= 0.9999) and
 *        exactly where the arithmetic is exact (integer-valued data, unit
 *        vectors).  Beyond that bar the bit pattern is this file's own choice
 *        of evaluation order: the reference's device code is built with
 *        -cl-fast-relaxed-math and holds no known-answer vector for a GEMV, so
 *        there is no reference bit pattern to match.
 *   orc_gemv_q4_add : the reference has no Q4 residual kernel (its fused residual form,
 *        SM/kernels/block_fused_int8.cl:105-174, is int8 only), so the mathematics pins it:
 *        res + dequant(W) x in fp64 within one fp16 step, zero residual == orc_gemv_q4
 *        bit for bit, a swamping residual returned unchanged (tests/test_oracle_gemv.py).
 *   decode.c (rmsnorm, rotary, attention, SwiGLU, adds, whole step): fp64
 *        statements and index probes in tests/test_oracle_decode.py.
 */
#ifndef ORACLE_H
#define ORACLE_H
#include <stdint.h>
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

/* fp16 codec: QW/src/utils.cpp:497-564 (nnopt_f16_to_f32 / nnopt_f32_to_f16). */
float    orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
uint16_t orc_f64_to_f16(double d);   /* single rounding, as numpy.float16(python_float) */

/* Quantizers: LF/scripts/quantize_weights.py:53-57, LF/scripts/quantize_q4.py:62-82. */
void orc_quantize_int8(const uint16_t* w_f16, int N, int K, int8_t* q, uint16_t* scale_f16);
int  orc_quantize_q4(const uint16_t* w_f16, int N, int K, uint8_t* packed, uint16_t* scale_f16);

/* Dequant views. LV/kernels/lfm2_ops.cl:731-743; LF/kernels/gemv_m1_q4.cl:31-40. */
void orc_dequant_int8_to_f16(const int8_t* q, const uint16_t* scale, int N, int K, uint16_t* w16);
void orc_unpack_q4(const uint8_t* packed, int N, int K, int8_t* w);
void orc_dequant_q4_to_f32(const uint8_t* packed, const uint16_t* scale, int N, int K, float* w);

/* GEMV, M = 1.  x fp16 [K], y fp16 [N].  n_threads <= 1 runs single threaded. */
void orc_gemv_f16(const uint16_t* x, const uint16_t* W, uint16_t* y, int N, int K, int n_threads);
void orc_gemv_i8 (const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* y, int N, int K, int n_threads);
void orc_gemv_q4 (const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* y, int N, int K, int n_threads);

/* fp32 pre-rounding values of the same GEMVs (for tolerance analysis in tests). */
void orc_gemv_i8_f32(const uint16_t* x, const int8_t* q, const uint16_t* s, float* y, int N, int K);

/* Fused epilogues: SM/kernels/block_fused_int8.cl:105-174, 176-236, 238-291;
 * QW/kernels/gemv_m1.cl:708-809 (fp16 residual form). */
void orc_gemv_f16_add(const uint16_t* x, const uint16_t* W, uint16_t* res, int N, int K);
void orc_gemv_i8_add (const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* res, int N, int K);
void orc_gemv_q4_add (const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* res, int N, int K);
void orc_gate_up_silu_i8(const uint16_t* x, const int8_t* qg, const int8_t* qu,
                         const uint16_t* sg, const uint16_t* su, uint16_t* out, int N, int K);
void orc_gate_up_silu_f16(const uint16_t* x, const uint16_t* Wg, const uint16_t* Wu,
                          uint16_t* out, int N, int K);

/* LF/kernels/mlp_fused.cl:19-79: gate[n] = fp16((gate * sigmoid(gate)) * (W x)[n]), W x in fp32
 * (the reference has the fp16 form; int8 and Q4 use the scaled row sum of their GEMV). */
void orc_gemv_f16_silu_gate(const uint16_t* x, const uint16_t* W, uint16_t* gate, int N, int K);
void orc_gemv_i8_silu_gate (const uint16_t* x, const int8_t* q, const uint16_t* s, uint16_t* gate, int N, int K);
void orc_gemv_q4_silu_gate (const uint16_t* x, const uint8_t* p, const uint16_t* sc, uint16_t* gate, int N, int K);

/* M > 1: out[M,N] row i = GEMV of X row i (LF/src/model.cpp:243-250). */
void orc_gemm_f16(const uint16_t* X, const uint16_t* W, uint16_t* out, int M, int N, int K, int n_threads);
void orc_gemm_i8 (const uint16_t* X, const int8_t* q, const uint16_t* s, uint16_t* out, int M, int N, int K, int n_threads);
void orc_gemm_q4 (const uint16_t* X, const uint8_t* p, const uint16_t* sc, uint16_t* out, int M, int N, int K, int n_threads);

int orc_max_threads(void);
const char* orc_build_flags(void);   /* compiler and flags of this build */

/* argmax_partial (NP work-groups of 64 over contiguous chunks) + argmax_finalize, literally:
 * QW/kernels/gemv_m1.cl:198-280.  Index of the greatest fp16 value with the kernels' own tie
 * behaviour; 1 <= NP <= 4096.  Parity: the tie order is what the source spells out (strict ">" in
 * the strided scan and in both trees); checked against a brute-force statement of that order in
 * tests/test_oracle_gemv.py. */
int orc_argmax_f16(const uint16_t* x, int N, int NP);

#ifdef __cplusplus
}
#endif
#endif
