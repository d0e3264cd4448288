/*
 * mi_linear.h -- C ABI of the MI355X (gfx950) weight-only quantized matmul path.
 *
 * Drop-in boundary for the `pytorch_linear` family of a8nova/adreno-llms: the
 * entry points below are what a foreign-function binding for the projection /
 * lm_head calls in src/models/<model>/src would bind.  Device pointers stand where the
 * reference passes cl_mem handles, a stream (hipStream_t passed as void*, NULL =
 * the default stream) stands where it passes a cl_command_queue.
 *
 * Conventions, as in the reference (QW/src/utils.h:98-121, QW/src/debug_utils.h:56-64):
 *   - functions that the reference declares `bool` return 1 (work enqueued) or 0
 *     (nothing usable was enqueued); every failure prints
 *     "ERROR: <message> (<file>:<line>)" on stderr; no exceptions, no errno;
 *   - calls are asynchronous: they return after the launch; work on one stream runs
 *     in order, so `out` is visible to the next call on the same stream;
 *   - x, W, scale and out are caller-owned; the library keeps only the registry
 *     entries made by mi_register_*_weight, keyed by the raw pointer value;
 *   - the quantisation of W is not an argument: it is looked up from the W pointer
 *     (LF/src/utils.cpp:1286-1325: Q4 first, then int8, then fp16);
 *   - layouts are the ones of the reference bundles (scripts/convert_hf_to_bin.py,
 *     LF/scripts/quantize_weights.py, LF/scripts/quantize_q4.py): W [N,K] row-major,
 *     fp16, or int8 with fp16 scale[N], or Q4 packed [N,K/2] (low nibble = even
 *     element, value = nibble-8) with fp16 scale[N,K/32].
 *
 * Paths: QW/ = src/models/qwen2-5-0-5b/, LF/ = src/models/lfm2-5-350m/,
 * SM/ = src/models/smollm2-135m-instruct/, LV/ = src/models/lfm2-5-vl-450m/.
 */
#ifndef MI_LINEAR_H
#define MI_LINEAR_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- runtime plumbing: what the reference host code takes from cl.h ------------- */

/* Select the GPU and check that it is a gfx950 part.  Replaces
 * OpenCLContext::initialize (QW/src/opencl_context.cpp:171-205).  Returns 1/0. */
int mi_init(int device);
/* Name of the device's architecture ("gfx950..."), valid after mi_init. */
const char* mi_device_arch(void);
/* Number of compute units of the selected device. */
int mi_device_cus(void);

/* clCreateBuffer / clReleaseMemObject (QW/src/weights.cpp:262-293). */
void* mi_malloc(size_t bytes);
int   mi_free(void* dev_ptr);
/* clEnqueueWriteBuffer / clEnqueueReadBuffer, blocking form. */
int mi_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);
int mi_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);
int mi_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
int mi_memset(void* dst_dev, int byte, size_t bytes, void* stream);
/* clCreateCommandQueue / clReleaseCommandQueue / clFinish (QW/src/opencl_context.cpp:196-205). */
void* mi_stream_create(void);
int   mi_stream_destroy(void* stream);
int   mi_stream_sync(void* stream);
/* Event timing on a stream; stands for CL_QUEUE_PROFILING_ENABLE + clGetEventProfilingInfo
 * (QW/src/prof.cpp:34-135). */
void* mi_event_create(void);
int   mi_event_destroy(void* ev);
int   mi_event_record(void* ev, void* stream);
int   mi_event_sync(void* ev);
float mi_event_elapsed_ms(void* start_ev, void* stop_ev);

/* ---- weight registry ------------------------------------------------------------ */

/* nnopt_register_int8_weight (LF/src/utils.h:129, LF/src/utils.cpp:357-368). */
int mi_register_int8_weight(const void* W_int8, const void* scale_fp16, int N, int K);
/* nnopt_register_q4_weight (LF/src/utils.h:134, LF/src/utils.cpp:584-595); K = unpacked K. */
int mi_register_q4_weight(const void* W_q4, const void* scale_fp16, int N, int K);
/* The reference never unregisters; provided so that a freed pointer can be reused. */
int mi_unregister_weight(const void* W);
/* 0 = not registered (fp16), 8 = int8, 4 = Q4. */
int mi_weight_kind(const void* W);

/* ---- the hot path --------------------------------------------------------------- */

/* pytorch_linear (QW/src/utils.h:119-121, QW/src/utils.cpp:758-823, LF/src/utils.cpp:1263-1374):
 * out[M,N] = x[M,K] @ W[N,K]^T, fp16 in/out, fp32 accumulate. */
int mi_linear(void* stream, int M, int N, int K, const void* x, const void* W, void* out);

/* pytorch_linear_add (QW/src/utils.h:133-135; int8 form SM/kernels/block_fused_int8.cl:105-174,
 * 238-291): residual_inout[n] = fp16(f32(residual_inout[n]) + (W x)[n]).  M must be 1;
 * returns 0 (caller runs the unfused path) otherwise. */
int mi_linear_add(void* stream, int M, int N, int K, const void* x, const void* W, void* residual_inout);

/* fused_gate_up_silu_m1 (QW/src/utils.h:157-159; SM/kernels/block_fused_int8.cl:176-236,
 * SM/kernels/block_fused.cl:473-526): out[c] = fp16(silu(Wg x)[c] * (Wu x)[c]).  Wg and Wu
 * must be of the same kind (both fp16 or both int8); returns 0 otherwise. */
int mi_linear_gate_up_silu(void* stream, int N, int K, const void* x, const void* Wg, const void* Wu, void* out);

/* pytorch_linear_silu_gate_fused (LF/src/utils.h:140-142, LF/src/utils.cpp:1377-1406; kernel
 * LF/kernels/mlp_fused.cl:19-79): the second projection of a SwiGLU with the activation behind it.
 * gate_inout[n] holds (W1 x)[n] from an earlier mi_linear call and becomes
 * fp16((gate * sigmoid(gate)) * (W x)[n]), the product W x entering in fp32.  M = 1.  The reference
 * takes fp16 weights at K = 1024 only and returns false otherwise; here every kind and K of
 * mi_linear is taken (int8 and Q4: the scaled fp32 product). */
int mi_linear_silu_gate(void* stream, int N, int K, const void* x, const void* W, void* gate_inout);

/* dequant_int8_weight_to_fp16 (LV/src/utils.cpp:594-634, LV/kernels/lfm2_ops.cl:731-743):
 * w16[n,k] = fp16(f32(q[n,k]) * f32(scale[n])). */
int mi_dequant_int8_to_fp16(void* stream, const void* W_int8, const void* scale_fp16, int N, int K, void* w16);
/* Debug view of the Q4 unpack (UNPACK8_FROM_PIXEL, LF/kernels/gemv_m1_q4.cl:31-40):
 * w8[n,k] = nibble(n,k) - 8 as int8. */
int mi_unpack_q4_to_int8(void* stream, const void* W_q4, int N, int K, void* w8);

/* Greedy token on the device.  argmax_partial + argmax_finalize (QW/kernels/gemv_m1.cl:198-280, as
 * enqueued by dispatch_lm_head_argmax, QW/src/model.cpp:436-482, with NUM_PARTIALS = 32 and
 * work-groups of 64): token_out[0] (one int32 in device memory) = index of the greatest of the N fp16
 * logits; NaN and -inf never win, no candidate gives 0, and equal maxima are resolved as the two
 * reference kernels resolve them for the same num_partials (chunks of ceil(N / num_partials) logits;
 * strict ">" in the strided scans and in the trees makes the smaller bit-reversed work-item number
 * win: the chunk p with the lowest (bitrev6(p % 64), p), then the lowest
 * bitrev6((index - chunk start) % 64), then the lowest index).  Two launches on a stream made by
 * mi_stream_create or the null stream (512 bytes of the stream's workspace take the place of the
 * reference's two scratch buffers), one slower launch on any other stream.  The token stays on
 * the device for the next step. */
int mi_argmax_f16(void* stream, const void* logits, int N, int num_partials, void* token_out);
/* mi_linear with M = 1 followed by mi_argmax_f16 on its output: the lm_head of a greedy decode step
 * (QW/src/model.cpp:436-482).  logits [N] fp16 is written as by mi_linear, token_out as by
 * mi_argmax_f16 from those logits.  For int8 and fp16 weights with K in {576, 896, 960, 1024, 1536, 2048, 4864},
 * and for Q4 weights where the throughput GEMV runs (gemv mode 1, K in {576, 896, 960, 1024, 1536}, at
 * least 4096 rows), on a stream with a workspace, the GEMV's wavefronts also leave their best row
 * (same order of preference) and the second launch reduces those candidates, so the logits are not
 * read back; otherwise the two calls run one after the other. */
int mi_linear_argmax(void* stream, int N, int K, const void* x, const void* W, void* logits, int num_partials,
                     void* token_out);

/* mi_linear_argmax for callers that cannot allocate or depend on an allocation made for them:
 * code under HIP graph capture on a stream this library did not create, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same
 * logits and token as mi_linear_argmax; the scratch of its kernels (the wavefronts' argmax
 * candidates, 64 KiB) is an array inside the library's code object instead of a stream's
 * workspace, so it works on any stream and calls no hipMalloc / hipFree.  Each device holds one
 * such array, set up by mi_init for that device (which must have run: this call does no lazy set-up)
 * and kept until the process ends.  The first launch of a kernel loads its code, so call once before
 * capturing.  All calls on a
 * device share it: calls that overlap in time on one device (two streams, two threads) race on the
 * candidates and may return a wrong token; calls on one stream are ordered and safe.
 * N above MI_LINEAR_ARGMAX_STATIC_MAX_N is refused with an error line. */
#define MI_LINEAR_ARGMAX_STATIC_MAX_N (1 << 22)
int mi_linear_argmax_static(void* stream, int N, int K, const void* x, const void* W, void* logits,
                            int num_partials, void* token_out);

/* One call of mi_linear, for mi_linear_batch. */
typedef struct mi_linear_call {
    int M, N, K;
    const void* x;
    const void* W;
    void* out;
} mi_linear_call;

/* Enqueues calls[0..n) in order on one stream, exactly as n calls of mi_linear would: the
 * host-side loop of a decode step (Model::forward_chained_enqueue, QW/src/model.cpp:709-856,
 * issues its ~170 projections this way).  Returns the number of calls enqueued (n on success). */
int mi_linear_batch(void* stream, const mi_linear_call* calls, int n);

/* Record / replay of everything enqueued on a stream between begin and end, as a HIP graph;
 * the counterpart of the reference's recordable-queue replay of the decode step
 * (NNOPT_RECORD, QW/src/model.cpp:709-720).  Only kernel launches may be recorded: no
 * mi_malloc, mi_memcpy_* or mi_memset between begin and end.  A graph replays on the stream it
 * was recorded on and on no other: its launches use that stream's workspace (the K slices of a
 * GEMM, the argmax candidates), which only that stream's order keeps apart from the stream's
 * other work; mi_graph_launch with another stream prints an error and returns 0. */
int   mi_graph_begin(void* stream);
void* mi_graph_end(void* stream);              /* returns an executable graph or NULL */
int   mi_graph_launch(void* graph, void* stream);
int   mi_graph_destroy(void* graph);

/* Selects how M > 1 is computed: 0 (default) = MFMA GEMM with fused dequant for M >= 16, and
 * for 2 <= M < 16 where it is estimated to beat M rows of GEMV (each row streams W again; e.g. an
 * lm_head from M = 2, an MLP projection from M = 3 to 6, a projection of a million weights from
 * about 12); K not a multiple of 64 or operands not 16-byte aligned always take the batched GEMV;
 * 1 = always the batched GEMV, whose rows
 * are bit-identical to M = 1 calls (the reference's prefill loop, LF/src/model.cpp:243-250);
 * 2, 3 and 11..15 = as 0 with the kernel choice pinned (tests and tuning: results stay within
 * the same tolerance, only the speed differs): 2 = the 64 x 64 tile kernel (int8 and fp16
 * weights; fails for Q4), 3 = the wide kernel, 10 + t (t = 1..5) = the wide kernel with 32 t
 * rows of x per block, 100 s + 10 + t (s = 1..24) = the same with K cut into s slices (refused where the
 * slices' fp32 sums do not fit the stream's workspace), 30 = the kernel with 256 x 256 blocks (int8 weights only; mode 0
 * takes it by itself for contractions of several rounds of such blocks at K >= 2048), 5 = the streaming kernel for up to 64 rows of x (every kind of weights takes
 * it by itself in mode 0 up to 32 to 64 rows, depending on the shape, where it is the faster one;
 * fails for more than 64 rows).
 * Q4 weights: a weight q * scale (4 and 11 significant bits) is not an fp16 number in general.
 * Every mode but 4 feeds it to the matrix cores exactly, as two fp16 terms q * hi + q * lo with
 * scale = hi + lo, and stays within one fp16 step of the batched GEMV.  Mode 4 = as 0, but each
 * Q4 weight is rounded to the nearest fp16 number first: half the matrix work (about 1.5 times
 * faster), at an error of up to 2^-12 * sum_k |w x| on top; it changes nothing for other weights. */
void mi_set_gemm_mode(int mode);

/* Selects the M = 1 arithmetic.  0 = every GEMV evaluates the reference kernels' sum in the
 * reference's own order (results bit-identical to a literal evaluation of
 * LF/kernels/gemv_m1_q4.cl etc.).  1 (default) = as 0 for fp16 and int8, which are HBM-bound
 * either way; Q4 matrices with enough rows to fill the chip four rows to a wavefront (about 4096)
 * run a kernel that sums the same fp32 products in another order, about twice as fast, within the tolerance the reference's own tests
 * accept (cosine per layer), not bit-identical. */
void mi_set_gemv_mode(int mode);

/* The two modes above are process defaults.  This gives one stream its own: every later call
 * enqueued on `stream` computes in gemv_mode / gemm_mode whatever the defaults are, so host
 * threads that drive different streams cannot change each other's arithmetic.  -1 for a mode =
 * follow the process default; (-1, -1) forgets the stream.  No counterpart in the reference (its
 * host is single threaded and has one arithmetic). */
int mi_stream_set_modes(void* stream, int gemv_mode, int gemm_mode);

/* What mi_linear(stream, M, N, K, x, W, out) would run, without running it: 0 = GEMV (once per
 * row of x), 1 = the wide MFMA kernel with *tile_rows rows of x per block and K cut into
 * *k_slices slices (more than one slice: fp32 partial sums in the stream's workspace and a
 * reduction launch), 2 / 3 = the 64 x 64 / 128 x 128 tile kernel, 4 = the streaming kernel for up
 * to 64 rows of x (*tile_rows = M rounded up to 16, *k_slices = wavefronts, over one or several
 * blocks, that share one strip of 16 rows of W; slices over several blocks also end in a reduction
 * launch), 5 = the MFMA kernel with 256 x 256 blocks (int8 weights), -1 = bad arguments.  For tests and tuning; tile_rows and k_slices
 * may be NULL. */
int mi_linear_plan(void* stream, int M, int N, int K, const void* x, const void* W, int* tile_rows, int* k_slices);

/* Streaming-read probe: reads `bytes` (a multiple of 16 is read; src 16-byte aligned) from src
 * with the GEMV kernels' access pattern and grid and does nothing with them; timed by the caller,
 * it gives the rate the memory system sustains for a pure reader, the practical ceiling beside
 * the published peak.  The reference ships the same probe for its GEMVs (gemv_stream_buf,
 * QW/kernels/gemv_m1.cl:105-131, driven by QW/src/main.cpp:27-154).  sink: 4 bytes of device
 * memory or NULL (never written for ordinary data). */
int mi_stream_read_probe(void* stream, const void* src, size_t bytes, void* sink);

/* ---- offline tools (host) -------------------------------------------------------- */

/* quantize_row_symmetric over N rows (LF/scripts/quantize_weights.py:53-57). */
int mi_quantize_int8(const uint16_t* w_fp16, int N, int K, int8_t* q, uint16_t* scale_fp16);
/* quantize_row_q4 over N rows (LF/scripts/quantize_q4.py:62-82); 0 if K % 32 != 0. */
int mi_quantize_q4(const uint16_t* w_fp16, int N, int K, uint8_t* packed, uint16_t* scale_fp16);
/* Host fp16 codec (QW/src/utils.cpp:497-564). */
float    mi_f16_to_f32(uint16_t h);
uint16_t mi_f32_to_f16(float f);
/* Seeded synthetic tensors: n values ~ N(0, sigma) rounded to fp16.  Counter-based
 * (splitmix64 of seed and index, Box-Muller in double), so any slice can be made
 * independently and the bits do not depend on thread count. */
void mi_synth_normal_f16(uint64_t seed, double sigma, size_t n, uint16_t* out);

/* ---- weight bundles (.bin + .meta.json) ------------------------------------------ */

/* Weights::load / parse_meta_json / get_buffer (QW/src/weights.cpp:22-140, 165-254, 262-293;
 * int8 / q4_packed sizes LF/src/weights.cpp:143-148).  The .bin is mmap-ed. */
void* mi_bundle_open(const char* bin_path, const char* meta_path);
void  mi_bundle_close(void* bundle);
int   mi_bundle_count(void* bundle);
const char* mi_bundle_name(void* bundle, int index);              /* sorted-name order */
/* Returns 1 and fills the outputs if the tensor exists.  dtype: "float16" | "int8" | "q4_packed". */
int   mi_bundle_tensor(void* bundle, const char* name, const void** host_ptr, size_t* size_bytes,
                       const char** dtype, int* ndim, int64_t shape[4]);
/* Uploads every tensor to the device and registers each int8 / q4_packed tensor that has a
 * "<name>.scale" (or "<name>.scales") sibling, as LF/src/main.cpp:527-566 does. Returns the
 * number of registered weights, or -1 on error. */
int   mi_bundle_upload(void* bundle);
void* mi_bundle_device_ptr(void* bundle, const char* name);

#ifdef __cplusplus
}
#endif
#endif
