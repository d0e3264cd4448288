/* mi_decode.h - a greedy decode step of a Qwen2-shaped model that stays on the device.
 *
 * The projections and the lm_head go through mi_linear / mi_linear_batch / mi_linear_argmax
 * (mi_linear.h); this header adds the harness around them that a decode loop needs to run without
 * the host: embedding lookup, RMSNorm, q/k/v bias, rotary embedding + KV-cache write, single-query
 * grouped-query attention, SwiGLU, residual adds.  It stands for Model::forward_greedy and the
 * decode loop of QW/src/model.cpp:243-376, 387-500, 709-856 with QW/src/layers/attention.cpp:336-674
 * and QW/src/layers/mlp.cpp:97-237, restricted to batch 1, one new token per step.
 *
 * Position and token are device state (the reference keeps {start_pos, seq_k} in a counter buffer
 * read by the kernels, QW/src/model.cpp:490-500): mi_decoder_step enqueues the same launches with
 * the same arguments at every position, so it can be captured once (mi_graph_begin / mi_graph_end)
 * and replayed for every token.
 */
#ifndef MI_DECODE_H
#define MI_DECODE_H

#ifdef __cplusplus
extern "C" {
#endif

/* MODEL_CONFIG of QW/src/model_config.h:12-34. */
typedef struct mi_decoder_config {
    int hidden, inter, n_heads, n_kv_heads, head_dim, n_layers, vocab, max_pos;
    float rms_eps, rope_theta;
} mi_decoder_config;

/* Device pointers, caller-owned, alive as long as the decoder.  Norm weights and biases are fp16
 * vectors; embed is fp16 [vocab, hidden]; projection weights are fp16 [N, K] or quantised and
 * registered (mi_register_int8_weight / mi_register_q4_weight).  Arrays have n_layers entries.
 * Norm weights and projection weights must be 16-byte aligned (anything from mi_malloc is). */
typedef struct mi_decoder_weights {
    const void* embed;
    const void* final_norm;
    const void* lm_head;                 /* [vocab, hidden] */
    const void* const* in_norm;          /* input_layernorm          [hidden] */
    const void* const* post_norm;        /* post_attention_layernorm [hidden] */
    const void* const* bq;               /* [n_heads * head_dim] */
    const void* const* bk;               /* [n_kv_heads * head_dim] */
    const void* const* bv;
    const void* const* wq;               /* [n_heads * head_dim, hidden] */
    const void* const* wk;               /* [n_kv_heads * head_dim, hidden] */
    const void* const* wv;
    const void* const* wo;               /* [hidden, n_heads * head_dim] */
    const void* const* wgate;            /* [inter, hidden] */
    const void* const* wup;
    const void* const* wdown;            /* [hidden, inter] */
} mi_decoder_weights;

/* Allocates the KV caches ([n_layers, max_pos, n_kv_heads * head_dim] fp16 each), the activation
 * buffers, the rotary tables (QW/src/layers/attention.cpp:133-172) and the device state
 * (position 0, token 0).  max_pos <= 8192.  NULL on failure. */
void* mi_decoder_create(const mi_decoder_config* cfg, const mi_decoder_weights* weights);
int   mi_decoder_destroy(void* decoder);

/* Device state := {pos, token}; synchronises the stream.  The KV cache rows below pos are kept. */
int   mi_decoder_reset(void* decoder, void* stream, int pos, int token);
/* Overrides the token the next step consumes (prompt feeding); synchronises the stream. */
int   mi_decoder_set_token(void* decoder, void* stream, int token);

/* Enqueues one step: consumes the device token at the device position, writes the KV rows of that
 * position, leaves the greedy next token as the device token and advances the position.  Nothing is
 * allocated or synchronised; may be captured into a graph.  A step at position max_pos - 1 is the
 * last valid one (later steps clamp the position and overwrite that row). */
int   mi_decoder_step(void* decoder, void* stream);

/* A prompt at once: Model::forward with seq_len = n_tokens (QW/src/model.cpp:243-376), where every
 * pytorch_linear is an M = n_tokens call (QW/src/utils.cpp:785-796) and so reaches the GEMM of
 * mi_linear.  Consumes tokens[0 .. n_tokens) (host memory) at positions pos0 .. pos0 + n_tokens - 1,
 * writes their KV rows (rows below pos0 are read as they are), leaves the greedy token after the
 * last one as the device token and pos0 + n_tokens as the device position: the state n_tokens
 * calls of mi_decoder_step with the tokens forced would leave.  The cache rows and the logits
 * are those of such steps bit for bit when the M > 1 projections run as rows of GEMV
 * (mi_set_gemm_mode(1), the reference's quantised prefill, LF/src/model.cpp:243-250), and within
 * the GEMM's tolerance of them on the matrix cores.  pos0 + n_tokens <= max_pos.  The first prompt
 * makes device copies of every layer's q, k, v and gate, up matrices stacked into one matrix each
 * (the reference's stacked qkv, QW/src/layers/attention.cpp:414; as much memory again as those
 * matrices), so that the projections of one input are one GEMM; it, and any longer prompt later,
 * allocates the prompt's activation rows (about 40 KB per token at Qwen2.5-0.5B widths).  Not for
 * graph capture.  mi_decoder_buffer(0) afterwards holds the residual
 * stream of the last position; buffers 1 .. 5 are left as they were. */
int   mi_decoder_prefill(void* decoder, void* stream, const int* tokens, int n_tokens, int pos0);
/* Does now what the first (or a longer) prompt would otherwise do inside mi_decoder_prefill: makes
 * the stacked copies of the projection matrices and the activation rows for prompts of up to
 * max_tokens tokens, and waits for the copies.  After it, mi_decoder_prefill with n_tokens <=
 * max_tokens allocates nothing, frees nothing and waits for nothing (it still copies the token ids
 * from host memory, so it stays out of graph capture).  No counterpart in the reference, whose
 * layers allocate their activation buffers on first use (QW/src/layers/mlp.cpp:228-232). */
int   mi_decoder_reserve_prompt(void* decoder, void* stream, int max_tokens);

/* Reads the device state back (synchronises the stream). */
int   mi_decoder_read(void* decoder, void* stream, int* pos, int* token);
/* An arithmetic mode of the attention inside mi_decoder_step, for long contexts.  0 or 1 (default): the
 * launch that keeps the reference's order of operations (QW/kernels/attention.cl: one work-group per
 * head, the sum of the exponentials and every output element's sum over the keys in key order), bit
 * for bit; its time grows by about 24 ns per position and layer.  2..32: the keys of a head are taken
 * by that many blocks, each with its own maximum and sums, and a second launch merges them: the same
 * real numbers summed in another order, without the fp16 roundings of the probabilities, within
 * max-abs/rel 1e-3 and cosine 0.9999 of the default, not bit-identical; one launch more per layer.
 * head_dim 64 or 128.  Measured on Qwen2.5-0.5B shapes: 16 is the fastest up to about 2000 positions, 32 beyond
 * (position 4000: 594 us per step against 659 with 16 and 2723 in the reference's order); below about 150
 * positions the default is faster.  Allocates once; call it between steps, never under graph capture (a graph
 * captured afterwards keeps the mode it was captured in).  No counterpart in the reference. */
int   mi_decoder_set_attention_splits(void* decoder, int splits);
/* fp16 [vocab] logits of the last step, in device memory. */
const void* mi_decoder_logits(void* decoder);
/* Activations left by the last step, fp16 in device memory, for comparing implementations buffer
 * by buffer: which = 0 residual stream [hidden], 1 q after bias and rotary [n_heads*head_dim],
 * 2 k, 3 v [n_kv_heads*head_dim], 4 attention output [n_heads*head_dim], 5 swiglu(gate, up)
 * [intermediate], all of the last layer; 6 / 7 the rotary cos / sin tables [max_pos*head_dim].
 * NULL for any other value. */
const void* mi_decoder_buffer(void* decoder, int which);

#ifdef __cplusplus
}
#endif
#endif
