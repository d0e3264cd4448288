/*
 * CPU oracle, part 2 -- TEST INFRASTRUCTURE ONLY: one greedy decode step of a
 * Qwen2-shaped model, used as the harness for the "identical greedy token IDs over 32
 * steps" check.  Every projection goes through a caller-supplied `linear` callback, so
 * the same harness runs once with the oracle's int8 GEMV and once with the GPU library
 * behind the callback; everything that is not a projection runs here, on the CPU, in
 * both runs, so a difference in the token list can only come from the GEMV path.
 *
 * The non-projection arithmetic restates the reference's OpenCL kernels (fp16 storage
 * between kernels, fp32 inside, a*b+c contracted to fma as in oracle.c):
 *   rmsnorm_forward            QW/kernels/rmsnorm.cl (64 lanes, vec4 stride, tree reduce)
 *   bias_add_rowmajor          QW/kernels/bias_add.cl
 *   rope_apply_qk + tables     QW/kernels/rope.cl, QW/src/layers/attention.cpp:133-172
 *   gqa_attn_scores/softmax/out QW/kernels/attention.cl
 *   swiglu_inplace             QW/kernels/mlp.cl
 *   element_add                QW/kernels/utils.cl
 *   argmax_partial/finalize    QW/kernels/gemv_m1.cl:198-280 (32 partials)
 * Graph: QW/src/model.cpp:243-376, QW/src/layers/attention.cpp:336-674,
 * QW/src/layers/mlp.cpp:97-237.  The prompt is fed token by token through the same
 * step (the reference's quantised prefill is such a loop, LF/src/model.cpp:243-250).
 * Pins (tests/test_oracle_decode.py, CPU only): every function below against an fp64 numpy
 * statement of the reference kernel within one fp16 step (rmsnorm, rotary pairs and tables,
 * SwiGLU) or bit for bit (bias / element add); the attention against an fp64 grouped-query
 * attention plus probes that place each probability at an element that depends on the key's
 * index and on the query head's key/value head; the whole step (logits and the last layer's
 * q, k, v, attention output, SwiGLU output, residual stream at 20 positions) against an
 * independent fp64 forward of the graph.  The reference holds no fixture for these kernels
 * that can be used without the real checkpoints, so what is pinned is the mathematics and
 * the indexing, not a bit pattern of the reference's device.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

float orc_expf_export(float x);

typedef struct {
    int hidden, inter, n_heads, n_kv_heads, head_dim, n_layers, vocab, max_pos;
    float rms_eps, rope_theta;
    const uint16_t* embed;          /* [vocab, hidden] fp16 */
    const uint16_t* final_norm;     /* [hidden] */
    const uint16_t* const* in_norm;     /* [n_layers] -> [hidden] */
    const uint16_t* const* post_norm;
    const uint16_t* const* bq;          /* [n_heads*head_dim] */
    const uint16_t* const* bk;          /* [n_kv_heads*head_dim] */
    const uint16_t* const* bv;
    const int8_t* const* w8;            /* [n_layers*7 + 1]: q,k,v,o,gate,up,down per layer, then lm_head */
    const uint16_t* const* wscale;      /* matching fp16 row scales */
} orc_model;

typedef void (*orc_linear_fn)(void* ctx, int index, const uint16_t* x, uint16_t* y);

typedef struct {
    orc_model m;
    uint16_t *kc, *vc;              /* [n_layers][max_pos][kv_dim] */
    uint16_t *cosT, *sinT;          /* [max_pos][head_dim] */
    uint16_t *h, *xn, *q, *k, *v, *attn, *proj, *gate, *up, *logits, *scores;
    int threads;
} orc_decoder;

static inline float H(uint16_t x) { return orc_f16_to_f32(x); }
static inline uint16_t F(float x) { return orc_f32_to_f16(x); }

static void rmsnorm(const uint16_t* x, const uint16_t* w, uint16_t* out, int cols, float eps)
{
    float part[64];
    int c4n = cols >> 2;
    for (int lid = 0; lid < 64; ++lid) {
        float acc = 0.0f;
        for (int c4 = lid; c4 < c4n; c4 += 64) {
            float v0 = H(x[4 * c4]), v1 = H(x[4 * c4 + 1]), v2 = H(x[4 * c4 + 2]), v3 = H(x[4 * c4 + 3]);
            float d = v0 * v0;
            d = fmaf(v1, v1, d); d = fmaf(v2, v2, d); d = fmaf(v3, v3, d);
            acc = acc + d;
        }
        for (int c = c4n * 4 + lid; c < cols; c += 64) acc = fmaf(H(x[c]), H(x[c]), acc);
        part[lid] = acc;
    }
    for (int s = 32; s > 0; s >>= 1)
        for (int t = 0; t < s; ++t) part[t] = part[t] + part[t + s];
    float inv = 1.0f / sqrtf(part[0] / (float)cols + eps);
    for (int c = 0; c < cols; ++c) out[c] = F((H(x[c]) * inv) * H(w[c]));
}

static void bias_add(uint16_t* out, const uint16_t* b, int n)
{
    for (int i = 0; i < n; ++i) out[i] = F(H(out[i]) + H(b[i]));
}

static void element_add(uint16_t* a, const uint16_t* b, int n)
{
    for (int i = 0; i < n; ++i) a[i] = F(H(a[i]) + H(b[i]));
}

static void rope(uint16_t* buf, int heads, int D, const uint16_t* cosr, const uint16_t* sinr)
{
    int hd2 = D / 2;
    for (int h = 0; h < heads; ++h)
        for (int i = 0; i < hd2; ++i) {
            float x1 = H(buf[h * D + i]), x2 = H(buf[h * D + i + hd2]);
            float c = H(cosr[i]), s = H(sinr[i]);
            float o1 = fmaf(x1, c, -(x2 * s));
            float o2 = fmaf(x2, c, x1 * s);
            buf[h * D + i] = F(o1);
            buf[h * D + i + hd2] = F(o2);
        }
}

/* gqa_attn_scores + gqa_softmax + gqa_attn_out for one query row (QW/kernels/attention.cl:43-101,
 * 109-135, 148-186): q [n_heads*D], kc / vc [>= seq_k][n_kv_heads*D], scores scratch
 * [n_heads][score_stride], out [n_heads*D]. */
static void gqa_attention(const uint16_t* q, const uint16_t* kc, const uint16_t* vc, uint16_t* scores,
                          uint16_t* out, int n_heads, int n_kv_heads, int D, int score_stride, int seq_k)
{
    int kvd = n_kv_heads * D, nrep = n_heads / n_kv_heads;
    float scale = 1.0f / sqrtf((float)D);
    for (int qh = 0; qh < n_heads; ++qh) {
        int kvh = qh / nrep;
        uint16_t* sc = scores + (size_t)qh * score_stride;
        for (int tk = 0; tk < seq_k; ++tk) {                   /* gqa_attn_scores */
            float acc = 0.0f;
            const uint16_t* qv = q + qh * D;
            const uint16_t* kv = kc + (size_t)tk * kvd + kvh * D;
            for (int d4 = 0; d4 < D / 4; ++d4) {
                float t = H(qv[4 * d4]) * H(kv[4 * d4]);
                t = fmaf(H(qv[4 * d4 + 1]), H(kv[4 * d4 + 1]), t);
                t = fmaf(H(qv[4 * d4 + 2]), H(kv[4 * d4 + 2]), t);
                t = fmaf(H(qv[4 * d4 + 3]), H(kv[4 * d4 + 3]), t);
                acc = acc + t;
            }
            sc[tk] = F(acc * scale);
        }
        float maxv = -3.402823466e+38f;                        /* gqa_softmax */
        for (int c = 0; c < seq_k; ++c) { float v = H(sc[c]); if (v > maxv) maxv = v; }
        float sum = 0.0f;
        for (int c = 0; c < seq_k; ++c) {
            float e = orc_expf_export(H(sc[c]) - maxv);
            sum = sum + e;
            sc[c] = F(e);
        }
        float inv = 1.0f / (sum + 1e-20f);
        for (int c = 0; c < seq_k; ++c) sc[c] = F(H(sc[c]) * inv);
        for (int e = 0; e < D; ++e) {                          /* gqa_attn_out */
            float acc = 0.0f;
            for (int tk = 0; tk < seq_k; ++tk)
                acc = fmaf(H(sc[tk]), H(vc[(size_t)tk * kvd + kvh * D + e]), acc);
            out[qh * D + e] = F(acc);
        }
    }
}

static void attention(orc_decoder* d, int layer, int pos)
{
    const orc_model* m = &d->m;
    int kvd = m->n_kv_heads * m->head_dim;
    gqa_attention(d->q, d->kc + (size_t)layer * m->max_pos * kvd, d->vc + (size_t)layer * m->max_pos * kvd,
                  d->scores, d->attn, m->n_heads, m->n_kv_heads, m->head_dim, m->max_pos, pos + 1);
}

static void swiglu(uint16_t* gate, const uint16_t* up, int n)
{
    for (int i = 0; i < n; ++i) {
        float g = H(gate[i]), u = H(up[i]);
        float sig = 1.0f / (1.0f + orc_expf_export(-g));
        gate[i] = F((g * sig) * u);
    }
}

/* The pieces above one at a time, for the tests that pin them against independent statements
 * (tests/test_oracle_decode.py). */
void orc_rmsnorm(const uint16_t* x, const uint16_t* w, uint16_t* out, int cols, float eps) { rmsnorm(x, w, out, cols, eps); }
void orc_bias_add(uint16_t* out, const uint16_t* b, int n) { bias_add(out, b, n); }
void orc_element_add(uint16_t* a, const uint16_t* b, int n) { element_add(a, b, n); }
void orc_rope(uint16_t* buf, int heads, int D, const uint16_t* cosr, const uint16_t* sinr) { rope(buf, heads, D, cosr, sinr); }
void orc_swiglu(uint16_t* gate, const uint16_t* up, int n) { swiglu(gate, up, n); }
void orc_gqa_attention(const uint16_t* q, const uint16_t* kc, const uint16_t* vc, uint16_t* scores, uint16_t* out,
                       int n_heads, int n_kv_heads, int D, int score_stride, int seq_k)
{
    gqa_attention(q, kc, vc, scores, out, n_heads, n_kv_heads, D, score_stride, seq_k);
}

/* argmax_partial with NP partials of 64 lanes, then argmax_finalize
 * (QW/kernels/gemv_m1.cl:198-280); NP <= 4096. */
int orc_argmax_f16(const uint16_t* x, int N, int NP)
{
    static _Thread_local float pv[4096]; static _Thread_local int pi[4096];
    if (NP < 1 || NP > 4096 || N < 1) return -1;
    int chunk = (N + NP - 1) / NP;
    for (int wg = 0; wg < NP; ++wg) {
        int start = wg * chunk, end = start + chunk < N ? start + chunk : N;
        float lv[64]; int li[64];
        for (int t = 0; t < 64; ++t) {
            float bv = -3.402823466e+38f; int bi = start < N ? start : 0;
            for (int i = start + t; i < end; i += 64) { float v = H(x[i]); if (v > bv) { bv = v; bi = i; } }
            lv[t] = bv; li[t] = bi;
        }
        for (int s = 32; s > 0; s >>= 1)
            for (int t = 0; t < s; ++t)
                if (lv[t + s] > lv[t]) { lv[t] = lv[t + s]; li[t] = li[t + s]; }
        pv[wg] = lv[0]; pi[wg] = li[0];
    }
    float lv[64]; int li[64];
    for (int t = 0; t < 64; ++t) {
        float bv = -3.402823466e+38f; int bi = 0;
        for (int i = t; i < NP; i += 64) { float v = pv[i]; if (v > bv) { bv = v; bi = pi[i]; } }
        lv[t] = bv; li[t] = bi;
    }
    for (int s = 32; s > 0; s >>= 1)
        for (int t = 0; t < s; ++t)
            if (lv[t + s] > lv[t]) { lv[t] = lv[t + s]; li[t] = li[t + s]; }
    return li[0];
}

static void linear(orc_decoder* d, orc_linear_fn fn, void* ctx, int index, int N, int K,
                   const uint16_t* x, uint16_t* y)
{
    if (fn) fn(ctx, index, x, y);
    else orc_gemv_i8(x, d->m.w8[index], d->m.wscale[index], y, N, K, d->threads);
}

/* Rotary tables [max_pos][D], both halves of a row hold the same D/2 values
 * (QW/src/layers/attention.cpp:147-160: fp32 pow / cos / sin, then one rounding to fp16). */
void orc_rope_tables(int max_pos, int D, float theta, uint16_t* cosT, uint16_t* sinT)
{
    for (int t = 0; t < max_pos; ++t)
        for (int i = 0; i < D / 2; ++i) {
            float exponent = (2.0f * (float)i) / (float)D;
            float inv_freq = powf(theta, -exponent);
            float angle = (float)t * inv_freq;
            uint16_t c = F(cosf(angle)), s = F(sinf(angle));
            cosT[(size_t)t * D + i] = c; cosT[(size_t)t * D + i + D / 2] = c;
            sinT[(size_t)t * D + i] = s; sinT[(size_t)t * D + i + D / 2] = s;
        }
}

void* orc_decoder_new(const orc_model* m, int threads)
{
    orc_decoder* d = (orc_decoder*)calloc(1, sizeof *d);
    d->m = *m;
    d->threads = threads;
    int D = m->head_dim, kvd = m->n_kv_heads * D, qd = m->n_heads * D;
    size_t cache = (size_t)m->n_layers * m->max_pos * kvd;
    d->kc = (uint16_t*)calloc(cache, 2);
    d->vc = (uint16_t*)calloc(cache, 2);
    d->cosT = (uint16_t*)malloc((size_t)m->max_pos * D * 2);
    d->sinT = (uint16_t*)malloc((size_t)m->max_pos * D * 2);
    orc_rope_tables(m->max_pos, D, m->rope_theta, d->cosT, d->sinT);
    d->h = (uint16_t*)malloc(m->hidden * 2);   d->xn = (uint16_t*)malloc(m->hidden * 2);
    d->q = (uint16_t*)malloc(qd * 2);          d->k = (uint16_t*)malloc(kvd * 2);
    d->v = (uint16_t*)malloc(kvd * 2);         d->attn = (uint16_t*)malloc(qd * 2);
    d->proj = (uint16_t*)malloc(m->hidden * 2);
    d->gate = (uint16_t*)malloc(m->inter * 2); d->up = (uint16_t*)malloc(m->inter * 2);
    d->logits = (uint16_t*)malloc((size_t)m->vocab * 2);
    d->scores = (uint16_t*)malloc((size_t)m->n_heads * m->max_pos * 2);
    return d;
}

void orc_decoder_free(void* p)
{
    orc_decoder* d = (orc_decoder*)p;
    if (!d) return;
    free(d->kc); free(d->vc); free(d->cosT); free(d->sinT); free(d->h); free(d->xn); free(d->q);
    free(d->k); free(d->v); free(d->attn); free(d->proj); free(d->gate); free(d->up);
    free(d->logits); free(d->scores); free(d);
}

/* Runs one token at position pos, returns the greedy next token; *margin (if not null)
 * receives logit(top1) - logit(top2) in fp32 of the fp16 logits. */
int orc_decoder_step(void* p, int token, int pos, orc_linear_fn fn, void* ctx, float* margin)
{
    orc_decoder* d = (orc_decoder*)p;
    const orc_model* m = &d->m;
    int Hd = m->hidden, D = m->head_dim, qd = m->n_heads * D, kvd = m->n_kv_heads * D;
    if (pos < 0 || pos >= m->max_pos || token < 0 || token >= m->vocab) return -1;
    memcpy(d->h, m->embed + (size_t)token * Hd, (size_t)Hd * 2);
    for (int l = 0; l < m->n_layers; ++l) {
        int b = l * 7;
        rmsnorm(d->h, m->in_norm[l], d->xn, Hd, m->rms_eps);
        linear(d, fn, ctx, b + 0, qd, Hd, d->xn, d->q);   bias_add(d->q, m->bq[l], qd);
        linear(d, fn, ctx, b + 1, kvd, Hd, d->xn, d->k);  bias_add(d->k, m->bk[l], kvd);
        linear(d, fn, ctx, b + 2, kvd, Hd, d->xn, d->v);  bias_add(d->v, m->bv[l], kvd);
        rope(d->q, m->n_heads, D, d->cosT + (size_t)pos * D, d->sinT + (size_t)pos * D);
        rope(d->k, m->n_kv_heads, D, d->cosT + (size_t)pos * D, d->sinT + (size_t)pos * D);
        memcpy(d->kc + ((size_t)l * m->max_pos + pos) * kvd, d->k, (size_t)kvd * 2);
        memcpy(d->vc + ((size_t)l * m->max_pos + pos) * kvd, d->v, (size_t)kvd * 2);
        attention(d, l, pos);
        linear(d, fn, ctx, b + 3, Hd, qd, d->attn, d->proj);
        element_add(d->h, d->proj, Hd);
        rmsnorm(d->h, m->post_norm[l], d->xn, Hd, m->rms_eps);
        linear(d, fn, ctx, b + 4, m->inter, Hd, d->xn, d->gate);
        linear(d, fn, ctx, b + 5, m->inter, Hd, d->xn, d->up);
        swiglu(d->gate, d->up, m->inter);
        linear(d, fn, ctx, b + 6, Hd, m->inter, d->gate, d->proj);
        element_add(d->h, d->proj, Hd);
    }
    rmsnorm(d->h, m->final_norm, d->xn, Hd, m->rms_eps);
    linear(d, fn, ctx, m->n_layers * 7, m->vocab, Hd, d->xn, d->logits);
    int best = orc_argmax_f16(d->logits, m->vocab, 32);
    if (margin) {
        float top = H(d->logits[best]), second = -3.402823466e+38f;
        for (int i = 0; i < m->vocab; ++i)
            if (i != best && H(d->logits[i]) > second) second = H(d->logits[i]);
        *margin = top - second;
    }
    return best;
}

const uint16_t* orc_decoder_logits(void* p) { return ((orc_decoder*)p)->logits; }

/* Activations left by the last step: 0 = residual stream h, 1 = q (after bias and rotary, last
 * layer), 2 = k, 3 = v, 4 = attention output, 5 = swiglu(gate, up), 6 / 7 = the rotary cos / sin
 * tables [max_pos][head_dim]; for comparing a device implementation buffer by buffer. */
const uint16_t* orc_decoder_buffer(void* p, int which)
{
    orc_decoder* d = (orc_decoder*)p;
    switch (which) {
        case 0: return d->h;
        case 1: return d->q;
        case 2: return d->k;
        case 3: return d->v;
        case 4: return d->attn;
        case 5: return d->gate;
        case 6: return d->cosT;
        case 7: return d->sinT;
        default: return NULL;
    }
}
