/*
 * lpp_oracle.c -- CPU oracle for the Lighter++ batch-1 decode path.
 *
 * TEST INFRASTRUCTURE ONLY (see lpp_oracle.h).  Every function restates, in
 * plain C, the arithmetic of one function of the reference's CPU path, in the
 * same operation order, so that a build with the reference's own flags
 * (-O3, no fast-math, no FMA contraction) is bit-identical to it.  Citations
 * are to files under the reference's src/ directory.
 */
#include "lpp_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* binary16 <-> binary32                                                    */
/* ------------------------------------------------------------------------ */

/* loader.cpp:346-379: widen one IEEE half.  Zero keeps its sign, subnormals are
 * renormalised, exponent 31 maps to Inf/NaN with the payload shifted up. */
float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    int      e    = (h >> 10) & 0x1f;
    uint32_t m    = h & 0x3ffu;
    uint32_t bits;
    if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e == 0 && m == 0) {
        bits = sign;
    } else {
        if (e == 0) {              /* subnormal: shift until the hidden bit shows */
            e = 1;
            while (!(m & 0x400u)) { m <<= 1; --e; }
            m &= 0x3ffu;
        }
        bits = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* Round-to-nearest-even narrowing; what the GPU operator API does to K/V on
 * their way into the cache (scatter_kv.cu:17-18 uses __float2half). */
uint16_t orc_f32_to_f16_rn(float f)
{
    uint32_t x;
    memcpy(&x, &f, sizeof x);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u)                          /* Inf / NaN */
        return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
    if (ax >= 0x477ff000u)                          /* rounds to >= 65520 -> Inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u)                           /* <= 2^-25 rounds to zero */
        return sign;
    int e = (int)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;      /* 24-bit significand */
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;  /* bits dropped */
    uint32_t keep = m >> shift;
    uint32_t rem  = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) ++keep;
    if (e < -14)                                    /* subnormal (may carry into normal) */
        return (uint16_t)(sign | keep);
    /* keep holds hidden bit at 0x400; adding the exponent lets a mantissa
     * carry bump the exponent naturally. */
    return (uint16_t)(sign | (uint16_t)(((uint32_t)(e + 15 - 1) << 10) + keep));
}

static float        g_f16_lut[65536];
static volatile int g_f16_lut_ready = 0;

static const float *f16_lut(void)
{
    if (!g_f16_lut_ready) {
        for (uint32_t i = 0; i < 65536u; ++i) g_f16_lut[i] = orc_f16_to_f32((uint16_t)i);
        g_f16_lut_ready = 1;
    }
    return g_f16_lut;
}

/* ------------------------------------------------------------------------ */
/* ops.cpp                                                                  */
/* ------------------------------------------------------------------------ */

/* ops.cpp:9-17: out[i] = sum_k x[k]*w[i][k], one fp32 accumulator, k ascending. */
void orc_naive_matmul(float *out, const float *x, const float *w, int n, int d)
{
    for (int r = 0; r < n; ++r) {
        const float *row = w + (size_t)r * (size_t)d;
        float acc = 0.0f;
        for (int c = 0; c < d; ++c) acc += x[c] * row[c];
        out[r] = acc;
    }
}

/* Same sum with binary16 weights widened exactly per element; equals
 * orc_naive_matmul on the widened copy the reference's GGUF loader makes
 * (loader.cpp:391-395). */
void orc_matmul_f16w(float *out, const float *x, const uint16_t *w, int n, int d)
{
    const float *lut = f16_lut();
    for (int r = 0; r < n; ++r) {
        const uint16_t *row = w + (size_t)r * (size_t)d;
        float acc = 0.0f;
        for (int c = 0; c < d; ++c) acc += x[c] * lut[row[c]];
        out[r] = acc;
    }
}

/* ops.cpp:20-32: mean of squares, + 1e-5f, reciprocal square root as 1/sqrtf,
 * then (x*scale)*gain left to right.  out may alias x. */
void orc_rmsnorm(float *out, const float *x, const float *weight, int n)
{
    float ms = 0.0f;
    for (int i = 0; i < n; ++i) ms += x[i] * x[i];
    ms /= n;
    ms += 1e-5f;
    float scale = 1.0f / sqrtf(ms);
    for (int i = 0; i < n; ++i) out[i] = x[i] * scale * weight[i];
}

/* ops.cpp:34-54: adjacent pairs (i, i+1); frequency index is i mod head_size;
 * angle = (float)pos * (1/powf(base, idx/head_size)); k rotated while i < kv_dim. */
void orc_rope(float *q, float *k, int pos, int dim, int kv_dim, int head_size,
              float rope_base)
{
    for (int i = 0; i < dim; i += 2) {
        int   idx   = i % head_size;
        float freq  = 1.0f / powf(rope_base, idx / (float)head_size);
        float angle = pos * freq;
        float c = cosf(angle);
        float s = sinf(angle);
        float a = q[i], b = q[i + 1];
        q[i]     = a * c - b * s;
        q[i + 1] = a * s + b * c;
        if (i < kv_dim) {
            float ka = k[i], kb = k[i + 1];
            k[i]     = ka * c - kb * s;
            k[i + 1] = ka * s + kb * c;
        }
    }
}

/* ops.cpp:56-75: first-element-seeded max, expf(x-max) summed ascending, true
 * division by the sum. */
void orc_softmax(float *x, int size)
{
    float top = x[0];
    for (int i = 1; i < size; ++i)
        if (x[i] > top) top = x[i];
    float total = 0.0f;
    for (int i = 0; i < size; ++i) {
        x[i] = expf(x[i] - top);
        total += x[i];
    }
    for (int i = 0; i < size; ++i) x[i] = x[i] / total;
}

/* ops.cpp:78-87: (g * (1/(1+expf(-g)))) * u; hb may alias h1 or h3. */
void orc_swiglu(float *hb, const float *h1, const float *h3, int size)
{
    for (int i = 0; i < size; ++i) {
        float g = h1[i];
        float sigma = 1.0f / (1.0f + expf(-g));
        hb[i] = (g * sigma) * h3[i];
    }
}

/* ------------------------------------------------------------------------ */
/* model.cpp                                                                */
/* ------------------------------------------------------------------------ */

static int kv_dim_of(const orc_config *p) { return (p->dim * p->n_kv_heads) / p->n_heads; }

/* model.cpp:18-51 (host buffers only; zero-initialised like calloc there). */
int orc_state_alloc(orc_state *s, const orc_config *p)
{
    int kv_dim = kv_dim_of(p);
    size_t cache = (size_t)p->n_layers * (size_t)p->seq_len * (size_t)kv_dim;
    memset(s, 0, sizeof *s);
    s->x   = calloc((size_t)p->dim, sizeof(float));
    s->xb  = calloc((size_t)p->dim, sizeof(float));
    s->xb2 = calloc((size_t)p->dim, sizeof(float));
    s->q   = calloc((size_t)p->dim, sizeof(float));
    s->k   = calloc((size_t)kv_dim, sizeof(float));
    s->v   = calloc((size_t)kv_dim, sizeof(float));
    s->hb  = calloc((size_t)p->hidden_dim, sizeof(float));
    s->he  = calloc((size_t)p->hidden_dim, sizeof(float));
    s->att = calloc((size_t)p->n_heads * (size_t)p->seq_len, sizeof(float));
    s->logits = calloc((size_t)p->vocab_size, sizeof(float));
    s->key_cache   = calloc(cache, sizeof(float));
    s->value_cache = calloc(cache, sizeof(float));
    if (!s->x || !s->xb || !s->xb2 || !s->q || !s->k || !s->v || !s->hb || !s->he ||
        !s->att || !s->logits || !s->key_cache || !s->value_cache) {
        orc_state_free(s);
        return -1;
    }
    return 0;
}

void orc_state_free(orc_state *s)
{
    free(s->x); free(s->xb); free(s->xb2); free(s->q); free(s->k); free(s->v);
    free(s->hb); free(s->he); free(s->att); free(s->logits);
    free(s->key_cache); free(s->value_cache);
    memset(s, 0, sizeof *s);
}

static void matmul_any(float *out, const float *x, const void *w, size_t elem_off,
                       int n, int d, int is_f16)
{
    if (is_f16) orc_matmul_f16w(out, x, (const uint16_t *)w + elem_off, n, d);
    else        orc_naive_matmul(out, x, (const float *)w + elem_off, n, d);
}

/* model.cpp:121-127 and the CPU branch :163-202. */
void orc_attention(orc_state *s, const orc_weights *w, const orc_config *p,
                   int layer, int pos)
{
    const int dim = p->dim;
    const int kv_dim = kv_dim_of(p);
    const int hs = dim / p->n_heads;
    const int group = p->n_heads / p->n_kv_heads;
    const size_t off_q  = (size_t)layer * (size_t)dim * (size_t)dim;
    const size_t off_kv = (size_t)layer * (size_t)kv_dim * (size_t)dim;
    const size_t head_span  = (size_t)p->seq_len * (size_t)hs;      /* one KV head's cache */
    const size_t layer_span = (size_t)kv_dim * (size_t)p->seq_len;  /* one layer's cache   */

    matmul_any(s->q, s->xb, w->wq, off_q,  dim,    dim, w->w_is_f16);
    matmul_any(s->k, s->xb, w->wk, off_kv, kv_dim, dim, w->w_is_f16);
    matmul_any(s->v, s->xb, w->wv, off_kv, kv_dim, dim, w->w_is_f16);

    orc_rope(s->q, s->k, pos, dim, kv_dim, hs, p->rope_base);

    /* :171-176  cache[layer][kvh][pos][0..hs) <- k,v[kvh*hs ..] */
    for (int kvh = 0; kvh < p->n_kv_heads; ++kvh) {
        size_t dst = (size_t)layer * layer_span + (size_t)kvh * head_span + (size_t)pos * (size_t)hs;
        const float *ksrc = s->k + (size_t)kvh * hs;
        const float *vsrc = s->v + (size_t)kvh * hs;
        if (s->kv_round_f16) {
            for (int i = 0; i < hs; ++i) {
                s->key_cache[dst + i]   = orc_f16_to_f32(orc_f32_to_f16_rn(ksrc[i]));
                s->value_cache[dst + i] = orc_f16_to_f32(orc_f32_to_f16_rn(vsrc[i]));
            }
        } else {
            memcpy(s->key_cache + dst,   ksrc, (size_t)hs * sizeof(float));
            memcpy(s->value_cache + dst, vsrc, (size_t)hs * sizeof(float));
        }
    }

    /* :178-199  per query head: scores over 0..pos, scale, softmax, weighted V sum */
    for (int h = 0; h < p->n_heads; ++h) {
        const float *qh = s->q + (size_t)h * hs;
        size_t base = (size_t)layer * layer_span + (size_t)(h / group) * head_span;
        const float *kc = s->key_cache + base;
        const float *vc = s->value_cache + base;
        float *att = s->att + (size_t)h * (size_t)p->seq_len;

        orc_naive_matmul(att, qh, kc, pos + 1, hs);
        float inv_sqrt = 1.0f / sqrtf(hs);
        for (int t = 0; t <= pos; ++t) att[t] *= inv_sqrt;
        orc_softmax(att, pos + 1);

        float *oh = s->xb + (size_t)h * hs;
        memset(oh, 0, (size_t)hs * sizeof(float));
        for (int t = 0; t <= pos; ++t) {
            float a = att[t];
            const float *vt = vc + (size_t)t * hs;
            for (int i = 0; i < hs; ++i) oh[i] += vt[i] * a;
        }
    }

    matmul_any(s->xb2, s->xb, w->wo, off_q, dim, dim, w->w_is_f16);
}

/* model.cpp:205-210 and the CPU branch :229-239. */
void orc_transformer_block(orc_state *s, const orc_weights *w,
                           const orc_config *p, int layer, int pos)
{
    const int dim = p->dim, hidden = p->hidden_dim;
    const size_t off_ffn  = (size_t)layer * (size_t)hidden * (size_t)dim;
    const size_t off_norm = (size_t)layer * (size_t)dim;

    orc_rmsnorm(s->xb, s->x, w->rms_att_weight + off_norm, dim);
    orc_attention(s, w, p, layer, pos);
    for (int i = 0; i < dim; ++i) s->x[i] += s->xb2[i];

    orc_rmsnorm(s->xb, s->x, w->rms_ffn_weight + off_norm, dim);
    matmul_any(s->hb, s->xb, w->w1, off_ffn, hidden, dim, w->w_is_f16);
    matmul_any(s->he, s->xb, w->w3, off_ffn, hidden, dim, w->w_is_f16);
    orc_swiglu(s->hb, s->hb, s->he, hidden);
    matmul_any(s->xb2, s->hb, w->w2, off_ffn, dim, hidden, w->w_is_f16);
    for (int i = 0; i < dim; ++i) s->x[i] += s->xb2[i];
}

/* model.cpp:342-345 and the CPU branch :373-380. */
void orc_forward_logits(int token, int pos, orc_state *s, const orc_weights *w,
                        const orc_config *p)
{
    const int dim = p->dim;
    memcpy(s->x, w->token_embedding_table + (size_t)token * (size_t)dim,
           (size_t)dim * sizeof(float));
    for (int layer = 0; layer < p->n_layers; ++layer)
        orc_transformer_block(s, w, p, layer, pos);
    orc_rmsnorm(s->x, s->x, w->rms_final_weight, dim);
    matmul_any(s->logits, s->x, w->w_cls, 0, p->vocab_size, dim, w->w_is_f16);
}

/* model.cpp:258-270: one pass over the window in order, so a token that occurs
 * k times is penalised k times; positive logits are divided, the rest
 * multiplied; ids outside [0, vocab) are skipped. */
static void apply_penalty(float *logits, int vocab, float penalty,
                          const int *history, int history_len)
{
    if (!(penalty > 1.0f) || !history || history_len <= 0) return;
    for (int i = 0; i < history_len; ++i) {
        int t = history[i];
        if (t < 0 || t >= vocab) continue;
        if (logits[t] > 0) logits[t] /= penalty;
        else               logits[t] *= penalty;
    }
}

/* model.cpp:272-283: first maximum wins (strict >). */
static int first_argmax(const float *v, int n)
{
    int best = 0;
    float top = v[0];
    for (int i = 1; i < n; ++i)
        if (v[i] > top) { top = v[i]; best = i; }
    return best;
}

typedef struct { float prob; int index; } orc_prob_index;

/* model.cpp:247-253: descending by probability, equal keys compare equal. */
static int by_prob_desc(const void *a, const void *b)
{
    const orc_prob_index *pa = a, *pb = b;
    if (pa->prob > pb->prob) return -1;
    if (pa->prob < pb->prob) return 1;
    return 0;
}

/* model.cpp:256-340 with r supplied by the caller. */
int orc_sample(float *logits, int vocab_size, float temperature, float topp,
               float penalty, const int *history, int history_len, float r)
{
    apply_penalty(logits, vocab_size, penalty, history, history_len);
    if (temperature == 0.0f) return first_argmax(logits, vocab_size);

    for (int i = 0; i < vocab_size; ++i) logits[i] /= temperature;
    orc_softmax(logits, vocab_size);

    if (topp <= 0.0f || topp >= 1.0f) {
        /* :294-303 sequential CDF, first bucket whose upper edge exceeds r */
        float cdf = 0.0f;
        for (int i = 0; i < vocab_size; ++i) {
            cdf += logits[i];
            if (r < cdf) return i;
        }
        return vocab_size - 1;
    }

    /* :305-339 nucleus: sort descending, cut where the mass first exceeds topp,
     * rescale r by the kept mass, walk the kept prefix. */
    orc_prob_index *order = malloc((size_t)vocab_size * sizeof *order);
    for (int i = 0; i < vocab_size; ++i) { order[i].index = i; order[i].prob = logits[i]; }
    qsort(order, (size_t)vocab_size, sizeof *order, by_prob_desc);
    float mass = 0.0f;
    int last = vocab_size - 1;
    for (int i = 0; i < vocab_size; ++i) {
        mass += order[i].prob;
        if (mass > topp) { last = i; break; }
    }
    float target = r * mass;
    float run = 0.0f;
    int pick = order[last].index;
    for (int i = 0; i <= last; ++i) {
        run += order[i].prob;
        if (target < run) { pick = order[i].index; break; }
    }
    free(order);
    return pick;
}

int orc_sample_cdf(float *logits, int vocab_size, float temperature,
                   float penalty, const int *history, int history_len, float r,
                   float *cdf_lo, float *cdf_hi)
{
    apply_penalty(logits, vocab_size, penalty, history, history_len);
    if (temperature == 0.0f) {
        if (cdf_lo) *cdf_lo = 0.0f;
        if (cdf_hi) *cdf_hi = 1.0f;
        return first_argmax(logits, vocab_size);
    }
    for (int i = 0; i < vocab_size; ++i) logits[i] /= temperature;
    orc_softmax(logits, vocab_size);
    float cdf = 0.0f, prev = 0.0f;
    for (int i = 0; i < vocab_size; ++i) {
        prev = cdf;
        cdf += logits[i];
        if (r < cdf) {
            if (cdf_lo) *cdf_lo = prev;
            if (cdf_hi) *cdf_hi = cdf;
            return i;
        }
    }
    if (cdf_lo) *cdf_lo = prev;
    if (cdf_hi) *cdf_hi = cdf;
    return vocab_size - 1;
}

int orc_forward(int token, int pos, orc_state *s, const orc_weights *w,
                const orc_config *p, float temperature, float topp,
                float penalty, const int *history, int history_len, float r)
{
    orc_forward_logits(token, pos, s, w, p);
    return orc_sample(s->logits, p->vocab_size, temperature, topp, penalty,
                      history, history_len, r);
}

/* main.cpp:164-170 / 184-189 / 203-208. */
void orc_history_push(int *history, int *len, int capacity, int token)
{
    if (*len < capacity) {
        history[(*len)++] = token;
    } else {
        memmove(history, history + 1, (size_t)(capacity - 1) * sizeof(int));
        history[capacity - 1] = token;
    }
}

/* main.cpp:139-232 without text.  One uniform per forward() call, in call order
 * (the reference draws rand() inside sample(), model.cpp:291, also for the
 * prefill forwards whose result it discards, and only when temperature != 0):
 * uniforms[pos]. */
int orc_run(const int *prompt, int n_prompt, int steps, float temperature, float topp,
            const float *uniforms, orc_state *s, const orc_weights *w, const orc_config *p,
            int *out_tokens, int out_capacity, orc_run_result *res)
{
    enum { HISTORY_LEN = 64 };                     /* main.cpp:158 */
    int history[HISTORY_LEN];
    int current_history_len = 0;
    int bos = 1;                                   /* main.cpp:147-151 */
    if (prompt == NULL || n_prompt <= 0) {
        prompt = &bos;
        n_prompt = 1;
    }
    int pos = 0;
    int n_out = 0;
    /* 1. prefill, main.cpp:163-180: penalty 1.1f, sampled token discarded */
    for (int i = 0; i < n_prompt - 1; i++) {
        orc_history_push(history, &current_history_len, HISTORY_LEN, prompt[i]);
        (void)orc_forward(prompt[i], pos, s, w, p, temperature, topp, 1.1f, history, current_history_len,
                          uniforms ? uniforms[pos] : 0.0f);
        pos++;
    }
    /* 2. main.cpp:182-190 */
    int token = prompt[n_prompt - 1];
    orc_history_push(history, &current_history_len, HISTORY_LEN, token);
    /* 3. generation, main.cpp:199-223: penalty 1.05f; the end-of-sequence ids stop the loop
     *    after they entered the window and before pos advances */
    int stopped = 0;
    for (; pos < steps; pos++) {
        token = orc_forward(token, pos, s, w, p, temperature, topp, 1.05f, history, current_history_len,
                            uniforms ? uniforms[pos] : 0.0f);
        orc_history_push(history, &current_history_len, HISTORY_LEN, token);
        if (token == 2 || token == 128001 || token == 128009) {  /* main.cpp:211-213, the id half of each test */
            stopped = 1;
            break;
        }
        if (n_out < out_capacity) out_tokens[n_out] = token;
        n_out++;
    }
    if (res) {
        res->n_tokens = n_out;
        res->final_pos = pos;
        res->stopped_by_eos = stopped;
        res->reported_count = pos - n_prompt;      /* main.cpp:229 */
        res->history_len = current_history_len;
        memcpy(res->history, history, sizeof(history));
    }
    return 0;
}

/* load_model_file (loader.cpp:134-172) + checkpoint_init_weights (loader.cpp:18-66):
 * seven ints, then fp32 tensors back to back in the order below; the classifier is
 * the embedding table.  Offsets and counts are in floats from the first weight. */
int orc_checkpoint_parse(const void *file_bytes, size_t file_size, orc_config *cfg,
                         size_t offsets[12], size_t counts[12])
{
    if (file_size < 28) return -1;
    int header[7];
    memcpy(header, file_bytes, sizeof(header));
    cfg->dim = header[0];
    cfg->hidden_dim = header[1];
    cfg->n_layers = header[2];
    cfg->n_heads = header[3];
    cfg->n_kv_heads = header[4];
    cfg->vocab_size = header[5];
    cfg->seq_len = header[6];
    cfg->rope_base = 10000.0f;                     /* loader.cpp:163 */
    if (cfg->dim <= 0 || cfg->hidden_dim <= 0 || cfg->n_layers <= 0 || cfg->n_heads <= 0 ||
        cfg->n_kv_heads <= 0 || cfg->vocab_size <= 0 || cfg->seq_len <= 0)
        return -2;
    const size_t dim = (size_t)cfg->dim, hidden = (size_t)cfg->hidden_dim, L = (size_t)cfg->n_layers;
    const size_t head_size = dim / (size_t)cfg->n_heads;           /* loader.cpp:19 */
    const size_t q_cols = (size_t)cfg->n_heads * head_size, kv_cols = (size_t)cfg->n_kv_heads * head_size;
    const size_t n[11] = {
        (size_t)cfg->vocab_size * dim,  /* token_embedding_table  :22-23 */
        L * dim,                        /* rms_att_weight         :26-27 */
        L * dim * q_cols,               /* wq                     :30-31 */
        L * dim * kv_cols,              /* wk                     :34-35 */
        L * dim * kv_cols,              /* wv                     :38-39 */
        L * q_cols * dim,               /* wo                     :42-43 */
        L * dim,                        /* rms_ffn_weight         :46-47 */
        L * dim * hidden,               /* w1                     :50-51 */
        L * hidden * dim,               /* w2                     :54-55 */
        L * dim * hidden,               /* w3                     :58-59 */
        dim                             /* rms_final_weight       :62-63 */
    };
    size_t at = 0;
    for (int t = 0; t < 11; t++) {
        offsets[t] = at;
        counts[t] = n[t];
        at += n[t];
    }
    offsets[11] = offsets[0];                      /* w_cls = token_embedding_table, :66 */
    counts[11] = counts[0];
    if (28 + at * sizeof(float) > file_size) return -3;
    return 0;
}
