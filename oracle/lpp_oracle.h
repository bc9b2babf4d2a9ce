/*
 * lpp_oracle.h -- CPU oracle for the Lighter++ batch-1 decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * CPU path (src/ops.cpp, the non-CUDA branches of src/model.cpp) used as the
 * checker for the HIP library.  Nothing in the product (the HIP library, its
 * host decode loop, the Python binding) may include, link or call it; only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * Pinning status of each function (what proves it follows the reference):
 *   orc_naive_matmul  runtests.cpp:87-126 known answers, fp64 brute force,
 *                     bit-equality with the compiled reference (oracle/_ref)
 *   orc_rmsnorm       runtests.cpp:128-144 known answer, closed form, _ref
 *   orc_rope          runtests.cpp:147-184 (pos 0 identity / pos 1 moves),
 *                     pair-norm preservation, fp64 closed form, _ref
 *   orc_softmax       runtests.cpp:256-283 known answer, sum = 1, _ref
 *   orc_swiglu        runtests.cpp:285-306 known answer, _ref
 *   orc_attention, orc_transformer_block, orc_forward, orc_sample
 *                     not covered by any reference test; pinned by fp64 brute
 *                     force on tiny shapes, hand-built sampler cases, golden
 *                     vectors written from the compiled reference
 *                     (tests/golden) and live bit-equality with oracle/_ref
 *   orc_run           golden token sequences written from the reference's own
 *                     executable (oracle/_ref/lighterpp_ref, built from main.cpp
 *                     and the six files it needs) on a tiny synthetic checkpoint
 *                     with a one-character-per-id tokenizer, greedy, with and
 *                     without a prompt (tests/golden/ref_driver.json)
 *   orc_checkpoint_parse  live equality with the compiled reference's
 *                     load_model_file + checkpoint_init_weights (oracle/_ref) and
 *                     the same golden run (the executable reads the file itself)
 *   orc_f16_to_f32    exhaustive over all 65536 half bit patterns against the
 *                     IEEE definition (numpy float16) and _ref-independent
 */
#ifndef LPP_ORACLE_H
#define LPP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Shape of a model; mirrors Config (src/model.h:21-31) minus weight_precision,
 * which the oracle replaces by the per-call "w_is_f16" flag below. */
typedef struct {
    int dim;
    int hidden_dim;
    int n_layers;
    int n_heads;
    int n_kv_heads;
    int vocab_size;
    int seq_len;
    float rope_base;
} orc_config;

/* Weight bundle; mirrors the host half of transformerWeights
 * (src/model.h:34-55).  Matrices are stacked per layer, row-major [rows][cols].
 * When w_is_f16 != 0 the nine matrix pointers address IEEE binary16 bit
 * patterns (uint16_t) that are widened exactly on the fly, which is what the
 * reference's GGUF loader does once at load time (src/loader.cpp:346-402).
 * The embedding table and the three norm gains are always fp32. */
typedef struct {
    const float *token_embedding_table; /* [vocab][dim]              */
    const float *rms_att_weight;        /* [L][dim]                  */
    const void  *wq;                    /* [L][dim][dim]             */
    const void  *wk;                    /* [L][kv_dim][dim]          */
    const void  *wv;                    /* [L][kv_dim][dim]          */
    const void  *wo;                    /* [L][dim][dim]             */
    const float *rms_ffn_weight;        /* [L][dim]                  */
    const void  *w1;                    /* [L][hidden][dim]  gate    */
    const void  *w2;                    /* [L][dim][hidden]  down    */
    const void  *w3;                    /* [L][hidden][dim]  up      */
    const float *rms_final_weight;      /* [dim]                     */
    const void  *w_cls;                 /* [vocab][dim]              */
    int w_is_f16;
} orc_weights;

/* Activation buffers + KV cache; mirrors the host half of RunState
 * (src/model.h:78-94).  Cache shape [L][n_kv_heads][seq_len][head_size] fp32.
 * kv_round_f16 != 0 rounds every K/V element through binary16 (RN) as it is
 * stored, which reproduces what the GPU operator API does by contract
 * (kernels.cuh:34 stores __half); 0 is the reference CPU behaviour. */
typedef struct {
    float *x, *xb, *xb2, *hb, *he, *q, *k, *v, *att, *logits;
    float *key_cache, *value_cache;
    int kv_round_f16;
} orc_state;

/* ---- src/ops.cpp ------------------------------------------------------ */
void orc_naive_matmul(float *out, const float *x, const float *w, int n, int d);
void orc_matmul_f16w(float *out, const float *x, const uint16_t *w, int n, int d);
void orc_rmsnorm(float *out, const float *x, const float *weight, int n);
void orc_rope(float *q, float *k, int pos, int dim, int kv_dim, int head_size,
              float rope_base);
void orc_softmax(float *x, int size);
void orc_swiglu(float *hb, const float *h1, const float *h3, int size);

/* ---- src/loader.cpp:346-379 and its inverse ---------------------------- */
float    orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16_rn(float f);

/* ---- src/model.cpp ----------------------------------------------------- */
int  orc_state_alloc(orc_state *s, const orc_config *p);
void orc_state_free(orc_state *s);
void orc_attention(orc_state *s, const orc_weights *w, const orc_config *p,
                   int layer, int pos);
void orc_transformer_block(orc_state *s, const orc_weights *w,
                           const orc_config *p, int layer, int pos);
/* forward() up to and including the classifier; logits land in s->logits. */
void orc_forward_logits(int token, int pos, orc_state *s, const orc_weights *w,
                        const orc_config *p);
/* sample(): the uniform draw r replaces the reference's rand()/RAND_MAX
 * (src/model.cpp:292) so both sides of a parity test see the same number.
 * Mutates logits exactly as the reference does. */
int  orc_sample(float *logits, int vocab_size, float temperature, float topp,
                float penalty, const int *history, int history_len, float r);
/* As orc_sample on the plain-CDF branch, and also reports the sequential CDF
 * value just below and at the returned token so a harness can tell how close
 * r sat to a bucket edge. */
int  orc_sample_cdf(float *logits, int vocab_size, float temperature,
                    float penalty, const int *history, int history_len, float r,
                    float *cdf_lo, float *cdf_hi);
int  orc_forward(int token, int pos, orc_state *s, const orc_weights *w,
                 const orc_config *p, float temperature, float topp,
                 float penalty, const int *history, int history_len, float r);

/* Sliding repetition-penalty window of src/main.cpp:158-208 (append, or shift
 * left by one when full). */
void orc_history_push(int *history, int *len, int capacity, int token);

/* The driver loop of src/main.cpp:139-232 without text: prefill-by-decode of all
 * but the last prompt id (penalty 1.1, results discarded), generation from the
 * last one (penalty 1.05) until position `steps` or an end-of-sequence id (2,
 * 128001, 128009), 64-entry sliding window.  prompt == NULL: the single id 1. */
typedef struct {
    int n_tokens;        /* ids the reference would have printed during generation */
    int final_pos;
    int stopped_by_eos;
    int reported_count;  /* "Tokens generated", main.cpp:229: final_pos - n_prompt */
    int history_len;
    int history[64];
} orc_run_result;
int orc_run(const int *prompt, int n_prompt, int steps, float temperature, float topp,
            const float *uniforms, orc_state *s, const orc_weights *w, const orc_config *p,
            int *out_tokens, int out_capacity, orc_run_result *res);

/* llama2.c checkpoint (src/loader.cpp:134-172 header, :18-66 tensor order). */
int orc_checkpoint_parse(const void *file_bytes, size_t file_size, orc_config *cfg,
                         size_t offsets[12], size_t counts[12]);

#ifdef __cplusplus
}
#endif
#endif
