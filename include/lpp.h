/*
 * lpp.h -- C ABI of liblpp_hip.so: the MI355X (gfx950) implementation of the
 * Lighter++ batch-1 decode path.
 *
 * Everything here is plain C: pointers, sizes and scalars, no C++ or HIP types.
 * Pointers named d_* are DEVICE pointers owned by the caller unless stated.
 * Every function returns an lpp_status (0 = LPP_OK); nothing aborts the
 * process.  lpp_last_error() describes the most recent failure on the calling
 * thread.  Launches are asynchronous on the library's current stream
 * (lpp_set_stream) and ordered only by stream order, exactly like the
 * reference's default-stream launches.
 *
 * Section A replaces, one for one, the twelve host wrappers declared in the
 * reference's src/kernels.cuh:24-36 (the operator surface src/model.cpp calls).
 * Section B replaces the model-level functions of src/model.h:117-164.
 * Section C is plumbing the reference gets from the CUDA runtime directly.
 * Section D is what sits either side of the path in the reference: the llama2.c
 * and GGUF readers (src/loader.cpp, src/gguf.cpp) and the driver loop (src/main.cpp).
 */
#ifndef LPP_H
#define LPP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int lpp_status;
enum {
    LPP_OK = 0,
    LPP_ERR_INVALID_ARG = 1, /* null pointer, non-positive size, shape the kernels cannot take */
    LPP_ERR_HIP = 2,         /* a HIP runtime call failed; see lpp_last_error()                */
    LPP_ERR_OOM = 3,         /* device or host allocation failed                               */
    LPP_ERR_STATE = 4,       /* call order violated (e.g. forward before weights are loaded)   */
    LPP_ERR_UNSUPPORTED = 5  /* valid in the reference, not provided here (e.g. INT4 weights)  */
};

/* binary16 storage; stands where the reference's signatures say __half. */
typedef uint16_t lpp_half;

/* Values of the reference's WeightPrecision (src/model.h:8-12). */
enum { LPP_WEIGHT_FP32 = 0, LPP_WEIGHT_FP16 = 1, LPP_WEIGHT_INT4 = 2 };

/* ===================================================================== */
/* A. Operator entry points (src/kernels.cuh:24-36)                       */
/* ===================================================================== */

/* kernels.cuh:24 cuda_convert_f32_to_f16 (matmul.cu:150-161): dst[i] = RN(src[i]). */
lpp_status lpp_convert_f32_to_f16(lpp_half *d_dst, const float *d_src, int n);

/* kernels.cuh:26 cuda_gemv (matmul.cu:134-147): out[n] = W[n][d] . x[d], W
 * row-major.  precision LPP_WEIGHT_FP16 reads binary16 weights, anything else
 * fp32 (the reference's default: branch).  x stays fp32 and accumulation is
 * fp32; d_workspace is accepted for signature compatibility and never touched. */
lpp_status lpp_gemv(float *d_out, const float *d_x, const void *d_w, void *d_workspace,
                    int n, int d, int precision);

/* kernels.cuh:27 cuda_rmsnorm (RMSNorm.cu:11-71): out = x * w / sqrt(mean(x^2) + 1e-5).
 * d_out may alias d_x. */
lpp_status lpp_rmsnorm(float *d_out, const float *d_x, const float *d_w, int n);

/* kernels.cuh:28 cuda_rope (rope.cu:7-38): rotate adjacent pairs (2i, 2i+1) of q,
 * and of k while 2i < kv_dim, by angle pos / base^((2i mod head_size)/head_size).
 * The cos/sin values are computed on the host with the C library and cached
 * on the device, so they match a CPU run on the same machine bit for bit. */
lpp_status lpp_rope(float *d_q, float *d_k, int pos, int dim, int kv_dim, int head_size,
                    float rope_base);

/* kernels.cuh:29 cuda_swiglu (swiglu.cu:6-33): hb = h1 * sigmoid(h1) * h3; hb may
 * alias h1 or h3.  Every element is processed (no size %% 4 tail is dropped). */
lpp_status lpp_swiglu(float *d_hb, const float *d_h1, const float *d_h3, int size);

/* kernels.cuh:30 cuda_softmax_multihead (softmax.cu:5-125): for each of n_heads
 * rows of stride att_stride, softmax over the first seq_len entries.  d_out may
 * alias d_x. */
lpp_status lpp_softmax_multihead(float *d_out, const float *d_x, int n_heads, int seq_len,
                                 int att_stride);

/* kernels.cuh:31 cuda_scale_multihead (scale.cu:6-21): att[h][t] *= scale, t < seq_len. */
lpp_status lpp_scale_multihead(float *d_att, float scale, int n_heads, int seq_len,
                               int att_stride);

/* kernels.cuh:32 cuda_aggregation_multihead (aggregation.cu:6-31):
 * out[h][i] = sum_{t<seq_len} att[h][t] * V[h/gqa_factor][t][i].  d_v is already
 * offset to the layer; att_stride is both the att row stride and the cache's
 * positions-per-head, as in the reference. */
lpp_status lpp_aggregation_multihead(float *d_out, const lpp_half *d_v, const float *d_att,
                                     int n_heads, int seq_len, int head_size, int gqa_factor,
                                     int att_stride);

/* kernels.cuh:33 cuda_residual_add (residual.cu:5-31): out = a + b; out may alias a or b. */
lpp_status lpp_residual_add(float *d_out, const float *d_a, const float *d_b, int n);

/* kernels.cuh:34 cuda_scatter_kv (scatter_kv.cu:6-26):
 * cache[layer][h][pos][i] = RN16(k or v[h*head_size + i]), cache shape
 * [layers][n_kv_heads][seq_len][head_size].  Offsets are computed in 64 bits. */
lpp_status lpp_scatter_kv(lpp_half *d_key_cache, lpp_half *d_value_cache, const float *d_k,
                          const float *d_v, int layer, int pos, int n_kv_heads, int head_size,
                          int seq_len);

/* kernels.cuh:35 cuda_multihead_gemv (multihead_gemv.cu:6-68):
 * out[h][t] = q_h . K[layer][h/(n_heads/n_kv_heads)][t], t in [0,pos]; d_k_cache is
 * the cache BASE; out row stride is seq_len; unscaled. */
lpp_status lpp_multihead_gemv(float *d_out, const float *d_q, const lpp_half *d_k_cache,
                              int layer, int pos, int n_heads, int n_kv_heads, int head_size,
                              int seq_len);

/* kernels.cuh:36 cuda_sample (sample.cu:6-214), following the CPU sampler's
 * semantics (model.cpp:256-303): repetition penalty applied once per occurrence
 * in history order; temperature 0 returns the lowest index of the maximum;
 * otherwise logits / temperature, softmax, and the first index whose cumulative
 * probability exceeds r (vocab_size-1 if none).  r is the uniform draw the
 * reference's wrapper takes from rand()/RAND_MAX (sample.cu:211); here the caller
 * supplies it.  topp and d_rng_state are accepted and ignored, as in the
 * reference.  d_logits is overwritten (penalised and scaled logits, then
 * probabilities); the 4-byte result lands in d_sampled_token[0]. */
lpp_status lpp_sample(float *d_logits, int vocab_size, float temperature, float topp,
                      float penalty, const int *d_history, int history_len,
                      int *d_sampled_token, unsigned int *d_rng_state, float r);

/* ===================================================================== */
/* B. Model-level entry points (src/model.h:21-164, src/model.cpp)        */
/* ===================================================================== */

/* Same fields, order and meaning as Config (src/model.h:21-31). */
typedef struct lpp_config {
    int dim;
    int hidden_dim;
    int n_layers;
    int n_heads;
    int n_kv_heads;
    int vocab_size;
    int seq_len;
    float rope_base;
    int weight_precision; /* LPP_WEIGHT_FP32 or LPP_WEIGHT_FP16 */
} lpp_config;

/* Tensor names of transformerWeights (src/model.h:34-55); per-layer tensors are
 * stacked [n_layers][rows][cols] exactly as the reference's loaders lay them out. */
enum {
    LPP_T_TOKEN_EMBEDDING = 0, /* fp32 [vocab][dim]                        */
    LPP_T_RMS_ATT = 1,         /* fp32 [L][dim]                            */
    LPP_T_WQ = 2,              /* [L][dim][dim]         weight_precision   */
    LPP_T_WK = 3,              /* [L][kv_dim][dim]                         */
    LPP_T_WV = 4,              /* [L][kv_dim][dim]                         */
    LPP_T_WO = 5,              /* [L][dim][dim]                            */
    LPP_T_RMS_FFN = 6,         /* fp32 [L][dim]                            */
    LPP_T_W1 = 7,              /* [L][hidden][dim]  gate                   */
    LPP_T_W2 = 8,              /* [L][dim][hidden]  down                   */
    LPP_T_W3 = 9,              /* [L][hidden][dim]  up                     */
    LPP_T_RMS_FINAL = 10,      /* fp32 [dim]                               */
    LPP_T_WCLS = 11,           /* [vocab][dim]                             */
    LPP_T_COUNT = 12
};

/* Run-state buffers of RunState (src/model.h:96-114), for inspection. */
enum {
    LPP_B_X = 0, LPP_B_XB = 1, LPP_B_XB2 = 2, LPP_B_HB = 3, LPP_B_HE = 4, LPP_B_Q = 5,
    LPP_B_K = 6, LPP_B_V = 7, LPP_B_ATT = 8, LPP_B_LOGITS = 9,
    LPP_B_KEY_CACHE = 10,  /* binary16 [L][n_kv_heads][seq_len][head_size] */
    LPP_B_VALUE_CACHE = 11,
    LPP_B_COUNT = 12
};

/* How lpp_forward schedules a token. */
enum {
    LPP_PATH_OPS = 0,   /* the twelve section-A operators in the reference's call order
                           (model.cpp:133-160, 216-226, 357-366)                        */
    LPP_PATH_FUSED = 1, /* fused kernels, one HIP graph per token                        */
    LPP_PATH_PERSISTENT = 2 /* one persistent kernel per token                           */
};

typedef struct lpp_model lpp_model;

/* malloc_run_state (model.cpp:18-81) plus device storage for the weights:
 * allocates, zero-fills the KV cache, keeps everything resident in HBM. */
lpp_status lpp_model_create(lpp_model **out, const lpp_config *cfg);
/* free_run_state (model.cpp:83-118) + free_weights_cuda (loader.cpp:181-194). */
lpp_status lpp_model_destroy(lpp_model *m);

/* Size in bytes the named tensor occupies for this model. */
lpp_status lpp_model_tensor_bytes(const lpp_model *m, int tensor, size_t *bytes);
/* Copy host data into (part of) a weight tensor; the upload half of
 * checkpoint_init_weights / gguf_init_weights (loader.cpp:73-131, 543-637). */
lpp_status lpp_model_upload(lpp_model *m, int tensor, size_t byte_offset, const void *host_src,
                            size_t bytes);
/* loader.cpp:619-632: classifier shares the embedding; for FP16 models this makes
 * the binary16 copy on the device with lpp_convert_f32_to_f16. */
lpp_status lpp_model_tie_classifier(lpp_model *m);
/* Device pointer of a weight tensor / run-state buffer (caller must not free). */
lpp_status lpp_model_tensor_ptr(lpp_model *m, int tensor, void **d_ptr);
lpp_status lpp_model_buffer_ptr(lpp_model *m, int buffer, void **d_ptr, size_t *bytes);

/* LPP_PATH_PERSISTENT takes weight rows of up to 32 KiB (8192 fp32 or 16384 binary16
 * columns); for a wider dim or hidden_dim this returns LPP_ERR_UNSUPPORTED and the path
 * stays as it was. */
lpp_status lpp_model_set_path(lpp_model *m, int path);
/* Test hooks of LPP_PATH_PERSISTENT (no counterpart in the reference).  Its kernel waits
 * for values other workgroups publish with a bounded number of polls (default 2^20, far
 * beyond any real wait): a wait that runs out raises a flag that ends every other wait,
 * all workgroups leave the kernel normally, no token is delivered and the device's step
 * record stays as the launch found it, and lpp_forward / lpp_generate return LPP_ERR_HIP
 * ("gave up waiting"); the model is usable again at the next call (lpp_generate: from the
 * position the caller chooses; the cache holds every position decoded before the failed
 * launch), because values carry sequence numbers that never repeat.  One cause is
 * handled inside the library and never reaches the caller: a launch whose workgroups
 * the device dealt out unevenly over its XCDs (the per-XCD hand-overs assume equal
 * shares) switches those hand-overs off for the model and launches the same token again.
 * A give-up while the per-XCD hand-overs are in use switches them off as well.
 * set_spin_limit changes the bound; set_sequence_base moves the 32-bit sequence count
 * (the library re-zeroes its exchange slots and restarts the count before it can wrap).
 * Both are test hooks, like lpp_set_test_option in section C. */
lpp_status lpp_model_set_spin_limit(lpp_model *m, unsigned polls);
lpp_status lpp_model_set_sequence_base(lpp_model *m, unsigned base);
/* Forget the KV cache contents (zero-fill, as malloc_run_state leaves it). */
lpp_status lpp_model_reset(lpp_model *m);

/* attention (model.cpp:121-160) and transformer_block (:205-226), operator path. */
lpp_status lpp_attention(lpp_model *m, int layer, int pos);
lpp_status lpp_transformer_block(lpp_model *m, int layer, int pos);

/* forward (model.cpp:342-371): embed token, run every layer at position pos, final
 * norm, classifier, sample; returns the sampled id in *next_token after the 4-byte
 * device-to-host copy (the only synchronisation).  r is the uniform draw for the
 * sampler (ignored when temperature == 0).  The logits of this step remain
 * readable through LPP_B_LOGITS until the next call (raw, before the sampler
 * touches them, on the fused paths; sampler-mutated on LPP_PATH_OPS, as in the
 * reference). */
lpp_status lpp_forward(lpp_model *m, int token, int pos, float temperature, float topp,
                       float penalty, const int *history, int history_len, float r,
                       int *next_token);

/* Timing filled by lpp_generate. */
typedef struct lpp_gen_stats {
    double wall_seconds;   /* steady_clock around the generation loop, D2H per token included */
    double device_ms;      /* HIP events on the launch stream around the same loop           */
    double kernel_ms_sum;  /* sum of per-token event pairs around the dominant kernel        */
    int    kernel_launches;
    int    tokens;
} lpp_gen_stats;

/* Generation loop of src/main.cpp:158-223 without text: starting from
 * first_token at start_pos, run n_steps forwards, feeding each sampled token
 * back and keeping the sliding penalty window (capacity history_cap; initial
 * contents history[0..*history_len)).  uniforms[n_steps] supplies r per step.
 * out_tokens[n_steps] receives the sampled ids.  No EOS stop. */
lpp_status lpp_generate(lpp_model *m, int first_token, int start_pos, int n_steps,
                        float temperature, float topp, float penalty, int *history,
                        int *history_len, int history_cap, const float *uniforms,
                        int *out_tokens, lpp_gen_stats *stats);

/* ===================================================================== */
/* D. The callers either side of the path (src/main.cpp, src/loader.cpp)  */
/* ===================================================================== */

/* A llama2.c checkpoint mapped into host memory: seven-int header (dim,
 * hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len) followed by fp32
 * tensors in the order of LPP_T_TOKEN_EMBEDDING .. LPP_T_RMS_FINAL, classifier tied
 * to the embedding.  Host code only; needs no GPU. */
typedef struct lpp_checkpoint lpp_checkpoint;
/* load_model_file (loader.cpp:134-172): maps the file, reads the header, sets
 * rope_base 10000; weight_precision is LPP_WEIGHT_FP32.  Unlike the reference it
 * checks that every field is positive and that the file holds all its tensors. */
lpp_status lpp_checkpoint_open(lpp_checkpoint **out, const char *path);
/* free_model_file (loader.cpp:174-177). */
lpp_status lpp_checkpoint_close(lpp_checkpoint *ck);
lpp_status lpp_checkpoint_config(const lpp_checkpoint *ck, lpp_config *cfg);
/* Where checkpoint_init_weights (loader.cpp:18-66) points the named tensor:
 * host address inside the mapping and number of floats.  LPP_T_WCLS answers with
 * the embedding table (:66). */
lpp_status lpp_checkpoint_tensor(const lpp_checkpoint *ck, int tensor, const float **host,
                                 size_t *count);
/* lpp_model_create + the upload half of checkpoint_init_weights (loader.cpp:73-131)
 * + lpp_model_tie_classifier. */
lpp_status lpp_model_load_checkpoint(lpp_model **out, const lpp_checkpoint *ck);

/* A GGUF file (versions 2 and 3) mapped into host memory; src/gguf.cpp.  Host code
 * only; needs no GPU.  Tensor types read: F32 and F16 (gguf.h:10-17). */
typedef struct lpp_gguf lpp_gguf;
enum { LPP_GGML_F32 = 0, LPP_GGML_F16 = 1 };
/* gguf_open (gguf.cpp:125-266): header, key/value index, tensor descriptions, data
 * section at the next multiple of 32.  Unlike the reference it bounds every read,
 * every tensor's data and the number of dimensions by the file. */
lpp_status lpp_gguf_open(lpp_gguf **out, const char *path);
/* gguf_close (gguf.cpp:268-290). */
lpp_status lpp_gguf_close(lpp_gguf *g);
/* gguf_extract_config (loader.cpp:213-339): "<arch>.embedding_length",
 * ".feed_forward_length", ".block_count", ".attention.head_count",
 * ".attention.head_count_kv" (default: head_count), ".context_length" (capped at
 * 16384), ".rope.freq_base" (default 10000); vocab_size = number of entries of
 * "tokenizer.ggml.tokens".  weight_precision as gguf_init_weights detects it
 * (loader.cpp:426-433): FP16 iff blk.0.attn_q.weight is F16. */
lpp_status lpp_gguf_config(const lpp_gguf *g, lpp_config *cfg);
/* gguf_find_tensor + gguf_tensor_data (gguf.cpp:292-303): host address inside the
 * mapping, ggml type and number of elements of a named tensor. */
lpp_status lpp_gguf_tensor(const lpp_gguf *g, const char *name, const void **data, int *ggml_type,
                           size_t *nelements);
/* lpp_model_create + gguf_init_weights (loader.cpp:423-641): token_embd, output_norm,
 * blk.N.{attn_norm, attn_q, attn_k, attn_v, attn_output, ffn_norm, ffn_gate, ffn_down,
 * ffn_up}.weight into the stacked per-layer tensors, output.weight or the tied
 * classifier.  F16 matrices of an FP16 model are uploaded as they are; F16 data
 * destined for an fp32 tensor is widened exactly.  A tensor of another type, or an
 * F32 matrix in an FP16 file, is LPP_ERR_UNSUPPORTED (the reference zero-fills the
 * former and mis-sizes the latter). */
lpp_status lpp_model_load_gguf(lpp_model **out, const lpp_gguf *g);

/* The tokenizer of src/tokenizer.cpp.  Host code only. */
typedef struct lpp_tokenizer lpp_tokenizer;
enum { LPP_TOKENIZER_SENTENCEPIECE = 0, LPP_TOKENIZER_BPE = 1 }; /* TokenizerType, tokenizer.h:4-7 */
/* load_tokenizer (tokenizer.cpp:15-55): the llama2.c tokenizer file -- int maximum
 * token length, then per id a float score, an int length and the bytes. */
lpp_status lpp_tokenizer_load(lpp_tokenizer **out, const char *path, int vocab_size);
/* gguf_init_tokenizer (loader.cpp:648-699): the vocabulary embedded in a GGUF file. */
lpp_status lpp_tokenizer_from_gguf(lpp_tokenizer **out, const lpp_gguf *g);
/* free_tokenizer (tokenizer.cpp:237-245). */
lpp_status lpp_tokenizer_free(lpp_tokenizer *t);
lpp_status lpp_tokenizer_info(const lpp_tokenizer *t, int *vocab_size, int *kind, int *max_token_len);
/* encode (tokenizer.cpp:148-235): optional BOS, a blank in front of the text, one id
 * per byte (space marker / "<0xXX>" fallback; bytes without any entry are dropped),
 * then greedy merging by score.  Ids beyond max_tokens are dropped, as in the
 * reference.  An empty result is returned as such (the reference's merge loop
 * underflows on it). */
lpp_status lpp_tokenizer_encode(const lpp_tokenizer *t, const char *text, int *tokens, int max_tokens,
                                int *n_tokens);
/* decode_token (tokenizer.cpp:61-123): "<0xXX>" entries give their byte, other
 * "<...>" entries nothing, space (and newline) markers their character; at most
 * 255 bytes.  An id outside the vocabulary is an error (the reference exits). */
lpp_status lpp_tokenizer_decode(const lpp_tokenizer *t, int token_id, char *out, size_t capacity);

typedef struct lpp_run_result {
    int n_tokens;        /* ids generated before the stop (what main.cpp prints)          */
    int final_pos;
    int stopped_by_eos;  /* an id of main.cpp:211-213 (2, 128001, 128009) ended the loop  */
    int reported_count;  /* "Tokens generated" as main.cpp:229 counts: final_pos - n_prompt */
    int history_len;     /* the penalty window as the loop left it                        */
    int history[64];
    double wall_seconds; /* steady_clock around the generation loop (main.cpp:196-226)    */
} lpp_run_result;

/* The driver loop of main.cpp:139-232 without text: prefill by decode of
 * prompt[0 .. n_prompt-1) (penalty 1.1, sampled ids dropped), then generation from
 * the last prompt id (penalty 1.05) until position `steps` or an end-of-sequence
 * id; 64-entry sliding penalty window.  prompt == NULL stands for the single id 1
 * (main.cpp:147-151).  uniforms[pos] is the draw of the forward at position pos
 * (the reference draws inside every forward, prefill included): the array must hold
 * max(steps, n_prompt - 1) entries, since a prompt longer than `steps` is still
 * prefilled to its end; it may be NULL only when temperature is 0.  Positions beyond
 * seq_len are an error here (the reference overruns its cache). */
lpp_status lpp_run(lpp_model *m, const int *prompt, int n_prompt, int steps, float temperature,
                   float topp, const float *uniforms, int *out_tokens, int out_capacity,
                   lpp_run_result *res);

/* Batched prefill.  The reference has none: main.cpp:163-180 prefills by
 * decoding the prompt token by token and dropping what the sampler returns).  Writes
 * the key/value cache entries of tokens[0 .. n_tokens) at positions start_pos ..
 * start_pos + n_tokens - 1, all layers: what those decode steps leave behind for later
 * steps to read (K and V rounded to binary16, model.cpp:171-176), within one binary16
 * step of it (the GEMMs sum in another order than the decode GEMVs); no logits,
 * no sampling.  The prompt goes through each layer as one batch of up to 512 tokens:
 * GEMMs on the matrix cores, every weight read once per batch.  Needs binary16
 * weights, dim / kv_dim / hidden_dim multiples of 128, head_size 64 or 128, at most 8
 * query heads per KV head: lpp_prefill_supported says whether the model qualifies
 * (LPP_ERR_UNSUPPORTED and the reason in lpp_last_error otherwise).  `tokens` is host
 * memory.  Synchronous. */
lpp_status lpp_prefill_supported(const lpp_model *m);
/* What a prefill GEMM takes as its input.  LPP_PREFILL_EXACT (default): the fp32 activations as a binary16 head plus a
 * binary16 remainder, two matrix-core products per weight tile: every cache entry lands within one binary16 step of
 * what prefill-by-decode writes.  LPP_PREFILL_FAST: the head alone -- the activations rounded to binary16 where a
 * GEMM reads them, which is what the reference's own GPU GEMV does to x (matmul.cu:85-98), accumulation still fp32:
 * half the matrix-core products and a third fewer bytes through LDS, at a price in accuracy that grows with the
 * depth of the model: every rounded GEMM input adds about 3e-4 of the output's size.  The logits of the steps that
 * follow are then 1.5e-3 to 1.7e-3 from the CPU path's at 16 and 22 layers (inside the decode loop's bar of 2e-3,
 * not by much) and 5e-3 at 32 layers (outside it); cache entries drift by a few binary16 steps.  Opt-in for that
 * reason: the exact mode is the one whose results are held to the decode loop's bar at every shape. */
enum { LPP_PREFILL_EXACT = 0, LPP_PREFILL_FAST = 1 };
lpp_status lpp_model_set_prefill_mode(lpp_model *m, int mode);
lpp_status lpp_prefill(lpp_model *m, const int *tokens, int n_tokens, int start_pos);
/* lpp_run with the prompt (all ids but the last) prefilled by lpp_prefill instead of
 * by decode steps; everything else, the uniforms' indexing by position included, as
 * lpp_run.  Falls back to lpp_run's own prefill when the model does not qualify or the
 * prompt has fewer than 9 ids (a batch costs about five decode steps). */
lpp_status lpp_run_batched_prefill(lpp_model *m, const int *prompt, int n_prompt, int steps, float temperature,
                                   float topp, const float *uniforms, int *out_tokens, int out_capacity,
                                   lpp_run_result *res);
/* The prefill's GEMM on its own (no counterpart in the reference, whose products are
 * all matrix-vector): y[t][f] (+)= sum_j w[f][j] * x[t][j] for t < n_tokens, f < n;
 * w binary16 [n][k] row-major as the weight matrices are stored, x fp32 [n_tokens][k],
 * y fp32 [n_tokens][n]; device pointers.  x is split into a binary16 head and
 * remainder, both multiplied into fp32 accumulators (v_mfma_f32_32x32x16_f16).
 * n and n_tokens multiples of 128, k a multiple of 32. */
lpp_status lpp_prefill_gemm(float *d_y, const void *d_w, const float *d_x, int n, int k, int n_tokens,
                            int accumulate);

/* lpp_prefill_gemm for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, checks and result, bit for bit; the
 * binary16 head and remainder of x go to an 8 MiB array that lives in the library's
 * device image instead of two fresh allocations, so n_tokens * k may not exceed
 * 2097152 (LPP_ERR_INVALID_ARG beyond that).  Nothing is allocated, freed or
 * synchronised: the launches are queued on the library's stream and the call
 * returns.  Every call on a device uses that device's one array: calls that overlap
 * on one device (two streams, two threads) race. */
lpp_status lpp_prefill_gemm_noalloc(float *d_y, const void *d_w, const float *d_x, int n, int k,
                                    int n_tokens, int accumulate);

/* Per-kernel timing of the model's current path, measured with HIP events on the
 * launch stream.  LPP_PATH_FUSED: each kernel class is recorded n_layers times (one
 * launch per layer, so every launch streams different weights) into a graph that is
 * replayed `reps` times between two events.  LPP_PATH_PERSISTENT: `reps` launches of
 * the one kernel at a frozen position.  LPP_PATH_OPS: every operator of section A as
 * forward() launches it, stand-alone, one launch per layer, `reps` tokens' worth per
 * class (the run state is left holding whatever they wrote).  avg_ms is the mean
 * duration of one launch, bytes the algorithmic HBM bytes of one launch at `pos`. */
typedef struct lpp_kernel_time {
    char name[32];
    int launches_per_token;
    double avg_ms;
    double bytes_per_launch;
} lpp_kernel_time;
lpp_status lpp_profile_kernels(lpp_model *m, int pos, int reps, lpp_kernel_time *out, int capacity,
                               int *count);

/* Timeline of one token on LPP_PATH_PERSISTENT at position `pos`, as seen by
 * workgroup 0: out[marks * i + k] is mark k of phase i in 10 ns ticks from the
 * kernel's start (0 = mark not taken).  Phase order per layer: qkv, attention,
 * o-projection, gate/up, down; then classifier and sampler.  Marks of a GEMV
 * phase: 0 phase entered, 1 own inputs received, 2 inputs staged, 3 row results
 * ready, 4 outputs published, 5 first weight step multiplied, 6 last row
 * finished.  Attention (first work item): 0 entered, 5 q/k/v received, 1 = 6 = 2
 * shared through LDS, 7 context walked, 3 lane groups and wavefronts merged,
 * 4 published.
 * *count = marks * phases, *marks_per_phase = marks. */
lpp_status lpp_trace_token(lpp_model *m, int pos, unsigned long long *out, int capacity, int *count,
                           int *marks_per_phase);
/* The same with every workgroup traced: out[(w * *count) + marks * i + k], w < *workgroups,
 * all on workgroup 0's time axis; capacity >= *count * *workgroups (one workgroup per
 * compute unit).  The marks cost about half a microsecond each: a traced token is some
 * 10 % slower than an untraced one. */
lpp_status lpp_trace_token_all(lpp_model *m, int pos, unsigned long long *out, int capacity, int *count,
                               int *marks_per_phase, int *workgroups);

/* ===================================================================== */
/* C. Runtime plumbing                                                    */
/* ===================================================================== */

const char *lpp_last_error(void);
const char *lpp_version(void);
lpp_status lpp_device_count(int *count);
/* Select the device and create the library's stream; idempotent. */
lpp_status lpp_init(int device);
/* Launch on a caller-owned hipStream_t (passed as void*); NULL restores the
 * library's own stream. */
lpp_status lpp_set_stream(void *hip_stream);
lpp_status lpp_get_stream(void **hip_stream);
lpp_status lpp_synchronize(void);
lpp_status lpp_malloc(void **d_ptr, size_t bytes);
lpp_status lpp_free(void *d_ptr);
/* Page-locked host memory, for buffers the device copies into every token (the reference allocates its
 * host logits this way, model.cpp:42 and :94).  Memory that already exists cannot be registered: allocate it here. */
lpp_status lpp_malloc_host(void **h_ptr, size_t bytes);
lpp_status lpp_free_host(void *h_ptr);
lpp_status lpp_memset(void *d_ptr, int value, size_t bytes);
lpp_status lpp_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes);
lpp_status lpp_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes);
lpp_status lpp_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes);
/* Device facts used by the benchmark report. */
lpp_status lpp_device_info(char *name, size_t name_cap, int *compute_units, size_t *hbm_bytes);

/* Test hooks (no counterpart in the reference).  The library picks among alternative
 * plans and kernels by itself -- from the model's shape, the position, and what it
 * measured on the device at the first launch.  Each option below takes one of those
 * choices away so that a test can run the alternative the library would otherwise not
 * have taken on the machine at hand; none changes what is computed.  Process-wide;
 * a model picks a change up at its next launch (the persistent path rebuilds its step
 * lists then).  Defaults in brackets. */
enum lpp_test_option {
    /* LPP_PATH_PERSISTENT */
    LPP_OPT_DECODE_XCD_HANDOVERS = 0,   /* [1] number workgroups by XCD and hand hb / q,k,v over inside an XCD when the
                                               device deals workgroups out to its XCDs in turn; 0: as if it did not */
    LPP_OPT_DECODE_XCD_QKV = 1,         /* [1] deal the Wq/Wk/Wv rows out per XCD where the KV heads divide among them   */
    LPP_OPT_DECODE_PARKING = 2,         /* [1] keep gate/up rows in LDS at short contexts                               */
    LPP_OPT_DECODE_LANE_ITEM = 3,       /* [1] one-pass attention item for heads of size 64; 0: the walking item        */
    LPP_OPT_DECODE_FAIL_TICKETS = 4,    /* [0] n > 0: the n-th launch from now that uses the per-XCD numbering is told a
                                               wrong ticket base, so every workgroup reports an unevenly dealt XCD (the
                                               kernel drains normally) and the library's recovery runs; counts down to 0 */
    LPP_OPT_DECODE_XCD_ATTENTION = 5,   /* [1] split a KV head's context over the workgroups of its XCD at long contexts;
                                               0: work items dealt out over the whole device                            */
    /* batched prefill */
    LPP_OPT_PREFILL_STAGED_GEMM = 6,    /* [1] LDS-pipelined GEMM; 0: fragments straight from memory + separate SwiGLU   */
    LPP_OPT_PREFILL_WIDE_TILES = 7,     /* [1] 256 x 128 tiles where they fill the device                               */
    LPP_OPT_PREFILL_FUSED_FFN = 8,      /* [1] W1, W3 and SwiGLU in one launch                                          */
    LPP_OPT_PREFILL_MFMA_ATTENTION = 9, /* [1] matrix-core attention; 0: one wavefront per token and KV head            */
    LPP_OPT_DECODE_CALIBRATE = 10,      /* [1] LPP_PATH_PERSISTENT: before a model's first token, trace two tokens and deal the
                                               hidden units out by how fast each XCD got through the gate/up phase; 0: evenly  */
    LPP_OPT_COUNT = 11
};
lpp_status lpp_set_test_option(int option, int value);
lpp_status lpp_get_test_option(int option, int *value);

/* Deterministic synthetic tensors (host side): element i of a stream named by
 * seed is N(0, std) from a counter-based generator (splitmix64 -> Box-Muller in
 * double), so any slice can be produced independently.  _f16 rounds to nearest
 * even binary16. */
lpp_status lpp_synth_normal_f32(float *h_dst, size_t n, uint64_t seed, uint64_t first_index,
                                float std);
lpp_status lpp_synth_normal_f16(lpp_half *h_dst, size_t n, uint64_t seed, uint64_t first_index,
                                float std);
lpp_status lpp_synth_uniform_f32(float *h_dst, size_t n, uint64_t seed, uint64_t first_index);
lpp_status lpp_synth_token_ids(int *h_dst, size_t n, uint64_t seed, int vocab_size);
/* Exact widening / RN narrowing on the host (loader.cpp:346-379 and its inverse). */
lpp_status lpp_f16_to_f32_host(float *h_dst, const lpp_half *h_src, size_t n);
lpp_status lpp_f32_to_f16_host(lpp_half *h_dst, const float *h_src, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* LPP_H */
