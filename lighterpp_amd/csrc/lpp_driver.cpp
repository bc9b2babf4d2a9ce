// lpp_driver.cpp -- section D of lpp.h: the callers either side of the decode
// path.  The llama2.c checkpoint reader (reference src/loader.cpp:18-66,
// 134-177) and the driver loop of src/main.cpp:139-232 without its text I/O.
// Host code only; the arithmetic stays in the kernels behind lpp_forward.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <chrono>
#include <cstring>

#include "lpp_internal.hpp"
#include "lpp_model.hpp"

namespace {

constexpr size_t kHeaderBytes = 28;  // seven ints; loader.cpp:165 starts the weights there

}  // namespace

struct lpp_checkpoint {
    void* map = nullptr;
    size_t file_size = 0;
    lpp_config cfg{};
    size_t offset[LPP_T_COUNT] = {};  // in floats from the first weight
    size_t count[LPP_T_COUNT] = {};
};

extern "C" {

lpp_status lpp_checkpoint_open(lpp_checkpoint** out, const char* path) {
    using lpp::fail;
    LPP_REQUIRE(out != nullptr && path != nullptr, "lpp_checkpoint_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd == -1) return fail(LPP_ERR_INVALID_ARG, "lpp_checkpoint_open: cannot open %s: %s", path, strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) == -1) {
        close(fd);
        return fail(LPP_ERR_INVALID_ARG, "lpp_checkpoint_open: cannot stat %s", path);
    }
    const size_t file_size = static_cast<size_t>(sb.st_size);
    if (file_size < kHeaderBytes) {
        close(fd);
        return fail(LPP_ERR_INVALID_ARG, "lpp_checkpoint_open: %s holds %zu bytes, fewer than the header", path, file_size);
    }
    void* map = mmap(nullptr, file_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return fail(LPP_ERR_INVALID_ARG, "lpp_checkpoint_open: mmap of %s failed", path);

    lpp_checkpoint* ck = new lpp_checkpoint;
    ck->map = map;
    ck->file_size = file_size;
    int header[7];
    std::memcpy(header, map, sizeof header);
    lpp_config& c = ck->cfg;
    c.dim = header[0];
    c.hidden_dim = header[1];
    c.n_layers = header[2];
    c.n_heads = header[3];
    c.n_kv_heads = header[4];
    c.vocab_size = header[5];
    c.seq_len = header[6];
    // The reference copies 36 bytes of the file into its Config, i.e. the first two
    // weights land in rope_base and weight_precision (loader.cpp:158-160); it then
    // sets rope_base itself (:163) and its loader keeps every tensor fp32.
    c.rope_base = 10000.0f;
    c.weight_precision = LPP_WEIGHT_FP32;
    auto bad = [&](const char* what) {
        lpp_status st = fail(LPP_ERR_INVALID_ARG,
                             "lpp_checkpoint_open: %s: %s (dim %d hidden %d layers %d heads %d kv_heads %d vocab %d seq %d)",
                             path, what, c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len);
        munmap(map, file_size);
        delete ck;
        return st;
    };
    // (llama2.c marks an untied classifier with a negative vocabulary size; the reference's
    // reader knows tied checkpoints only, loader.cpp:66)
    if (c.dim <= 0 || c.hidden_dim <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.vocab_size <= 0 ||
        c.seq_len <= 0)
        return bad("header field not positive");
    if (c.dim % c.n_heads != 0 || c.n_heads % c.n_kv_heads != 0) return bad("heads do not divide");

    // checkpoint_init_weights, loader.cpp:18-66
    const size_t dim = static_cast<size_t>(c.dim), hidden = static_cast<size_t>(c.hidden_dim),
                 L = static_cast<size_t>(c.n_layers);
    const size_t head_size = dim / static_cast<size_t>(c.n_heads);
    const size_t q_cols = static_cast<size_t>(c.n_heads) * head_size, kv_cols = static_cast<size_t>(c.n_kv_heads) * head_size;
    const size_t n[LPP_T_COUNT - 1] = {static_cast<size_t>(c.vocab_size) * dim, L * dim,          L * dim * q_cols,
                                       L * dim * kv_cols,                      L * dim * kv_cols, L * q_cols * dim,
                                       L * dim,                                L * dim * hidden,  L * hidden * dim,
                                       L * dim * hidden,                       dim};
    size_t at = 0;
    for (int t = 0; t < LPP_T_COUNT - 1; ++t) {
        ck->offset[t] = at;
        ck->count[t] = n[t];
        at += n[t];
    }
    ck->offset[LPP_T_WCLS] = ck->offset[LPP_T_TOKEN_EMBEDDING];
    ck->count[LPP_T_WCLS] = ck->count[LPP_T_TOKEN_EMBEDDING];
    if (kHeaderBytes + at * sizeof(float) > file_size) return bad("file shorter than its tensors");
    *out = ck;
    return LPP_OK;
}

lpp_status lpp_checkpoint_close(lpp_checkpoint* ck) {
    if (ck == nullptr) return LPP_OK;
    if (ck->map != nullptr) munmap(ck->map, ck->file_size);
    delete ck;
    return LPP_OK;
}

lpp_status lpp_checkpoint_config(const lpp_checkpoint* ck, lpp_config* cfg) {
    LPP_REQUIRE(ck != nullptr && cfg != nullptr, "lpp_checkpoint_config: null argument");
    *cfg = ck->cfg;
    return LPP_OK;
}

lpp_status lpp_checkpoint_tensor(const lpp_checkpoint* ck, int tensor, const float** host, size_t* count) {
    LPP_REQUIRE(ck != nullptr && host != nullptr && count != nullptr, "lpp_checkpoint_tensor: null argument");
    LPP_REQUIRE(tensor >= 0 && tensor < LPP_T_COUNT, "lpp_checkpoint_tensor: tensor %d", tensor);
    *host = reinterpret_cast<const float*>(static_cast<const char*>(ck->map) + kHeaderBytes) + ck->offset[tensor];
    *count = ck->count[tensor];
    return LPP_OK;
}

lpp_status lpp_model_load_checkpoint(lpp_model** out, const lpp_checkpoint* ck) {
    LPP_REQUIRE(out != nullptr && ck != nullptr, "lpp_model_load_checkpoint: null argument");
    *out = nullptr;
    lpp_model* m = nullptr;
    LPP_TRY(lpp_model_create(&m, &ck->cfg));
    lpp_status st = LPP_OK;
    for (int t = 0; t < LPP_T_COUNT - 1 && st == LPP_OK; ++t) {
        const float* src = nullptr;
        size_t count = 0;
        st = lpp_checkpoint_tensor(ck, t, &src, &count);
        if (st == LPP_OK) st = lpp_model_upload(m, t, 0, src, count * sizeof(float));
    }
    if (st == LPP_OK) st = lpp_model_tie_classifier(m);  // loader.cpp:66
    if (st != LPP_OK) {
        lpp_model_destroy(m);
        return st;
    }
    *out = m;
    return LPP_OK;
}

namespace {
lpp_status run_loop(lpp_model* m, const int* prompt, int n_prompt, int steps, float temperature, float topp,
                    const float* uniforms, int* out_tokens, int out_capacity, lpp_run_result* res, bool batched);
}

lpp_status lpp_run(lpp_model* m, const int* prompt, int n_prompt, int steps, float temperature, float topp,
                   const float* uniforms, int* out_tokens, int out_capacity, lpp_run_result* res) {
    return run_loop(m, prompt, n_prompt, steps, temperature, topp, uniforms, out_tokens, out_capacity, res, false);
}

lpp_status lpp_run_batched_prefill(lpp_model* m, const int* prompt, int n_prompt, int steps, float temperature, float topp,
                                   const float* uniforms, int* out_tokens, int out_capacity, lpp_run_result* res) {
    return run_loop(m, prompt, n_prompt, steps, temperature, topp, uniforms, out_tokens, out_capacity, res, true);
}

}  // extern "C"

namespace {

lpp_status run_loop(lpp_model* m, const int* prompt, int n_prompt, int steps, float temperature, float topp,
                    const float* uniforms, int* out_tokens, int out_capacity, lpp_run_result* res, bool batched) {
    LPP_REQUIRE(m != nullptr, "lpp_run: null model");
    LPP_REQUIRE(out_capacity >= 0 && (out_capacity == 0 || out_tokens != nullptr), "lpp_run: output capacity %d", out_capacity);
    LPP_REQUIRE(temperature == 0.0f || uniforms != nullptr, "lpp_run: uniforms required when temperature != 0");
    const int bos = 1;  // main.cpp:147-151
    if (prompt == nullptr || n_prompt <= 0) {
        prompt = &bos;
        n_prompt = 1;
    }
    const lpp_config& cfg = m->cfg;
    LPP_REQUIRE(steps <= cfg.seq_len, "lpp_run: %d steps exceed seq_len %d", steps, cfg.seq_len);
    LPP_REQUIRE(n_prompt <= cfg.seq_len, "lpp_run: %d prompt ids exceed seq_len %d", n_prompt, cfg.seq_len);
    for (int i = 0; i < n_prompt; ++i)
        LPP_REQUIRE(prompt[i] >= 0 && prompt[i] < cfg.vocab_size, "lpp_run: prompt id %d at %d outside [0, %d)", prompt[i], i,
                    cfg.vocab_size);

    constexpr int kHistory = 64;  // main.cpp:158
    int history[kHistory];
    int history_len = 0;
    auto push = [&](int token) {  // main.cpp:164-170
        if (history_len < kHistory) {
            history[history_len++] = token;
        } else {
            std::memmove(history, history + 1, (kHistory - 1) * sizeof(int));
            history[kHistory - 1] = token;
        }
    };
    int pos = 0;
    int n_out = 0;
    // 1. prefill, main.cpp:163-180.  Batched: the cache entries of all but the last prompt id in one
    //    pass per 512 ids; what the decode steps would have sampled is what the reference drops.
    //    (a batch costs about as much as five decode steps at the 1B shape: short prompts stay with decode)
    constexpr int kShortestBatchedPrompt = 8;
    if (batched && n_prompt - 1 >= kShortestBatchedPrompt && lpp_prefill_supported(m) == LPP_OK) {
        for (int i = 0; i < n_prompt - 1; ++i) push(prompt[i]);
        LPP_TRY(lpp_prefill(m, prompt, n_prompt - 1, 0));
        pos = n_prompt - 1;
    }
    //    By decode: penalty 1.1, the sampled id is dropped
    for (int i = pos; i < n_prompt - 1; ++i) {
        push(prompt[i]);
        int ignored = 0;
        LPP_TRY(lpp_forward(m, prompt[i], pos, temperature, topp, 1.1f, history, history_len, uniforms ? uniforms[pos] : 0.0f,
                            &ignored));
        ++pos;
    }
    // 2. main.cpp:182-190
    int token = prompt[n_prompt - 1];
    push(token);
    // 3. generation, main.cpp:196-223: penalty 1.05; an end-of-sequence id ends the loop after it
    //    entered the window, before the position advances
    const auto t0 = std::chrono::steady_clock::now();
    int stopped = 0;
    for (; pos < steps; ++pos) {
        LPP_TRY(lpp_forward(m, token, pos, temperature, topp, 1.05f, history, history_len, uniforms ? uniforms[pos] : 0.0f,
                            &token));
        push(token);
        if (token == 2 || token == 128001 || token == 128009) {  // main.cpp:211-213
            stopped = 1;
            break;
        }
        if (n_out < out_capacity) out_tokens[n_out] = token;
        ++n_out;
    }
    const auto t1 = std::chrono::steady_clock::now();
    if (res != nullptr) {
        res->n_tokens = n_out;
        res->final_pos = pos;
        res->stopped_by_eos = stopped;
        res->reported_count = pos - n_prompt;  // main.cpp:229
        res->history_len = history_len;
        std::memset(res->history, 0, sizeof res->history);
        std::memcpy(res->history, history, static_cast<size_t>(history_len) * sizeof(int));
        res->wall_seconds = std::chrono::duration<double>(t1 - t0).count();  // main.cpp:196, 225-226
    }
    return LPP_OK;
}

}  // namespace
