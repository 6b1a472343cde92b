// C face of the engine's C++ API (model.h / inference.h / sampler.h) for callers
// that cannot pass std::string / std::vector (ctypes, cgo, JNI).  No exception leaves this file: what the C++
// functions throw (EngineError, std::bad_alloc) becomes T12_EENGINE / NULL with the text in t12_last_error().
#include <cstring>
#include <exception>
#include <string>
#include <vector>

#include "t12_abi.h"
#include "turbo/inference.h"
#include "turbo/sampler.h"
#include "../t12_host.h"

namespace {

template <typename F>
int guarded(F&& body)
{
    try {
        return body();
    } catch (const std::exception& e) {
        t12_set_error("%s", e.what());
        return T12_EENGINE;
    }
}

template <typename F>
void* guarded_ptr(F&& body)
{
    try {
        return body();
    } catch (const std::exception& e) {
        t12_set_error("%s", e.what());
        return nullptr;
    }
}

}  // namespace

extern "C" {

void* t12_engine_load(const char* path, int device)
{
    return guarded_ptr([&]() -> void* { return load_model(path ? path : "", device); });
}

// check_model_dir(); 0 = consistent, -1 = not (the first finding in msg, cut to cap bytes incl. the terminator).
int t12_engine_check_dir(const char* path, char* msg, size_t cap)
{
    std::string err;
    const bool ok = check_model_dir(path ? path : "", err);
    if (msg && cap) {
        strncpy(msg, err.c_str(), cap - 1);
        msg[cap - 1] = 0;
    }
    return ok ? 0 : -1;
}

void* t12_engine_create_synthetic(int n_vocab, int n_embd, int n_head, int n_head_kv, int n_layer, int n_ff, int n_ctx,
                                  float rope_theta, float rms_eps, uint64_t seed, int max_seq, float p_outlier)
{
    ModelConfig c = {n_vocab, n_embd, n_head, n_head_kv, n_layer, n_ff, n_ctx, rope_theta, rms_eps};
    return guarded_ptr([&]() -> void* { return create_synthetic_model(c, seed, max_seq, p_outlier); });
}

int t12_engine_save(void* model, const char* dir)
{
    return guarded([&] {
        if (save_model((Model*)model, dir)) return 0;
        t12_set_error("save_model: could not write the model files under %s (the directory must exist; the file is named on "
                      "standard error)", dir);
        return -1;
    });
}
void t12_engine_free_model(void* model) { free_model((Model*)model); }

void* t12_engine_create_state(void* model, int batch, int max_seq)
{
    return guarded_ptr([&]() -> void* { return create_inference_state((Model*)model, batch, max_seq); });
}
void* t12_engine_create_state_per_sequence(void* model, int batch, int max_seq)
{
    return guarded_ptr([&]() -> void* { return create_inference_state_per_sequence((Model*)model, batch, max_seq); });
}
void t12_engine_free_state(void* state) { free_inference_state((InferenceState*)state); }

int t12_engine_prefill(void* state, int seq, const int* tokens_host, int n_tokens)
{
    return guarded([&] {
        prefill((InferenceState*)state, seq, tokens_host, n_tokens);
        return 0;
    });
}

int t12_engine_forward(void* state, const int* tokens_host)
{
    return guarded([&] {
        forward((InferenceState*)state, tokens_host);
        return 0;
    });
}
void* t12_engine_logits(void* state) { return ((InferenceState*)state)->logits; }
void* t12_engine_stream(void* state) { return ((InferenceState*)state)->stream; }
int t12_engine_max_seq(void* model) { return ((Model*)model)->max_seq_len; }

void t12_engine_set_positions(void* state, const int* pos)
{
    auto* s = (InferenceState*)state;
    memcpy(s->positions, pos, sizeof(int) * s->batch_size);
}
void t12_engine_get_positions(void* state, int* pos)
{
    auto* s = (InferenceState*)state;
    memcpy(pos, s->positions, sizeof(int) * s->batch_size);
}

// Greedy sample of the logits of the last forward; tokens_out is a host array [batch].
int t12_engine_sample(void* state, int* tokens_out)
{
    return guarded([&] {
        auto* s = (InferenceState*)state;
        sample_greedy_batch(s->logits, tokens_out, s->model->config.n_vocab, s->batch_size, s->stream);
        return 0;
    });
}

// generate(); returns the number of tokens written to out (<= max_tokens).
int t12_engine_generate(void* state, const int* prompt, int n_prompt, int max_tokens, int* out)
{
    return guarded([&] {
        std::vector<int> p(prompt, prompt + n_prompt);
        std::vector<int> r = generate((InferenceState*)state, p, max_tokens);
        for (size_t i = 0; i < r.size(); i++) out[i] = r[i];
        return (int)r.size();
    });
}

int t12_engine_decode(void* state, int max_tokens, int stop_on_eos, int* out)
{
    return guarded([&] {
        std::vector<int> r = decode_greedy((InferenceState*)state, max_tokens, stop_on_eos != 0);
        if (out)
            for (size_t i = 0; i < r.size(); i++) out[i] = r[i];
        return (int)r.size();
    });
}

int t12_engine_decode_until(void* state, int max_tokens, int stop_id, int* out)
{
    return guarded([&] {
        std::vector<int> r = decode_greedy_until((InferenceState*)state, max_tokens, stop_id);
        if (out)
            for (size_t i = 0; i < r.size(); i++) out[i] = r[i];
        return (int)r.size();
    });
}

// decode_greedy_all(); out is a host array [max_tokens][batch]; returns the number of steps.
int t12_engine_decode_all(void* state, int max_tokens, int* out)
{
    return guarded([&] {
        auto* s = (InferenceState*)state;
        std::vector<int> r = decode_greedy_all(s, max_tokens);
        if (out)
            for (size_t i = 0; i < r.size(); i++) out[i] = r[i];
        return (int)(r.size() / (size_t)s->batch_size);
    });
}

int t12_engine_prefill_rows(void* state, const int* tokens_host, int n_tokens, int rows)
{
    return guarded([&] {
        prefill_rows((InferenceState*)state, tokens_host, n_tokens, rows);
        return 0;
    });
}

int t12_engine_shift_context(void* state, int seq, int current_pos, int discard)
{
    return guarded([&] {
        shift_context((InferenceState*)state, seq, current_pos, discard);
        return 0;
    });
}

// chat_turn(); out has room for max_tokens ids; returns how many were generated.
int t12_engine_chat_turn(void* state, int* current_pos, const int* tokens, int n_tokens, int max_tokens, int bos_id,
                         int eos_id, int prompt_rows, int* discarded, int* out)
{
    return guarded([&] {
        std::vector<int> t(tokens, tokens + n_tokens);
        std::vector<int> r = chat_turn((InferenceState*)state, current_pos, t, max_tokens, bos_id, eos_id, discarded, nullptr,
                                       prompt_rows);
        if (out)
            for (size_t i = 0; i < r.size(); i++) out[i] = r[i];
        return (int)r.size();
    });
}

int t12_engine_sync(void* state)
{
    return hipStreamSynchronize(((InferenceState*)state)->stream) == hipSuccess ? 0 : -1;
}

// The tensors of the model as segments (out = NULL), for tests that check the
// loader against the files.  which: 0 wq 1 wk 2 wv 3 wo 4 w_gate 5 w_up 6 w_down; layer -1 = output_proj.
int t12_engine_weight(void* model, int layer, int which, T12Segment* seg, int* K, int* num_patches)
{
    Model* m = (Model*)model;
    const CompressedWeight* w = nullptr;
    if (layer < 0) w = &m->output_proj;
    else if (layer < (int)m->layers.size()) {
        TransformerLayer& L = m->layers[layer];
        const CompressedWeight* all[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down};
        if (which >= 0 && which < 7) w = all[which];
    }
    if (!w || !w->split_sm) return -1;
    seg->sm = w->split_sm;
    seg->gr = w->split_gr;
    seg->row_off = w->row_offsets;
    seg->cols = w->patch_cols;
    seg->correct = w->patch_correct;
    seg->wrong = w->patch_wrong;
    seg->out = nullptr;
    seg->M = w->M;
    seg->base_exp = w->base_exp;
    seg->out_stride = seg->reserved = 0;
    *K = w->K;
    *num_patches = w->num_patches;
    return 0;
}

// The loader's derived escape tables of the same tensor (engine/model.cpp:86-160): device pointers to
// escape_row_base [M], escape_vals [num_patches], patch_nonempty_rows [*n_nonempty]; all NULL / 0 for a tensor
// without escapes.
int t12_engine_weight_tables(void* model, int layer, int which, const int32_t** row_base, const int16_t** vals,
                             const int32_t** nonempty_rows, int* n_nonempty)
{
    Model* m = (Model*)model;
    const CompressedWeight* w = nullptr;
    if (layer < 0) w = &m->output_proj;
    else if (layer < (int)m->layers.size()) {
        TransformerLayer& L = m->layers[layer];
        const CompressedWeight* all[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down};
        if (which >= 0 && which < 7) w = all[which];
    }
    if (!w || !w->split_sm) return -1;
    *row_base = w->escape_row_base;
    *vals = w->escape_vals;
    *nonempty_rows = w->patch_nonempty_rows;
    *n_nonempty = w->num_nonempty_rows;
    return 0;
}

}  // extern "C"
