// Decode loop of the split-12 engine: the reference's engine/inference.h API
// (InferenceState, create/free, forward, generate -- engine/inference.h:5-55).
#pragma once
#include <functional>
#include "model.h"

struct InferenceState {
    Model* model;
    int batch_size;
    int* positions;       // host, [batch_size]; the caller may overwrite it before forward()

    float* hidden;        // [batch_size, n_embd]
    float* hidden2;       // [batch_size, n_embd]
    float* attn_out;      // [batch_size, n_embd]
    float* q_buf;         // [batch_size, n_head * head_dim]
    float* k_buf;         // [batch_size, n_head_kv * head_dim]
    float* v_buf;         // [batch_size, n_head_kv * head_dim]
    float* ffn_gate;      // [batch_size, n_ff]
    float* ffn_up;        // [batch_size, n_ff]
    float* ffn_down;      // unused (w_down writes the residual buffer), kept for layout parity
    float* logits;        // [batch_size, n_vocab]
    float* attn_scores_buf; // unused
    int* d_positions;     // device [batch_size]
    int* d_tokens;        // device [batch_size]

    hipStream_t stream;
    hipStream_t stream2;
    hipEvent_t sync_event;

    int16_t* bf16_act;    // [batch_size * max(n_embd, n_ff)]
    int16_t* bf16_act2;
    void* patch_descs_gpu; // unused here (escape lists travel as kernel arguments)

    void* impl;           // this build's private per-state data (segment tables)
};

InferenceState* create_inference_state(Model* model, int batch_size, int max_seq_len);
void free_inference_state(InferenceState* state);

// Extension: a state of batch_size INDEPENDENT sequences, each with its own KV-cache region of max_seq_len
// positions owned by the state (int8 [n_layer][batch][max_seq][kv_dim] for K and for V, fp32 scales
// [n_layer][batch][max_seq][n_head_kv]).  The reference keeps one region in the model and lets every row of
// a batch read and write it (kv_stride = 0, engine/inference.cpp:427-435), which only serves lock-step copies
// of one stream.  forward / decode_greedy / prefill work on either kind of state.  nullptr when the caches
// do not fit in free device memory.
InferenceState* create_inference_state_per_sequence(Model* model, int batch_size, int max_seq_len);

// One decode step: token_ids is a HOST array [batch_size]; logits are left in
// state->logits on the device; positions are post-incremented.  Unlike the
// reference (engine/inference.cpp:672-714) every batch size runs all of its
// sequences: B = 1 takes the decode-GEMV path, B > 1 the decode+GEMM path.
void forward(InferenceState* state, const int* token_ids);

// Extension: batched prompt pass for sequence `seq` of the state (the reference prompts one token per
// forward, engine/inference.cpp:721-724).  The n_tokens ids (host array) enter at positions
// state->positions[seq] ... as the rows of a batch, up to batch_size at a time: the linears run on the
// decode+GEMM kernels, every row's K / V is stored before any row attends and row t attends to positions
// <= its own.  Leaves the logits of the last prompt token in row `seq` of state->logits and advances
// state->positions[seq] by n_tokens; the other sequences are untouched.  On a state that shares the model's
// one cache region (lock-step copies) every row's position advances and every row receives the logits.
// With batch_size 1 it is n_tokens calls of forward.
void prefill(InferenceState* state, int seq, const int* token_ids, int n_tokens);

// Extension: prefill for a state of batch size 1, `rows` prompt tokens per pass.  Such a state has no rows to
// batch over (prefill runs it token by token); here a helper state of `rows` rows on the same model, created on
// first use and kept by the state, lends its buffers: the prompt goes through the decode+GEMM kernels into this
// state's cache region, the last token's logits land in state->logits, positions[0] advances by n_tokens.
// rows <= 1 is prefill(state, 0, ...).  The logits agree with the token-by-token pass to rounding (other kernels,
// other summation order), not bit for bit.
void prefill_rows(InferenceState* state, const int* token_ids, int n_tokens, int rows);

// Prompt one token per forward, then greedy decode; stops at token id 2 like the
// reference (engine/inference.cpp:716-748).
std::vector<int> generate(InferenceState* state, const std::vector<int>& prompt_tokens, int max_tokens);

// The decode half of generate (extension): up to max_tokens greedy steps from the logits the state
// holds, each a sample followed by a forward on the sampled ids; returns the ids of sequence 0.
// forward(state, nullptr) runs on the ids already in state->d_tokens (device) -- what lets the loop
// enqueue step t + 1 before the host has seen token t.  The loop alternates state->logits between two buffers
// (the pointer may differ after the call); when a stop id ends the stream, state->logits are the logits it was
// sampled from, as in the reference's sample-wait-forward order (TURBO_NO_PIPELINE, read when the state is created).
std::vector<int> decode_greedy(InferenceState* state, int max_tokens, bool stop_on_eos);

// decode_greedy with the stop id named by the caller (-1: none): sequence 0 sampling it ends the stream; it is not
// returned, the positions do not count it, and state->logits are the logits it was sampled from.
std::vector<int> decode_greedy_until(InferenceState* state, int max_tokens, int stop_id);

// decode_greedy without the stop rule, returning every sequence's ids: element [t * batch_size + b].
std::vector<int> decode_greedy_all(InferenceState* state, int max_tokens);

// Extension: the context shift of the reference's interactive loop (engine/main.cpp:147-173) as a function.  The
// cache rows [discard, current_pos) of sequence `seq`, all layers, move to rows [0, current_pos - discard): int8 K
// and V as stored -- keys keep the rotation of the positions they were written at, as in the reference -- and
// their scales.  Enqueued on state->stream; the caller continues at position current_pos - discard.  On a state
// that shares the model's one region `seq` only has to be a valid row.
void shift_context(InferenceState* state, int seq, int current_pos, int discard);

// Extension: one turn of the reference's interactive loop (engine/main.cpp:139-213) for a state of batch size 1.
// turn_tokens = tokenize(line) (BOS first; dropped unless *current_pos == 0); when *current_pos + |tokens| +
// max_tokens + 64 exceeds the cache, or *current_pos > 1024, the older half of the context is discarded first
// (shift_context; *discarded receives the count).  Then the new tokens enter at *current_pos, up to max_tokens
// greedy tokens follow until eos_id or bos_id is sampled (neither is returned), and eos_id (2 when eos_id <= 0)
// is fed so that the context records the end of the turn.  *current_pos is advanced past all of it.  on_token
// (optional) receives every generated id as soon as the host has it.  prompt_rows > 1 enters the new tokens that
// many per pass (prefill_rows) instead of one per forward.
std::vector<int> chat_turn(InferenceState* state, int* current_pos, const std::vector<int>& turn_tokens, int max_tokens,
                           int bos_id, int eos_id, int* discarded = nullptr,
                           const std::function<void(int)>& on_token = nullptr, int prompt_rows = 1);
