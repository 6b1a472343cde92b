// Decode loop of the split-12 engine: the reference's engine/inference.h API
// (InferenceState, create/free, forward, generate -- engine/inference.h:5-55).
#pragma once
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

// Prompt one token per forward, then greedy decode; stops at token id 2 like the
// reference (engine/inference.cpp:716-748).
std::vector<int> generate(InferenceState* state, const std::vector<int>& prompt_tokens, int max_tokens);

// The decode half of generate (extension): up to max_tokens greedy steps from the logits the state
// holds, each a sample followed by a forward on the sampled ids; returns the ids of sequence 0.
// forward(state, nullptr) runs on the ids already in state->d_tokens (device) -- what lets the loop
// enqueue step t + 1 before the host has seen token t.
std::vector<int> decode_greedy(InferenceState* state, int max_tokens, bool stop_on_eos);

// decode_greedy without the stop rule, returning every sequence's ids: element [t * batch_size + b].
std::vector<int> decode_greedy_all(InferenceState* state, int max_tokens);
