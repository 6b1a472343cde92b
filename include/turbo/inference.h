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

// One decode step: token_ids is a HOST array [batch_size]; logits are left in
// state->logits on the device; positions are post-incremented.  Unlike the
// reference (engine/inference.cpp:672-714) every batch size runs all of its
// sequences: B = 1 takes the decode-GEMV path, B > 1 the decode+GEMM path.
void forward(InferenceState* state, const int* token_ids);

// Prompt one token per forward, then greedy decode; stops at token id 2 like the
// reference (engine/inference.cpp:716-748).
std::vector<int> generate(InferenceState* state, const std::vector<int>& prompt_tokens, int max_tokens);

// The decode half of generate (extension): up to max_tokens greedy steps from the logits the state
// holds, each a sample followed by a forward on the sampled ids; returns the ids of sequence 0.
// forward(state, nullptr) runs on the ids already in state->d_tokens (device) -- what lets the loop
// enqueue step t + 1 before the host has seen token t.
std::vector<int> decode_greedy(InferenceState* state, int max_tokens, bool stop_on_eos);
