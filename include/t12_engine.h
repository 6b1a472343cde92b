/* C face of the engine API (libturbo12.so) for callers that cannot include the C++ headers
 * include/turbo/{model,inference,sampler}.h: ctypes, cgo, JNI.  Each function forwards to the C++
 * function named beside it, which keeps the reference's name and meaning (engine/model.h:79-82,
 * engine/inference.h:43-55, engine/sampler.h:5-11).  Handles are the C++ objects as void*.
 *
 * Errors: where the reference ends the process (GPU_CHECK, gpu_compat.h:94-101; exit(1), inference.cpp:73,223,306)
 * the C++ functions throw EngineError (include/turbo/model.h).  No exception crosses this interface: a function
 * that returns int returns T12_EENGINE (counts are >= 0), one that returns a handle returns NULL, and
 * t12_last_error() has the text.  A state whose call failed is good only for t12_engine_free_state.
 */
#ifndef T12_ENGINE_H
#define T12_ENGINE_H

#include <stddef.h>
#include <stdint.h>
#include "t12_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

void* t12_engine_load(const char* model_dir, int device);            /* load_model; NULL on failure (model.cpp:165-328) */
/* check_model_dir: the host-only consistency check load_model starts with (files present, sizes, tensor shapes
 * against config.bin, escape-list invariants).  0 = consistent; -1 = not, first finding in msg (cap bytes).
 * No counterpart in the reference, which loads what it finds (model.cpp:203-242). */
int   t12_engine_check_dir(const char* model_dir, char* msg, size_t cap);
/* create_synthetic_model: a random-init model of the given shape, generated and packed on the GPU
 * (weights N(0, 0.02) with outliers N(0, 8) at rate p_outlier; norm weights 1).  No reference counterpart:
 * the reference loads converted checkpoints only. */
void* t12_engine_create_synthetic(int n_vocab, int n_embd, int n_head, int n_head_kv, int n_layer, int n_ff, int n_ctx,
                                  float rope_theta, float rms_eps, uint64_t seed, int max_seq, float p_outlier);
int   t12_engine_save(void* model, const char* dir);                 /* save_model: the files of convert_model.py:127-152; 0 = ok */
void  t12_engine_free_model(void* model);                            /* free_model */
int   t12_engine_max_seq(void* model);                               /* Model::max_seq_len (TURBO_CTX, model.cpp:192-195) */
/* which: 0 wq 1 wk 2 wv 3 wo 4 w_gate 5 w_up 6 w_down; layer -1 = output_proj.  Fills *seg (out = NULL), *K and the
 * escape count; returns 0, or -1 for a tensor that does not exist. */
int   t12_engine_weight(void* model, int layer, int which, T12Segment* seg, int* K, int* num_patches);
/* The derived escape tables load_compressed builds for the same tensor (engine/model.cpp:86-160), as device
 * pointers: escape_row_base [M], escape_vals [num_patches] (correct values ordered row, col % 256, col),
 * patch_nonempty_rows [*n_nonempty]. */
int   t12_engine_weight_tables(void* model, int layer, int which, const int32_t** row_base, const int16_t** vals,
                               const int32_t** nonempty_rows, int* n_nonempty);

void* t12_engine_create_state(void* model, int batch, int max_seq);  /* create_inference_state (inference.cpp:94-166) */
/* create_inference_state_per_sequence: batch INDEPENDENT sequences, each with its own KV-cache region of max_seq
 * positions owned by the state.  No counterpart in the reference, whose batch shares one region (kv_stride = 0,
 * inference.cpp:427-435).  NULL when the caches do not fit in free device memory. */
void* t12_engine_create_state_per_sequence(void* model, int batch, int max_seq);
void  t12_engine_free_state(void* state);                            /* free_inference_state */
/* prefill: the n_tokens prompt ids (host) of sequence seq go through the layer stack as the rows of a batch
 * (decode+GEMM kernels, causal), up to batch at a time; leaves the last token's logits in row seq and advances
 * positions[seq].  The reference prompts one token per forward (inference.cpp:721-724). */
int   t12_engine_prefill(void* state, int seq, const int* tokens_host, int n_tokens);
void  t12_engine_set_positions(void* state, const int* pos);         /* state->positions[0..batch) = pos (inference.cpp:722) */
void  t12_engine_get_positions(void* state, int* pos);
int   t12_engine_forward(void* state, const int* tokens_host);       /* forward: logits stay on the device */
void* t12_engine_logits(void* state);                                /* state->logits, fp32 [batch, n_vocab] on the device */
void* t12_engine_stream(void* state);                                /* state->stream (hipStream_t) */
int   t12_engine_sync(void* state);                                  /* hipStreamSynchronize(state->stream); 0 = ok */
int   t12_engine_sample(void* state, int* tokens_out_host);          /* sample_greedy_batch on state->logits (sampler.cpp:18-32) */
/* generate: prompt, then up to max_tokens greedy tokens (stops on id 2, inference.cpp:727,742); writes them to out
 * (room for max_tokens ints) and returns how many. */
int   t12_engine_generate(void* state, const int* prompt, int n_prompt, int max_tokens, int* out);
/* decode_greedy: the decode half of generate, from the logits the state holds: up to max_tokens steps of
 * (sample, forward), the next step enqueued before the host has read the token.  out may be NULL. */
int   t12_engine_decode(void* state, int max_tokens, int stop_on_eos, int* out);
/* decode_greedy_until: decode_greedy with the stop id named by the caller (-1: none). */
int   t12_engine_decode_until(void* state, int max_tokens, int stop_id, int* out);
/* decode_greedy_all: the same loop without the stop rule, every sequence's ids: out[t * batch + b] (host, room
 * for max_tokens * batch ints, may be NULL); returns the number of steps. */
int   t12_engine_decode_all(void* state, int max_tokens, int* out);

/* prefill_rows: prompt pass of a batch-1 state, `rows` tokens per pass through a helper state of that many rows that
 * the state creates on first use (decode+GEMM kernels; the reference prompts one token per forward,
 * inference.cpp:721-724); logits of the last token in state->logits, positions[0] advanced. */
int   t12_engine_prefill_rows(void* state, const int* tokens_host, int n_tokens, int rows);
/* shift_context: cache rows [discard, current_pos) of sequence seq -> rows [0, current_pos - discard), all layers,
 * K, V and scales (the reference does this inline, engine/main.cpp:147-173). */
int   t12_engine_shift_context(void* state, int seq, int current_pos, int discard);
/* chat_turn: one turn of the reference's interactive loop (engine/main.cpp:139-213) on a batch-1 state: drops a
 * leading BOS after the first turn, shifts the context when it is too long, enters the n_tokens ids at *current_pos,
 * generates up to max_tokens ids until eos_id / bos_id (into out, room for max_tokens), feeds eos_id, advances
 * *current_pos; *discarded (may be NULL) = cache rows dropped by the shift.  prompt_rows > 1: the new ids enter that
 * many per pass (prefill_rows) instead of one per forward.  Returns the number generated. */
int   t12_engine_chat_turn(void* state, int* current_pos, const int* tokens, int n_tokens, int max_tokens, int bos_id,
                           int eos_id, int prompt_rows, int* discarded, int* out);

/* ---- tokenizer: C face of include/turbo/tokenizer.h (the reference's engine/tokenizer.h:19-23), host only ---- */
void* t12_tokenizer_load(const char* model_dir);                      /* load_tokenizer; NULL without tokenizer.model or vocab.bin + merges.bin */
void  t12_tokenizer_free(void* tok);                                  /* free_tokenizer */
int   t12_tokenizer_info(void* tok, int* bos_id, int* eos_id, int* vocab_size);
int   t12_tokenizer_type(void* tok);                                  /* Tokenizer::type: 0 sentencepiece model, 1 byte-level BPE tables */
/* Tokenizer::special_tokens: returns their number; for 0 <= index < number also the text (NUL-terminated, cut to cap) and id. */
int   t12_tokenizer_special(void* tok, int index, char* text_out, size_t cap, int* id_out);
/* Adds to Tokenizer::special_tokens (kept longest first, engine/tokenizer.cpp:136-140): the text is cut out of
 * inputs before encoding and becomes `id` (engine/tokenizer.cpp:366-425). */
int   t12_tokenizer_add_special(void* tok, const char* text, int id);
/* tokenize (BOS first, engine/tokenizer.cpp:427-431): writes at most cap ids, returns how many the text has. */
int   t12_tokenizer_encode(void* tok, const char* text, size_t len, int* ids_out, int cap);
/* detokenize / detokenize_one (engine/tokenizer.cpp:433-506): write at most cap bytes (no terminator), return the length. */
int   t12_tokenizer_decode(void* tok, const int* ids, int n, char* out, size_t cap);
int   t12_tokenizer_decode_one(void* tok, int id, char* out, size_t cap);

/* Synthetic tensors on the device (what create_synthetic_model is built from). */
int   t12_synth_normal_bf16(void* out_bf16, size_t n, uint64_t seed, float sigma, float p_outlier, float sigma_outlier,
                            void* stream);
int   t12_fill_f32(void* out, size_t n, float value, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* T12_ENGINE_H */
