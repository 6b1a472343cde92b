// Model store of the split-12 engine: the reference's engine/model.h API
// (structs ModelConfig, CompressedWeight, TransformerLayer, Model; load_model,
// free_model -- engine/model.h:8-82) on HIP for gfx950.  Field names and
// meanings are the reference's so that host code written against it compiles
// unchanged; what differs is noted per field.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

// What the engine throws where the reference ends the process (its GPU_CHECK, gpu_compat.h:94-101, and the
// `exit(1)` of inference.cpp:73,223,306): a failed GPU call, a launch the library refused, a position past the
// cache, an argument outside the batch.  The message has already gone to stderr, as the reference prints it.  A
// caller that does not catch it still ends (std::terminate); the C face (t12_engine_*) catches it and returns a
// negative code with the text in t12_last_error().  The state the call worked on is not usable afterwards.
struct EngineError : std::runtime_error {
    using std::runtime_error::runtime_error;
};
// Prints "ERROR: <text>" to stderr and throws EngineError(<text>).
[[noreturn]] void engine_fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Model hyperparameters (config.bin: 7 x int32 + 2 x float32, engine/model.cpp:181-191)
struct ModelConfig {
    int n_vocab;
    int n_embd;
    int n_head;
    int n_head_kv;
    int n_layer;
    int n_ff;
    int n_ctx;
    float rope_theta;
    float rms_norm_eps;
    // Not in the reference's struct or in config.bin: the checkpoint's rope_scaling entry of the "llama3"
    // kind (factor, low_freq_factor, high_freq_factor, original_max_position_embeddings), read from the
    // optional file rope_scaling.bin (4 x float32); factor 0 = plain RoPE, as the reference always does
    // (engine/convert_model.py:54).
    float rope_scaling[4];
};

// One split-12 tensor on the GPU (engine/model.h:21-40).
struct CompressedWeight {
    int M, K;
    int32_t* row_offsets;         // [M+1] CSR row pointers (NULL when the tensor has no escapes)
    int32_t* patch_cols;          // [num_patches]
    int16_t* patch_correct;       // [num_patches] exact bf16 bits
    int16_t* patch_wrong;         // [num_patches] what the plain rule yields for group 0
    int num_patches;
    int base_exp;
    int32_t* escape_row_base;     // [M] escapes before row r (built at load, engine/model.cpp:101-112)
    uint8_t* escape_counts;       // always NULL here: the kernels of this build take escapes from the CSR list
    int16_t* escape_vals;         // [num_patches] correct values ordered (row, col % 256, col) (model.cpp:114-125)
    uint8_t* split_sm;            // [M*K]
    uint8_t* split_gr;            // [(M*K+1)/2]
    int32_t* patch_nonempty_rows; // [num_nonempty_rows]
    int num_nonempty_rows;
};

struct TransformerLayer {
    CompressedWeight wq, wk, wv, wo;
    CompressedWeight w_gate, w_up, w_down;
    float* attn_norm;   // [n_embd] fp32
    float* ffn_norm;    // [n_embd] fp32
};

struct Model {
    ModelConfig config;
    int16_t* token_embd;          // [n_vocab, n_embd] bf16
    std::vector<TransformerLayer> layers;
    float* output_norm;           // [n_embd] fp32
    CompressedWeight output_proj; // [n_vocab, n_embd]
    int8_t* kv_cache_k;           // [n_layer, max_seq, n_head_kv, head_dim] int8
    int8_t* kv_cache_v;
    float* kv_scale_k;            // [n_layer, max_seq, n_head_kv]
    float* kv_scale_v;
    int max_seq_len;
};

// Reads a converted model directory (config.bin, tok_embd.bin, *_norm.bin and the
// seven files of every tensor).  Returns nullptr when config.bin or tok_embd.bin is
// missing (engine/model.cpp:173-178,198) -- and, unlike the reference, which warns and
// carries on with null pointers (model.cpp:203-242), also when check_model_dir finds
// anything else wrong: the first forward would turn it into a device memory fault.
// Context length: TURBO_CTX, else min(8192, what fits in free HBM) (model.cpp:248-269).
Model* load_model(const std::string& model_path, int device_id = 0);

// Not in the reference: the host-only consistency check load_model starts with (no GPU call).
// Every norm file present with n_embd floats; every tensor's .dims equal to the shape its role
// implies from config.bin (wq n x n, wk/wv kv x n, wo n x n, w_gate/w_up ff x n, w_down n x ff,
// output_proj vocab x n), base_exp in -1..254, plane and list file sizes equal to what .dims
// says, row_off[0] == 0, non-decreasing, row_off[M] == num_patches, escape columns inside the
// row and ascending within it.  false + the first finding in err.
bool check_model_dir(const std::string& model_path, std::string& err);
void free_model(Model* model);

// ---- not in the reference -----------------------------------------------------
// A random-init model of the given shape generated and packed ON THE GPU:
// every weight ~ N(0, 0.02) with a fraction p_outlier replaced by N(0, 8) (so that
// ~0.045 % escape), embeddings N(0, 0.02) bf16, norm weights 1.0.
Model* create_synthetic_model(const ModelConfig& cfg, uint64_t seed, int max_seq_len, float p_outlier = 3e-4f);
// Writes the model in the directory layout load_model reads (the files
// engine/convert_model.py:57-62,127-152 emits).
bool save_model(const Model* model, const std::string& dir);
