/* C ABI of the decode-step glue kernels (libturbo12.so): embedding lookup, RMSNorm, SiLU*mul,
 * residual add, RoPE, INT8 KV-cache store, GQA decode attention, argmax.
 *
 * Names, argument order and meaning are those of the reference's launch layer in
 * engine/kernels.hip, as its callers declare them (engine/inference.cpp:9-20, engine/sampler.cpp:4-5),
 * so host code written against the reference links unchanged.  All calls are asynchronous on `stream`,
 * take device pointers, transfer no ownership and return nothing (failures are reported through
 * t12_last_error() of t12_abi.h).  bf16 values travel as int16_t, like in the reference.
 */
#ifndef T12_GLUE_H
#define T12_GLUE_H

#include <stddef.h>
#include <stdint.h>

#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t* hipStream_t;   /* the HIP stream handle, for callers without the HIP headers */
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* kernels.hip:129-140.  Builds the inverse-frequency table freq[d] = theta^(-2d/head_dim); optional here:
 * the RoPE launchers build (and cache per (head_dim, theta)) the table on first use. */
void launch_rope_init(int head_dim, float theta_base);

/* No counterpart in the reference, whose converter drops the checkpoint's rope_scaling entry
 * (engine/convert_model.py:54) and whose table is always theta^(-2d/head_dim) (kernels.hip:133-134).
 * t12_rope_freqs writes head_dim / 2 inverse frequencies on the host: that table, and for factor > 0 the
 * "llama3" rule on top of it -- wavelengths (2 pi / freq) above original_ctx / low_freq_factor are divided
 * by factor, those below original_ctx / high_freq_factor are kept, the band between is blended linearly in
 * original_ctx / wavelength.  launch_rope_scaling makes every RoPE launcher of this library use that rule from
 * then on (process-wide, like the table itself; factor <= 0 switches it off). */
void t12_rope_freqs(int head_dim, float theta, float factor, float low_freq_factor, float high_freq_factor,
                    float original_ctx, float* out);
void launch_rope_scaling(float factor, float low_freq_factor, float high_freq_factor, float original_ctx);

/* kernels.hip:142-147.  output[b, :] = f32(embd_table[token_ids[b], :]); ids outside [0, n_vocab) give zeros. */
void launch_embed_lookup(const int16_t* embd_table, const int* token_ids, float* output, int n_embd, int batch_size,
                         int n_vocab, hipStream_t stream);

/* kernels.hip:149-158.  First index of the maximum of each row of logits[batch, n_vocab] (device ints out). */
void launch_argmax(const float* logits, int* result, int n, hipStream_t stream);
void launch_argmax_batch(const float* logits, int* results, int n_vocab, int batch_size, hipStream_t stream);

/* kernels.hip:463-469.  y[b] = bf16(x[b] * rsqrt(mean(x[b]^2) + eps) * weight). */
void launch_rms_norm_bf16_batch(const float* x, const float* weight, int16_t* y, int n, float eps, int batch_size,
                                hipStream_t stream);
/* kernels.hip:471-477.  x[b] += residual[b] (stored), then as above. */
void launch_add_rms_norm_bf16_batch(float* x, const float* residual, const float* weight, int16_t* y, int n, float eps,
                                    int batch_size, hipStream_t stream);
/* The same, with x[b] first rebuilt as the ascending sum of nsplit partial rows
 * partials[z * split_stride + b * ld + i] (what t12_gemm_deferred leaves behind): the K-split reduction of
 * a decode+GEMM folded into the residual add + RMSNorm that follows it.  No counterpart in the reference. */
void launch_sum_add_rms_norm_bf16_batch(float* x, const float* partials, int nsplit, size_t split_stride, int ld,
                                        const float* residual, const float* weight, int16_t* y, int n, float eps,
                                        int batch_size, hipStream_t stream);
/* kernels.hip:479-485.  out = bf16(silu(gate) * up), [batch, n] contiguous. */
void launch_silu_mul_bf16_batch(const float* gate, const float* up, int16_t* out, int n, int batch_size,
                                hipStream_t stream);
/* kernels.hip:487-491.  y += x. */
void launch_add_batch(float* y, const float* x, int n, int batch_size, hipStream_t stream);

/* kernels.hip:848-858.  Rotate-half RoPE in place on q [batch, n_head*head_dim] and k [batch, n_head_kv*head_dim]
 * (row strides q_stride / k_stride in floats) at positions[b]. */
void launch_rope_batch(float* q, float* k, const int* positions, int head_dim, int n_head, int n_head_kv, int q_stride,
                       int k_stride, float theta, int batch_size, hipStream_t stream);
/* kernels.hip:860-874.  Symmetric INT8 per (position, kv head): cache[pos, h, :] = round(x / s), s = max|x| / 127. */
void launch_store_kv_batch(const float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k, float* scale_v,
                           const int* positions, int kv_dim, int max_seq, int n_head_kv, int head_dim, int batch_size,
                           hipStream_t stream);
/* kernels.hip:308-333.  RoPE on q and k, then the KV store of (k, v) at `position`, one launch (B = 1). */
void launch_rope_store_kv(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                          float* scale_v, int head_dim, int n_head, int n_head_kv, int position, int max_seq,
                          float theta, hipStream_t stream);
/* The same for a batch at positions[b] (all sequences write one shared cache region, as the reference's
 * batched mode does: inference.cpp:430-435).  No counterpart of its own in the reference (it issues
 * launch_rope_batch + launch_store_kv_batch). */
void launch_rope_store_kv_batch(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                float* scale_v, const int* positions, int head_dim, int n_head, int n_head_kv,
                                int q_stride, int k_stride, float theta, int batch_size, hipStream_t stream);

/* kernels.hip:589-599 / 1107-1118.  GQA decode attention of one query position over seq_len cached positions,
 * all heads, output bf16 [n_head*head_dim].  Both reference variants map to the same kernel here. */
void launch_attention_all_heads(const float* q, const int8_t* k_cache, const int8_t* v_cache, const float* scale_k,
                                const float* scale_v, int16_t* output, int n_head, int n_head_kv, int head_dim,
                                int seq_len, int max_seq, float scale, hipStream_t stream);
void launch_flash_attention(const float* q, const int8_t* k_cache, const int8_t* v_cache, const float* scale_k,
                            const float* scale_v, int16_t* output, int n_head, int n_head_kv, int head_dim, int seq_len,
                            int max_seq, float scale, hipStream_t stream);
/* kernels.hip:695-711 / 1120-1135.  Batched: sequence b attends positions 0..positions[b]; kv_stride = elements
 * between the caches of consecutive sequences (0 = one shared region). */
void launch_attention_all_heads_batch(const float* q, const int8_t* kv_k, const int8_t* kv_v, const float* scale_k,
                                      const float* scale_v, int16_t* output, const int* positions, int n_head,
                                      int n_head_kv, int head_dim, int max_seq, float scale, int batch_size,
                                      int kv_stride, hipStream_t stream);
void launch_flash_attention_batch(const float* q, const int8_t* kv_k, const int8_t* kv_v, const float* scale_k,
                                  const float* scale_v, int16_t* output, const int* positions, int n_head,
                                  int n_head_kv, int head_dim, int max_seq, float scale, int batch_size, int kv_stride,
                                  hipStream_t stream);
/* RoPE + KV store + attention in ONE launch (replaces inference.cpp:275-282: launch_rope_store_kv followed by
 * launch_attention_all_heads).  positions == NULL: every sequence is at `position`; with a position array
 * `position` is only a length hint (the largest position) for the choice of the attention kernel's form.  The
 * in-kernel fusion is used for batch_size 1 and for small batches on per-sequence caches (kv_stride != 0,
 * batch_size * n_head_kv <= 256); otherwise the RoPE/KV kernel runs first and q is left rotated.  No
 * counterpart of its own in the reference. */
void launch_rope_store_attention(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                 float* scale_v, int16_t* output, const int* positions, int position, int n_head,
                                 int n_head_kv, int head_dim, float theta, float scale, int batch_size, int kv_stride,
                                 hipStream_t stream);

/* launch_rope_store_attention for a batch whose q | k | v projection was one K-split launch of three segments
 * in this order (t12_gemm_deferred): the RoPE / KV-store kernel adds the partial sums up itself (element
 * (b, col) of the fused row = ascending sum over z < nsplit of partials[z * split_stride + b * ld + col]).  q and
 * k receive the rotated values; the v buffer is not written.  kv_stride as in launch_attention_all_heads_batch
 * (inference.cpp:430,435 pass 0): 0 = one cache region for all rows -- lock-step copies, or the rows of ONE
 * sequence's prompt at consecutive positions: all rows are stored before any row attends, so row t attends to
 * rows <= t (a causal prefill); otherwise the element distance between the regions of consecutive sequences
 * (scale arrays: kv_stride / head_dim).  No counterpart in the reference. */
void launch_rope_store_attention_partials(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v,
                                          float* scale_k, float* scale_v, int16_t* output, const int* positions,
                                          int position, int n_head, int n_head_kv, int head_dim, float theta,
                                          float scale, int batch_size, const float* partials, int nsplit,
                                          size_t split_stride, int ld, int kv_stride, hipStream_t stream);

/* The two launches above on HEAD-MAJOR cache regions: a region holds region_positions rows per KV head, laid out
 * [kv head][region_positions][head_dim] (scales [kv head][region_positions]) instead of the reference's
 * [position][kv head][head_dim] (engine/model.h:58-63, the layout every other launcher here keeps).  The workgroup of a
 * (sequence, KV head) then reads one contiguous stream; in the reference's layout it reads 128-byte pieces of rows that
 * it shares with the other KV heads' workgroups.  kv_stride: element distance between regions, as above (a region
 * still has region_positions * n_head_kv * head_dim elements).  Positions must stay below region_positions.  The
 * engine keeps its per-sequence caches this way.  No counterpart in the reference. */
void launch_rope_store_attention_regions(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                         float* scale_v, int16_t* output, const int* positions, int position, int n_head,
                                         int n_head_kv, int head_dim, float theta, float scale, int batch_size,
                                         int kv_stride, int region_positions, hipStream_t stream);
void launch_rope_store_attention_partials_regions(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v,
                                                  float* scale_k, float* scale_v, int16_t* output, const int* positions,
                                                  int position, int n_head, int n_head_kv, int head_dim, float theta,
                                                  float scale, int batch_size, const float* partials, int nsplit,
                                                  size_t split_stride, int ld, int kv_stride, int region_positions,
                                                  hipStream_t stream);

/* Process-wide choice of the decode-attention kernel form, for comparisons (set it before launching; it is read at
 * every launch, atomically, and is not a per-call argument because the reference-named launchers have fixed
 * signatures).  0: always the general attention kernel.  1 (default): shapes with a specialised kernel
 * (head_dim 128 with GQA ratio 1/2/4/8, head_dim 64 with ratio 1/4) use it in its INT8 MFMA form (scores and P.V by
 * v_mfma_i32_32x32x32_i8: Q in three INT8 limbs, the softmax weights in two, K and V as stored), and a launch without a
 * position array whose batch * n_head_kv workgroups would leave the chip idle is split along the context into
 * chunks of at least 256 positions (partial softmax per chunk, folded by the workgroup that finishes last; the
 * partial results live in a buffer the library keeps per device and stream).
 * 2: never split.  3: the specialised kernels in their fp32 FMA form.  4: same as 1.  n >= 16: chunks of at least n
 * positions. */
int t12_tune_attention(int mode);

#ifdef __cplusplus
}
#endif
#endif /* T12_GLUE_H */
