/*
 * t12_abi.h -- C ABI of libturbo12.so: split-12 fused decode + GEMV / GEMM,
 * standalone decompress and the engine glue kernels, hand-written for gfx950.
 *
 * Conventions (the same as the reference's launch layer, engine/inference.cpp:7-41):
 * extern "C", plain device pointers and sizes, the HIP stream passed as an
 * opaque pointer, launches are asynchronous on that stream, no ownership is
 * transferred.  Unlike the reference every entry point validates its operands
 * on the host and checks the launch; the return value is 0 on success and a
 * negative T12_E* code otherwise (t12_last_error() gives the text).
 *
 * Data layout (byte-exact with what split12_pack.c:47-128 emits):
 *   sm   u8  [M*K]        (sign << 7) | mantissa7, row-major
 *   gr   u8  [(M*K+1)/2]  4-bit group per element, flat index i -> byte i/2,
 *                         low nibble for even i; group = exponent - base_exp in
 *                         1..15, 0 = escape
 *   CSR  row_off i32[M+1], cols i32[P] (ascending in a row), correct i16[P]
 *        (exact bf16 bits), wrong i16[P] (what the plain rule yields for group 0)
 *   activations  bf16 [B, K] row-major (row stride act_stride elements)
 *   outputs      fp32 out[b * out_stride + m]
 */
#ifndef T12_ABI_H
#define T12_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define T12_OK          0
#define T12_EINVAL     (-1)   /* bad shape / null pointer / unsupported size */
#define T12_ELAUNCH    (-2)   /* HIP reported a launch or runtime error      */
#define T12_EENGINE    (-3)   /* a t12_engine_* call failed (EngineError)    */
#define T12_MAX_SEGMENTS 8
#define T12_MAX_KSPLIT 16      /* most K splits a decode+GEMM launch uses (T12GemmPartials.nsplit) */

/* One weight tensor of a fused launch.  Several tensors that consume the same
 * activations (wq|wk|wv, gate|up, the experts of one token group) are passed as
 * a segment table so that one launch fills the whole chip; each keeps its own
 * base_exp (replaces the pair of base_exp arguments of
 * launch_split12_v2_dual_async, decompress_v2.hip:549, and the
 * PatchBatchDesc table of decompress_v2.hip:36-44).  All pointers are device
 * pointers.  row_off == NULL means "no escape list": group-0 elements then
 * decode to the wrong value, exactly like the reference's unpatched kernels. */
typedef struct T12Segment {
    const uint8_t* sm;
    const uint8_t* gr;
    const int32_t* row_off;
    const int32_t* cols;
    const int16_t* correct;
    const int16_t* wrong;
    float*         out;        /* this tensor's output base: out[b*out_stride + m] */
    int32_t        M;
    int32_t        base_exp;
    int32_t        out_stride; /* row stride of `out` for B > 1; 0 = the call's out_stride */
    int32_t        reserved;   /* must be 0 */
} T12Segment;

/* ---- library ------------------------------------------------------------- */
const char* t12_version(void);
const char* t12_last_error(void);      /* text of the last failure on this thread */

/* dst[0..n) = src[0..n) (32-bit words) by a kernel; dst may be pinned host memory (the engine's sampled ids reach the
 * host this way, without a DMA-engine hand-over in the middle of the stream).  No counterpart in the reference. */
int t12_util_copy_i32(void* dst, const void* src, int n, void* stream);

/* Measurement aid, no counterpart in the reference: the shader clock under load.  Runs `workgroups` workgroups of
 * eight waves, each wave `iters` rounds of four independent v_mfma_f32_32x32x16_bf16 on pseudo-random operands
 * (mix = 0), or the same with what a decode+GEMM stage adds per round (mix = 1: two packed 8-weight decodes, two
 * 16-byte LDS writes, four 16-byte LDS reads), and reports the clock the waves saw (shader-clock counter against
 * the constant 100 MHz counter, mean over the workgroups, GHz) and the dense bf16 MFMA rate of the launch (TFLOP/s).
 * Synchronous.  The published 2.5 PFLOP/s is 256 CUs x 4 SIMDs x 1024 flop/clk at 2.4 GHz; bench.py prints the
 * measured clock beside the MFMA roofline. */
int t12_probe_clock(int workgroups, int iters, int mix, double* ghz, double* tflops, void* stream);

/* Measurement aid, no counterpart in the reference: the time per launch (us) of a chain of `launches` one-wave
 * kernels that do nothing, on `stream`, as the GPU paces them (a first kernel holds the stream for 4 us per launch
 * while the host enqueues the chain; the clock runs from its end).  any_order = 0: ordinary stream order (each kernel waits for the one
 * before it), the floor under a chain of dependent launches such as the B = 1 decode step.  any_order = 1: the
 * launches carry hipExtAnyOrderLaunch, which lifts the ordering between them -- such kernels overlap, so it is
 * no option for launches that read what their predecessor wrote; the difference is what the ordering costs.
 * Synchronous. */
int t12_probe_launch_gap(int launches, int any_order, double* us_per_launch, void* stream);

/* ---- (a) decode-GEMV, one activation vector ------------------------------
 * out_s[m] = sum_k dec(W_s[m,k]) * x[k] for every segment s, escapes exact.
 * Replaces launch_split12_v2_async (decompress_v2.hip:530) +
 * launch_split12_v2_dual_async (:549) + launch_patches_v2_async (:113) +
 * launch_patches_b1_batched_async (:129) with one launch.  `segs` is a HOST
 * array (it travels as a kernel argument; no device copy is made). */
int t12_gemv(const T12Segment* segs, int nseg, const void* act_bf16, int K, void* stream);

/* out[m] = residual[m] + W[m,:] . act (one segment): the residual add that follows wo / w_down
 * (first half of add_rms_norm_bf16_batch, engine/kernels.hip:399-442, inference.cpp:301,343) folded into
 * the store of the decode-GEMV.  out and residual may not alias. */
int t12_gemv_add(const T12Segment* seg, const void* act_bf16, int K, const float* residual, void* stream);

/* SwiGLU front half in one launch: out_bf16[m] = bf16( silu(gate[m,:].x) * (up[m,:].x) ).
 * Replaces launch_split12_v2_dual_async (decompress_v2.hip:549) + its patch launch +
 * launch_silu_mul_bf16_batch (engine/kernels.hip:480); bit-identical to that sequence.
 * Requires gate->M == up->M, K % 16 == 0, base_exp in 0..240. */
int t12_gemv_swiglu(const T12Segment* gate, const T12Segment* up, const void* act_bf16, int K,
                    void* out_bf16, void* stream);

/* The same two entry points with the reference's RMSNorm kernels folded into the prologue:
 * activations = bf16( rmsnorm(x [+ residual]) * norm_w ), x / residual / norm_w fp32 [K]
 * (engine/kernels.hip:355-442).  residual may be NULL (plain RMSNorm).  hidden_out, if not
 * NULL, receives x + residual (the updated residual stream) and may not alias x or residual.
 * Requires K % 16 == 0, K <= 8192, base_exp in 0..240. */
int t12_gemv_norm(const T12Segment* segs, int nseg, const float* x, const float* residual,
                  const float* norm_w, float eps, float* hidden_out, int K, void* stream);
int t12_gemv_swiglu_norm(const T12Segment* gate, const T12Segment* up, const float* x,
                         const float* residual, const float* norm_w, float eps, float* hidden_out,
                         int K, void* out_bf16, void* stream);

/* ---- (a') small batch, 1 <= B <= 8 -----------------------------------------
 * Same contract as t12_gemm, restricted to the batch sizes of the reference's
 * launch_split12_batch4_async / _batch8_async (decompress_v2.hip:860,877), with
 * the escapes taken from the CSR list instead of the derived escape tables. */
int t12_gemv_batch(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride,
                   int out_stride, int K, int B, void* stream);

/* ---- (b) decode+GEMM, any B >= 1 ------------------------------------------
 * out_s[b*out_stride + m] = sum_k dec(W_s[m,k]) * X[b*act_stride + k], bf16 MFMA with
 * fp32 accumulation, escapes exact.  B <= 16 (K a multiple of 128): kernels bound by the
 * weight stream, no K split (B = 2: whole-row waves with two accumulators, v_dot2; else
 * 16-row groups swept whole by eight waves, 16x16x32 MFMA; the same sweep up to B = 32 on
 * tensors of few, short rows); larger B: 128-row tiles staged
 * through LDS, K split across workgroups when the tiles alone do not fill the chip.  Replaces
 * nv_launch_split12_fused_gemm_async (nvidia_kernels.cu:444) +
 * nv_launch_patches_batch_async (:426) + nv_launch_split12_cublas_batch_async (:550). */
int t12_gemm(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride,
             int out_stride, int K, int B, void* stream);

/* t12_gemm with the last step left to the caller: when the launch splits K across workgroups, the
 * partial sums stay in the library's per-device workspace and *part describes them,
 *   value[b, m] = sum over z < nsplit (ascending) of ws[z * split_stride + b * ld + (segment's first column) + m],
 * so that the caller's next kernel (launch_sum_add_rms_norm_bf16_batch) adds them up while it reads
 * them anyway.  nsplit == 1: nothing was split, the outputs are complete in segs[].out.  The workspace is
 * reused by the next t12_gemm* call on the device: consume the partials first (same stream).  No
 * counterpart in the reference (its GEMM never splits K). */
typedef struct T12GemmPartials {
    const float* ws;
    int          nsplit;
    int          ld;            /* floats between consecutive batch rows of one split (sum of M over segments) */
    size_t       split_stride;  /* floats between consecutive splits */
} T12GemmPartials;
int t12_gemm_deferred(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride,
                      int out_stride, int K, int B, T12GemmPartials* part, void* stream);
/* out_bf16[b*out_stride + m] = bf16( silu(gate[m,:] . X[b,:]) * (up[m,:] . X[b,:]) ): the gate|up projection with
 * silu_mul_bf16 (engine/kernels.hip:447-459, inference.cpp:327) in the GEMM's epilogue -- no fp32 round trip of
 * the two projections.  Returns 0 when launched, 1 when the shape has no fused kernel (B <= 64 other than 5 .. 8, few rows, K not
 * a multiple of 64, base_exp outside 0..240): run t12_gemm on the two segments and launch_silu_mul_bf16_batch
 * then; negative on bad operands. */
int t12_gemm_swiglu(const T12Segment* gate, const T12Segment* up, const void* act_bf16, int act_stride,
                    int K, int B, void* out_bf16, int out_stride, void* stream);

/* Several decode+GEMM products in one launch, group i multiplying its own activations:
 *   seg.out[b*seg.out_stride + m] = sum_k dec(W_i[m,k]) * X_i[b*act_stride + k],  b < B   (B == 0: group skipped)
 * for the experts of a mixture-of-experts layer (each expert over the rows routed to it; gate and up of one expert
 * are two groups with the same activations).  Every group runs on the tile kernel (also groups of 16 rows or
 * fewer, which t12_gemm would give to its weight-stream kernels): the values are those of one t12_gemm per group
 * up to the order of the fp32 sums.  Up to 16 groups.  No counterpart in the reference, whose entry point (nv_launch_split12_fused_gemm_async,
 * nvidia_kernels.cu:444) takes one tensor and would be called once per expert. */
typedef struct T12Group {
    T12Segment  seg;          /* the tensor and its output (out, out_stride must be set) */
    const void* act_bf16;     /* [B, act_stride] */
    int         act_stride;
    int         B;
} T12Group;
int t12_gemm_grouped(const T12Group* groups, int ngroups, int K, void* stream);

/* A mixture-of-experts SwiGLU feed-forward layer over split-12 experts (a Mixtral-shaped layer):
 *   out[t, :] = sum_j weights[t*k + j] * W2_e( silu(W1_e x_t) * (W3_e x_t) ),  e = expert_ids[t*k + j],  j ascending
 * x bf16 [T, x_stride]; expert_ids [T, k] int32 or int64 (id_bytes 4 / 8) and weights [T, k] fp32 on the device;
 * out fp32 [T, out_stride].  The (token, slot) pairs are grouped per expert on the GPU, gate|up and down of all experts
 * run as grouped decode+GEMM launches (the SwiGLU activation rounded to bf16 in between, as the engine does,
 * inference.cpp:327; in the gate|up epilogue when the experts receive more than 128 rows each), and the weighted sum
 * is taken in a fixed order.  The call never waits for the stream: the grouped launches read the rows per expert from
 * the routing kernel's tables on the device (one workgroup per row tile, which walks the expert's batch tiles; with
 * few rows per expert -- a decode step -- the small-batch kernel that sweeps 16 whole weight rows per workgroup, and
 * an expert nobody names costs a workgroup's exit; with at most eight (token, expert) pairs on at most eight experts
 * of 2048 columns and more, every pair is one matrix-vector product with its expert's tensors, picked on the device,
 * gate|up with the SwiGLU in the epilogue).  An id
 * outside 0..E-1 leaves its pair out of the sum and raises a flag that t12_moe_status reads (it waits for the stream).
 * Shapes the tile kernel does not take (n_embd or n_ff not a multiple of 64, base_exp outside 0..240) copy the counts
 * to the host and wait once per call.
 * workspace: device memory of t12_moe_workspace_bytes(...) bytes, 256-byte aligned, owned by the caller (used from the
 * first launch to the last).  Up to 128 experts; w1, w3 are [n_ff, n_embd], w2 is [n_embd, n_ff]; their out fields are
 * ignored.  No counterpart in the reference (no MoE layer there); what it replaces is one
 * nv_launch_split12_fused_gemm_async (nvidia_kernels.cu:444) per expert and projection. */
typedef struct T12MoeExpert {
    T12Segment w1, w3, w2;
} T12MoeExpert;
size_t t12_moe_workspace_bytes(int T, int k, int n_embd, int n_ff, int E);
int t12_moe_ffn(const T12MoeExpert* experts, int E, const void* x_bf16, int x_stride, const void* expert_ids,
                int id_bytes, const float* weights, int T, int k, int n_embd, int n_ff, void* workspace,
                size_t workspace_bytes, float* out, int out_stride, void* stream);
int t12_moe_status(const void* workspace, void* stream);

/* t12_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference (its GEMM never splits K and so has no
 * workspace).  Same operands, kernels, K split and results as t12_gemm, bit for bit; the partial sums of a
 * K-split launch go to a fixed array of T12_GEMM_NOALLOC_WS_BYTES inside the library's device image (every GPU
 * the library runs on holds one until the process ends) and the call never calls hipMalloc / hipFree.  A launch
 * whose partial sums (nsplit * B * sum of M * 4 bytes) exceed the array is refused with T12_EINVAL.  All calls on
 * one GPU share the array: calls that overlap in time on one GPU, on any streams, race. */
#define T12_GEMM_NOALLOC_WS_BYTES (32u << 20)
int t12_gemm_noalloc(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride,
                     int out_stride, int K, int B, void* stream);

/* The library keeps device buffers per (device, stream): K-split partial sums of t12_gemm / _deferred / _grouped, argmax
 * partials and context-split buffers of the glue launchers.  t12_release_stream waits for the stream and frees those of
 * (current device, stream); call it before destroying a stream (free_inference_state does).  A launch that needs a
 * larger buffer than any before it on its stream calls hipMalloc once (sizes double, so this happens a few times per
 * stream) and keeps the outgrown buffer until t12_release_stream rather than freeing it, so no launch call waits for
 * the device; only when that hipMalloc fails are the outgrown buffers freed inside the call (a device-wide wait)
 * before one more attempt.  Callers that cannot allocate at all use t12_gemm_noalloc.  No counterpart in the
 * reference, which keeps no such buffers. */
int t12_release_stream(void* stream);

/* ---- (c) standalone decompress --------------------------------------------
 * out_bf16[m*K + k] = decoded weight bits.  patched != 0: escapes take
 * `correct` (lossless, bit-exact with the tensor that was packed).
 * patched == 0 (or row_off NULL): the reference's nv_decode_split12_to_bf16
 * semantics (nvidia_kernels.cu:533-548): escapes keep the wrong value. */
int t12_decompress(const void* sm, const void* gr, int base_exp, const void* row_off,
                   const void* cols, const void* correct, void* out_bf16,
                   int M, int K, int patched, void* stream);

/* ---- GPU-side packer ---------------------------------------------------------
 * The reference packs on one CPU thread (split12_pack.c); these entry points
 * produce byte-identical arrays from a bf16 matrix resident in HBM.
 *   t12_pack_histogram : 256-bin histogram of the exponent byte (u64 counters,
 *                        zeroed by the call)                  split12_pack.c:20-24
 *   t12_pack_base_exp  : HOST function, window rule on a host copy of the
 *                        histogram                            split12_pack.c:26-36
 *   t12_pack_planes    : sm, gr and per-row escape counts (i32[M], zeroed by
 *                        the call)                            split12_pack.c:76-97
 *   t12_pack_row_offsets: exclusive scan -> row_off[M+1]      split12_pack.c:99-101
 *   t12_pack_escapes   : cols / correct / wrong in CSR order  split12_pack.c:103-124
 * The caller reads row_off[M] (= P) back to size the three escape arrays. */
int t12_pack_histogram(const void* w_bf16, size_t n, void* hist_u64x256, void* stream);
int t12_pack_base_exp(const uint64_t* hist_host);
int t12_pack_planes(const void* w_bf16, int M, int K, int base_exp, void* sm, void* gr, void* row_cnt,
                    void* stream);
int t12_pack_row_offsets(const void* row_cnt, int M, void* row_off, void* stream);
int t12_pack_escapes(const void* w_bf16, int M, int K, int base_exp, const void* row_off, void* cols,
                     void* correct, void* wrong, void* stream);

/* ---- reference-named launchers (same signatures and semantics) -------------
 * For host code written against the reference's launch layer.
 * decompress_v2.hip:530,549,113,129,860,877 */
int launch_split12_v2_async(const void* sign_mantissa, const void* groups, int base_exp,
                            const void* activations, void* output, int M, int K, void* stream);
int launch_split12_v2_dual_async(const void* sm_a, const void* gr_a, int base_exp_a,
                                 const void* sm_b, const void* gr_b, int base_exp_b,
                                 const void* activations, void* output_a, void* output_b,
                                 int M, int K, void* stream);
int launch_patches_v2_async(const void* row_offsets, const void* patch_cols, const void* correct_vals,
                            const void* wrong_vals, const void* activations, void* output, int M,
                            void* stream);
int launch_patches_v2(const void* row_offsets, const void* patch_cols, const void* correct_vals,
                      const void* wrong_vals, const void* activations, void* output, int M);

/* Must match the reference's PatchBatchDesc (decompress_v2.hip:36-44): 56 bytes. */
typedef struct PatchBatchDesc {
    const int32_t* row_offsets;
    const int32_t* patch_cols;
    const int16_t* patch_correct;
    const int16_t* patch_wrong;
    const int16_t* activations;
    float*         output;
    int            M;
} PatchBatchDesc;
int launch_patches_b1_batched_async(void* descs_gpu, const void* descs_cpu, int num_descs,
                                    int max_M, void* stream);
/* Batches of 4 / 8 with the escapes as the derived tables of the reference's loader (engine/model.cpp:86-160):
 * esc_vals ordered (row, col % 256, ascending col), esc_row_base[row] = first slot of the row, esc_counts optional and
 * unused when K % 128 == 0 (both table pointers NULL: the unpatched product).  K % 128 == 0, K <= 65536, base_exp in
 * 0..240 and 16-byte aligned planes and activations stream the planes like t12_gemm at B <= 16 and place every escape by
 * its rank within its row; other shapes keep the reference's column ownership (one column per lane and step). */
int launch_split12_batch4_async(const void* sm, const void* gr, int base_exp,
                                const void* a0, const void* a1, const void* a2, const void* a3,
                                const void* esc_row_base, const void* esc_counts, const void* esc_vals,
                                void* o0, void* o1, void* o2, void* o3, int M, int K, void* stream);
int launch_split12_batch8_async(const void* sm, const void* gr, int base_exp,
                                const void* a0, const void* a1, const void* a2, const void* a3,
                                const void* a4, const void* a5, const void* a6, const void* a7,
                                const void* esc_row_base, const void* esc_counts, const void* esc_vals,
                                void* o0, void* o1, void* o2, void* o3,
                                void* o4, void* o5, void* o6, void* o7, int M, int K, void* stream);

/* The reference's larger-batch entry points (nvidia_kernels.cu:444-524, 426-442, 550-584), same names and arguments.
 * fused_gemm: out[b*out_stride + m] = sum_k dec(W[m,k]) * act[b*act_stride + k], escapes exact when all four list
 * pointers are non-NULL, "wrong" values otherwise.  patches_batch: the separate correction launch over the listed
 * rows, out[b*out_stride + row] += sum (correct - wrong) * act[b*act_stride + col].  cublas_batch: the unpatched
 * product; the reference decodes into bf16_weight_buf and calls a vendor GEMM, this build runs the fused kernel and
 * leaves the buffer alone. */
int nv_launch_split12_v2_async(const void* sm, const void* gr, int base_exp, const void* act, void* out, int M, int K,
                               void* stream);                                   /* nvidia_kernels.cu:385 = launch_split12_v2_async */
int nv_launch_split12_v2_dual_async(const void* sm_a, const void* gr_a, int base_exp_a, const void* sm_b, const void* gr_b,
                                    int base_exp_b, const void* act, void* out_a, void* out_b, int M, int K,
                                    void* stream);                              /* :402 = launch_split12_v2_dual_async */
int nv_launch_patches_async(const void* row_off, const void* cols, const void* correct, const void* wrong, const void* act,
                            void* out, int M, void* stream);                    /* :414 = launch_patches_v2_async */
int nv_launch_split12_fused_gemm_async(const void* sm, const void* gr, int base_exp, const void* act, int act_stride,
                                       void* out, int out_stride, int M, int K, int B, void* stream,
                                       const void* patch_row_off, const void* patch_cols, const void* patch_correct,
                                       const void* patch_wrong);
int nv_launch_patches_batch_async(const void* row_off, const void* cols, const void* correct, const void* wrong,
                                  const void* nonempty_rows, int num_nonempty, const void* act, int act_stride,
                                  void* out, int out_stride, int B, void* stream);
int nv_launch_split12_cublas_batch_async(const void* sign_mantissa, const void* groups, int base_exp,
                                         const void* activations, int act_stride, void* output, int out_stride,
                                         void* bf16_weight_buf, int buf_half_elems, int M, int K, int B, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* T12_ABI_H */
