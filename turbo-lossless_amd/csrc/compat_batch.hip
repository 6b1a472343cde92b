// Reference-named batch launchers: launch_split12_batch4_async / launch_split12_batch8_async
// (decompress_v2.hip:860-901) and, at the end of the file, the three entry points of the reference's larger-batch path
// (nvidia_kernels.cu:426-584).
//
// Their interface carries the escapes not as a CSR list but as the derived
// tables of engine/model.cpp:86-160: esc_row_base[row], optional
// esc_counts[row*256 + t] and esc_vals ordered (row, col % 256, ascending col).
// The position of an escape inside esc_vals is therefore defined by the
// reference's thread mapping (256 lanes, lane t owns columns t, t+256, ...), so
// this kernel keeps that column ownership; everything else is this library's:
// esc_counts may be NULL (each lane then counts its own group-0 nibbles) and any
// batch size 1..8 is one template.  That ownership (one column per lane and step,
// byte loads) is also what bounds this kernel; it exists for callers that hold the
// derived tables -- the engine itself sends batches of 2..8 through t12_gemm, which
// reads the CSR list and streams 16 columns per lane.
#include "t12_device.h"
#include "t12_host.h"

namespace {

struct BatchPtrs {
    const uint16_t* act[8];
    float* out[8];
};

template <int NB>
__global__ __launch_bounds__(256) void compat_batch_kernel(const uint8_t* __restrict__ sm,
                                                           const uint8_t* __restrict__ gr, int base_exp,
                                                           const BatchPtrs bp, const int32_t* __restrict__ esc_row_base,
                                                           const uint8_t* __restrict__ esc_counts,
                                                           const int16_t* __restrict__ esc_vals, int M, int K)
{
    __shared__ int wave_tot[4];
    __shared__ float red[4][NB];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t base = (size_t)row * K;

    // this lane's first slot in esc_vals
    int esc_ptr = 0;
    if (esc_row_base) {
        int mine = 0;
        if (esc_counts) mine = esc_counts[(size_t)row * 256 + tid];
        else
            for (int k = tid; k < K; k += 256) {
                const size_t i = base + k;
                mine += ((gr[i >> 1] >> (4 * (i & 1))) & 0xF) == 0;
            }
        int incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, T12_WAVE);
            if (lane >= off) incl += v;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int before = 0;
        for (int w = 0; w < wave; w++) before += wave_tot[w];
        esc_ptr = esc_row_base[row] + before + incl - mine;
    }

    float acc[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) acc[j] = 0.0f;
    for (int k = tid; k < K; k += 256) {
        const size_t i = base + k;
        const uint32_t g = (gr[i >> 1] >> (4 * (i & 1))) & 0xFu;
        uint16_t w = t12_decode_scalar(sm[i], g, base_exp);
        if (g == 0 && esc_vals) w = (uint16_t)esc_vals[esc_ptr++];
        const float wf = t12_bf16_to_f32(w);
#pragma unroll
        for (int j = 0; j < NB; j++) acc[j] += wf * t12_bf16_to_f32(bp.act[j][k]);
    }
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const float v = t12_wave_sum(acc[j]);
        if (lane == 0) red[wave][j] = v;
    }
    __syncthreads();
    if (tid < NB) bp.out[tid][row] = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
}

template <int NB>
int launch(const void* sm, const void* gr, int base_exp, const void* const* a, const void* rb, const void* cnt,
           const void* vals, void* const* o, int M, int K, void* stream)
{
    if (M == 0) return 0;
    T12_REQUIRE(sm && gr && M > 0 && K > 0, "launch_split12_batch%d_async: null plane or bad shape", NB);
    T12_REQUIRE(base_exp >= -1 && base_exp <= 254, "launch_split12_batch%d_async: base_exp out of range", NB);
    T12_REQUIRE((rb == nullptr) == (vals == nullptr), "launch_split12_batch%d_async: esc_row_base and esc_vals go together", NB);
    BatchPtrs bp;
    for (int j = 0; j < NB; j++) {
        T12_REQUIRE(a[j] && o[j], "launch_split12_batch%d_async: null activation/output %d", NB, j);
        bp.act[j] = (const uint16_t*)a[j];
        bp.out[j] = (float*)o[j];
    }
    hipLaunchKernelGGL(compat_batch_kernel<NB>, dim3(M), dim3(256), 0, (hipStream_t)stream, (const uint8_t*)sm,
                       (const uint8_t*)gr, base_exp, bp, (const int32_t*)rb, (const uint8_t*)cnt,
                       (const int16_t*)vals, M, K);
    T12_CHECK_LAUNCH("launch_split12_batch");
    return T12_OK;
}


// nv_apply_patches_batch (nvidia_kernels.cu:295-319): one thread per (listed row, batch row) pair walks the row's
// escape slice: out[b, row] += sum over entries of (correct - wrong) * x[b, col]; nothing is written when the sum is 0.
__global__ __launch_bounds__(256) void patches_batch_kernel(const int32_t* __restrict__ row_off, const int32_t* __restrict__ cols,
                                                            const int16_t* __restrict__ correct, const int16_t* __restrict__ wrong,
                                                            const int32_t* __restrict__ rows, const uint16_t* __restrict__ act,
                                                            int act_stride, float* __restrict__ out, int out_stride, int n_rows,
                                                            int B)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int ri = (int)(idx / B), b = (int)(idx % B);
    if (ri >= n_rows) return;
    const int row = rows[ri];
    const uint16_t* x = act + (size_t)b * act_stride;
    float c = 0.0f;
    for (int q = row_off[row]; q < row_off[row + 1]; q++)
        c += (t12_bf16_to_f32((uint16_t)correct[q]) - t12_bf16_to_f32((uint16_t)wrong[q])) * t12_bf16_to_f32(x[cols[q]]);
    if (c != 0.0f) out[(size_t)b * out_stride + row] += c;
}

}  // namespace

extern "C" {

int launch_split12_batch4_async(const void* sm, const void* gr, int base_exp, const void* a0, const void* a1,
                                const void* a2, const void* a3, const void* esc_row_base, const void* esc_counts,
                                const void* esc_vals, void* o0, void* o1, void* o2, void* o3, int M, int K,
                                void* stream)
{
    const void* a[4] = {a0, a1, a2, a3};
    void* o[4] = {o0, o1, o2, o3};
    return launch<4>(sm, gr, base_exp, a, esc_row_base, esc_counts, esc_vals, o, M, K, stream);
}

int launch_split12_batch8_async(const void* sm, const void* gr, int base_exp, const void* a0, const void* a1,
                                const void* a2, const void* a3, const void* a4, const void* a5, const void* a6,
                                const void* a7, const void* esc_row_base, const void* esc_counts, const void* esc_vals,
                                void* o0, void* o1, void* o2, void* o3, void* o4, void* o5, void* o6, void* o7, int M,
                                int K, void* stream)
{
    const void* a[8] = {a0, a1, a2, a3, a4, a5, a6, a7};
    void* o[8] = {o0, o1, o2, o3, o4, o5, o6, o7};
    return launch<8>(sm, gr, base_exp, a, esc_row_base, esc_counts, esc_vals, o, M, K, stream);
}

// ---- the reference's entry points for larger batches (nvidia_kernels.cu:426-584), same names and arguments ----

// out[b, m] = sum_k dec(W[m, k]) * X[b, k]; escapes exact when the four list pointers are given, "wrong" values when
// they are null (the reference's V1 kernel adds the correction in its epilogue under the same condition,
// split12_gemm.cuh:273-284).  The reference reads the activations with a row stride of K whatever act_stride says
// (nvidia_kernels.cu:446,467); its callers pass K, and this entry point honours the argument.
int nv_launch_split12_fused_gemm_async(const void* sm, const void* gr, int base_exp, const void* act, int act_stride,
                                       void* out, int out_stride, int M, int K, int B, void* stream,
                                       const void* patch_row_off, const void* patch_cols, const void* patch_correct,
                                       const void* patch_wrong)
{
    const bool lists = patch_row_off && patch_cols && patch_correct && patch_wrong;
    T12Segment g = {(const uint8_t*)sm, (const uint8_t*)gr, lists ? (const int32_t*)patch_row_off : nullptr,
                    lists ? (const int32_t*)patch_cols : nullptr, lists ? (const int16_t*)patch_correct : nullptr,
                    lists ? (const int16_t*)patch_wrong : nullptr, (float*)out, M, base_exp, out_stride, 0};
    return t12_gemm(&g, 1, act, act_stride, out_stride, K, B, stream);
}

// The separate correction launch that follows an unpatched GEMM in the reference (nvidia_kernels.cu:426-442).
int nv_launch_patches_batch_async(const void* row_off, const void* cols, const void* correct, const void* wrong,
                                  const void* nonempty_rows, int num_nonempty, const void* act, int act_stride, void* out,
                                  int out_stride, int B, void* stream)
{
    if (num_nonempty == 0 || B == 0) return 0;
    T12_REQUIRE(row_off && cols && correct && wrong && nonempty_rows && act && out && num_nonempty > 0 && B > 0,
                "nv_launch_patches_batch_async: null operand or negative count");
    const long pairs = (long)num_nonempty * B;
    hipLaunchKernelGGL(patches_batch_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const int32_t*)row_off, (const int32_t*)cols, (const int16_t*)correct, (const int16_t*)wrong,
                       (const int32_t*)nonempty_rows, (const uint16_t*)act, act_stride, (float*)out, out_stride, num_nonempty, B);
    T12_CHECK_LAUNCH("nv_launch_patches_batch_async");
    return T12_OK;
}

// The reference decodes the tensor (unpatched) into bf16_weight_buf and calls a vendor GEMM on it
// (nvidia_kernels.cu:550-584).  Here the same product comes from the fused decode+GEMM: the buffer is not touched.
int nv_launch_split12_cublas_batch_async(const void* sign_mantissa, const void* groups, int base_exp, const void* activations,
                                         int act_stride, void* output, int out_stride, void* bf16_weight_buf,
                                         int buf_half_elems, int M, int K, int B, void* stream)
{
    (void)bf16_weight_buf;
    (void)buf_half_elems;
    T12Segment g = {(const uint8_t*)sign_mantissa, (const uint8_t*)groups, nullptr, nullptr, nullptr, nullptr, (float*)output,
                    M, base_exp, out_stride, 0};
    return t12_gemm(&g, 1, activations, act_stride, out_stride, K, B, stream);
}

// The B = 1 entry points under the names the reference's other build uses (nvidia_kernels.cu:385-424): same
// arguments and meaning as launch_split12_v2_async / _v2_dual_async / launch_patches_v2_async.
int nv_launch_split12_v2_async(const void* sm, const void* gr, int base_exp, const void* act, void* out, int M, int K,
                               void* stream)
{
    return launch_split12_v2_async(sm, gr, base_exp, act, out, M, K, stream);
}

int nv_launch_split12_v2_dual_async(const void* sm_a, const void* gr_a, int base_exp_a, const void* sm_b, const void* gr_b,
                                    int base_exp_b, const void* act, void* out_a, void* out_b, int M, int K, void* stream)
{
    return launch_split12_v2_dual_async(sm_a, gr_a, base_exp_a, sm_b, gr_b, base_exp_b, act, out_a, out_b, M, K, stream);
}

int nv_launch_patches_async(const void* row_off, const void* cols, const void* correct, const void* wrong, const void* act,
                            void* out, int M, void* stream)
{
    return launch_patches_v2_async(row_off, cols, correct, wrong, act, out, M, stream);
}

// Small-batch entry point: 1 <= B <= 8 rows of activations; same contract as t12_gemm.
int t12_gemv_batch(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K,
                   int B, void* stream)
{
    T12_REQUIRE(B >= 1 && B <= 8, "t12_gemv_batch: B must be 1..8 (got %d)", B);
    if (B == 1) return t12_gemv(segs, nseg, act_bf16, K, stream);
    return t12_gemm(segs, nseg, act_bf16, act_stride, out_stride, K, B, stream);
}

}  // extern "C"
