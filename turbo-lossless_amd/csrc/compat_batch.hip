// Reference-named batch launchers: launch_split12_batch4_async / launch_split12_batch8_async
// (decompress_v2.hip:860-901) and, at the end of the file, the three entry points of the reference's larger-batch path
// (nvidia_kernels.cu:426-584).
//
// Their interface carries the escapes not as a CSR list but as the derived
// tables of engine/model.cpp:86-160: esc_row_base[row], optional
// esc_counts[row*256 + t] and esc_vals ordered (row, col % 256, ascending col).
// The position of an escape inside esc_vals is therefore defined by the
// reference's thread mapping (256 lanes, lane t owns columns t, t+256, ...).
// Two kernels compute the same function:
//   * compat_sweep_kernel (K % 128 == 0, K <= 65536, 0 <= base_exp <= 240, 16-byte aligned operands): the planes are
//     streamed the way the library's small-batch GEMM streams them (16-row groups, 16-byte pieces straight into MFMA
//     operands, "wrong" values multiplied); the columns of the group-0 nibbles met on the way are collected per row,
//     ranked by (col % 256, col) -- which is their position in esc_vals -- and the products are corrected by
//     (correct - wrong) * x[col] in rank order (a fixed order: results do not depend on timing);
//   * compat_batch_kernel, the reference's column ownership itself (one column per lane and step, byte loads): any
//     shape, esc_counts used when given; also what a workgroup of the first kernel falls back to for rows with more
//     escapes than its LDS list holds.
#include "t12_device.h"
#include "t12_host.h"

namespace {

struct BatchPtrs {
    const uint16_t* act[8];
    float* out[8];
};

// One row the reference's way, by the 256 threads t = 0..255 of a workgroup (work == false: a thread that only keeps
// the barriers company).  wave_tot[4] and red[4][NB] are LDS scratch; the call ends with a barrier, so they can be
// reused at once.
template <int NB>
__device__ __forceinline__ void compat_row_256(const uint8_t* __restrict__ sm, const uint8_t* __restrict__ gr, int base_exp,
                                               const BatchPtrs& bp, const int32_t* __restrict__ esc_row_base,
                                               const uint8_t* __restrict__ esc_counts, const int16_t* __restrict__ esc_vals,
                                               int row, int K, int t, bool work, int* wave_tot, float (*red)[NB])
{
    const int lane = t & 63, wave = (t >> 6) & 3;
    const size_t base = (size_t)row * K;

    // this lane's first slot in esc_vals
    int esc_ptr = 0;
    if (esc_row_base) {
        int mine = 0;
        if (work) {
            if (esc_counts) mine = esc_counts[(size_t)row * 256 + t];
            else
                for (int k = t; k < K; k += 256) {
                    const size_t i = base + k;
                    mine += ((gr[i >> 1] >> (4 * (i & 1))) & 0xF) == 0;
                }
        }
        int incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, T12_WAVE);
            if (lane >= off) incl += v;
        }
        if (work && lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        if (work) {
            int before = 0;
            for (int w = 0; w < wave; w++) before += wave_tot[w];
            esc_ptr = esc_row_base[row] + before + incl - mine;
        }
    }

    float acc[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) acc[j] = 0.0f;
    if (work)
        for (int k = t; k < K; k += 256) {
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
        if (work && lane == 0) red[wave][j] = v;
    }
    __syncthreads();
    if (work && t < NB) {
#pragma unroll
        for (int j = 0; j < NB; j++)
            if (t == j) bp.out[j][row] = red[0][j] + red[1][j] + red[2][j] + red[3][j];
    }
    __syncthreads();
}

template <int NB>
__global__ __launch_bounds__(256) void compat_batch_kernel(const uint8_t* __restrict__ sm,
                                                           const uint8_t* __restrict__ gr, int base_exp,
                                                           const BatchPtrs bp, const int32_t* __restrict__ esc_row_base,
                                                           const uint8_t* __restrict__ esc_counts,
                                                           const int16_t* __restrict__ esc_vals, int M, int K)
{
    __shared__ int wave_tot[4];
    __shared__ float red[4][NB];
    compat_row_256<NB>(sm, gr, base_exp, bp, esc_row_base, esc_counts, esc_vals, blockIdx.x, K, threadIdx.x,
                       (int)blockIdx.x < M, wave_tot, red);
}

// ---------------------------------------------------------------------------
// The streaming form.  A workgroup = CB_NW waves owns 16 consecutive rows and all of K; wave w takes the 128-column
// blocks w, w + CB_NW, ... of the rows.  v_mfma_f32_16x16x32_bf16 with the activations as A operand (rows = batch;
// the rows past NB repeat row NB - 1 and are never stored) and the weights as B operand: lane (n, g) = (lane % 16,
// lane / 16) holds 32 columns of row n, loaded as 2 x 16 bytes of sign/mantissa and 16 bytes of nibbles per block and
// rebuilt with t12_decode8.  A nibble word with a zero nibble is met rarely: its lane appends the columns to the row's
// list in LDS.  After the stream: the lists are ranked (thread per entry, c compares each), the entry of rank i takes
// esc_vals[esc_row_base[row] + i], and thread (row, batch row) adds the corrections in rank order.
// ESC == false (no tables given): the unpatched product, as the reference computes it without esc_vals.
// ---------------------------------------------------------------------------
constexpr int CB_NW = 8;          // waves per workgroup
constexpr int CB_D = 2;           // blocks in flight per wave
constexpr int CB_CAP = 128;       // escapes per row the LDS lists hold

template <int NB, typename T>
__device__ __forceinline__ T* compat_pick(T* const (&arr)[8], int j)
{
    T* r = arr[0];
#pragma unroll
    for (int i = 1; i < NB; i++)
        if (j >= i) r = arr[i];
    return r;
}

template <int NB, bool ESC>
__global__ __launch_bounds__(CB_NW * 64) void compat_sweep_kernel(const uint8_t* __restrict__ sm,
                                                                  const uint8_t* __restrict__ gr, int base_exp,
                                                                  const BatchPtrs bp, const int32_t* __restrict__ esc_row_base,
                                                                  const int16_t* __restrict__ esc_vals, int M, int K)
{
    __shared__ t12_f32x4 red[CB_NW][64];
    __shared__ uint16_t found[16][CB_CAP];             // columns of the group-0 nibbles met, in arrival order
    __shared__ int nfound[16];
    __shared__ uint16_t s_col[16][CB_CAP];             // the same by rank
    __shared__ float s_delta[16][CB_CAP];
    __shared__ float fix[16][8];
    __shared__ int wave_tot[4];
    __shared__ float red_row[4][NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.x * 16;
    if (ESC) {
        if (tid < 16) nfound[tid] = 0;
        __syncthreads();
    }
    const int nblk = K >> 7;
    const int mine = nblk > wave ? (nblk - wave + CB_NW - 1) / CB_NW : 0;     // blocks of this wave
    const int wblk = mine > 0 ? wave : 0;              // a wave without a block aims its first requests at block 0 and drops them
    const uint32_t be2 = t12_opaque(((uint32_t)base_exp << 7) | ((uint32_t)base_exp << 23));
    const int row = m0 + n;
    const size_t e0 = (size_t)min(row, M - 1) * K;     // rows past the end are clamped, never stored
    const uint8_t* smp = sm + e0 + 32 * g + (size_t)wblk * 128;
    const uint8_t* grp = gr + (e0 >> 1) + 16 * g + (size_t)wblk * 64;
    const uint16_t* xp = compat_pick<NB>(bp.act, n) + 32 * g + (size_t)wblk * 128;

    uint4 rS[CB_D][2], rG[CB_D], rX[CB_D][4];
    auto fetch = [&](int slot, int j) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < 4; q++) rX[slot][q] = *(const uint4*)(xp + (size_t)j * (CB_NW * 128) + 8 * q);
        rS[slot][0] = *(const uint4*)(smp + (size_t)j * (CB_NW * 128));
        rS[slot][1] = *(const uint4*)(smp + (size_t)j * (CB_NW * 128) + 16);
        rG[slot] = *(const uint4*)(grp + (size_t)j * (CB_NW * 64));
    };
    t12_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    auto consume = [&](int slot, int j) __attribute__((always_inline)) {
        const uint32_t gw[4] = {rG[slot].x, rG[slot].y, rG[slot].z, rG[slot].w};
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint4 xa = t12_pair_acts(rX[slot][q]);
            const uint4 sv = rS[slot][q >> 1];
            uint32_t w_[4];
            if (q & 1) t12_decode8(sv.z, sv.w, gw[q], be2, w_);
            else t12_decode8(sv.x, sv.y, gw[q], be2, w_);
            const uint4 wv = make_uint4(w_[0], w_[1], w_[2], w_[3]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(t12_bf16x8, xa),
                                                          __builtin_bit_cast(t12_bf16x8, wv), acc, 0, 0, 0);
        }
        if (ESC) {
            // any zero nibble among the 32?  (v - 0x1111..) & ~v has bit 3 of a nibble set when it is zero, or when it
            // is one and sits above such a nibble: exact as a test for "any"
            uint32_t any = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) any |= (gw[q] - 0x11111111u) & ~gw[q];
            if ((any & 0x88888888u) && row < M) {
                const int cbase = (wblk + j * CB_NW) * 128 + 32 * g;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    uint32_t t = gw[q] | (gw[q] >> 1);
                    t |= t >> 2;
                    uint32_t z = ~t & 0x11111111u;                      // bit 4e: nibble e is zero
                    while (z) {
                        const int e = __builtin_ctz(z) >> 2;
                        z &= z - 1;
                        const int idx = atomicAdd(&nfound[n], 1);
                        if (idx < CB_CAP) found[n][idx] = (uint16_t)(cbase + 8 * q + e);
                    }
                }
            }
        }
    };
#pragma unroll
    for (int d = 0; d < CB_D; d++) {
        fetch(d, min(d, max(mine - 1, 0)));            // (fewer blocks than slots: the last one again, in bounds)
        __builtin_amdgcn_sched_barrier(0);
    }
    int j = 0;
    for (; j + 2 * CB_D <= mine; j += CB_D) {          // every slot is refilled
#pragma unroll
        for (int d = 0; d < CB_D; d++) {
            consume(d, j + d);
            fetch(d, j + d + CB_D);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (; j < mine; j += CB_D) {                      // the last (up to 2 CB_D - 1) blocks
#pragma unroll
        for (int d = 0; d < CB_D; d++) {
            if (j + d < mine) {
                consume(d, j + d);
                if (j + d + CB_D < mine) fetch(d, j + d + CB_D);
            }
        }
    }

    // accumulator register r of lane (n, g) is D[batch 4 g + r][row n]
    red[wave][lane] = acc;
    __syncthreads();
    bool overflow = false;
    if (ESC) {
        int cmax = 0;
#pragma unroll
        for (int r = 0; r < 16; r++) cmax = max(cmax, nfound[r]);
        overflow = cmax > CB_CAP;                       // the same value in every thread
        if (!overflow) {
            {
                const int r = tid >> 5, sub = tid & 31;
                const int c = nfound[r];
                for (int e = sub; e < c; e += 32) {
                    const uint32_t col = found[r][e];
                    const uint32_t key = ((col & 255u) << 16) | col;
                    int rank = 0;
                    for (int f = 0; f < c; f++) {
                        const uint32_t cf = found[r][f];
                        rank += ((((cf & 255u) << 16) | cf) < key) ? 1 : 0;
                    }
                    const uint16_t correct = (uint16_t)esc_vals[esc_row_base[m0 + r] + rank];
                    const uint16_t wrong = t12_decode_scalar(sm[(size_t)(m0 + r) * K + col], 0, base_exp);
                    s_col[r][rank] = (uint16_t)col;
                    s_delta[r][rank] = t12_bf16_to_f32(correct) - t12_bf16_to_f32(wrong);
                }
            }
            __syncthreads();
            if (tid < 128) {
                const int r = tid >> 3, b = tid & 7;
                if (b < NB) {
                    const uint16_t* x = compat_pick<NB>(bp.act, b);
                    const int c = nfound[r];
                    float sum = 0.0f;
                    for (int i = 0; i < c; i++) sum += s_delta[r][i] * t12_bf16_to_f32(x[s_col[r][i]]);
                    fix[r][b] = sum;
                }
            }
            __syncthreads();
        }
    }
    if (!overflow) {
        // thread (r, l) of the first four waves finishes element D[batch 4 (l / 16) + r][row l % 16]
        if (tid < 256) {
            const int r = tid >> 6, l = tid & 63;
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < CB_NW; w++) v += red[w][l][r];
            const int b = 4 * (l >> 4) + r, orow = m0 + (l & 15);
            if (b < NB && orow < M) compat_pick<NB>(bp.out, b)[orow] = ESC ? v + fix[l & 15][b] : v;
        }
    } else {
        // a row of this group has more escapes than the lists hold: the 16 rows one after the other, the reference's way
        for (int r = 0; r < 16; r++)
            compat_row_256<NB>(sm, gr, base_exp, bp, esc_row_base, nullptr, esc_vals, m0 + r, K, tid & 255,
                               tid < 256 && m0 + r < M, wave_tot, red_row);
    }
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
    bool sweep = K % 128 == 0 && K <= 65536 && base_exp >= 0 && base_exp <= 240 && (uintptr_t)sm % 16 == 0 &&
                 (uintptr_t)gr % 16 == 0;
    for (int j = 0; j < NB; j++)
        if ((uintptr_t)a[j] % 16 != 0) sweep = false;
    if (sweep && vals)
        hipLaunchKernelGGL((compat_sweep_kernel<NB, true>), dim3((M + 15) / 16), dim3(CB_NW * 64), 0, (hipStream_t)stream,
                           (const uint8_t*)sm, (const uint8_t*)gr, base_exp, bp, (const int32_t*)rb, (const int16_t*)vals, M, K);
    else if (sweep)
        hipLaunchKernelGGL((compat_sweep_kernel<NB, false>), dim3((M + 15) / 16), dim3(CB_NW * 64), 0, (hipStream_t)stream,
                           (const uint8_t*)sm, (const uint8_t*)gr, base_exp, bp, nullptr, nullptr, M, K);
    else
        hipLaunchKernelGGL(compat_batch_kernel<NB>, dim3(M), dim3(256), 0, (hipStream_t)stream, (const uint8_t*)sm,
                           (const uint8_t*)gr, base_exp, bp, (const int32_t*)rb, (const uint8_t*)cnt,
                           (const int16_t*)vals, M, K);
    T12_CHECK_LAUNCH("launch_split12_batch");
    return T12_OK;
}


// nv_apply_patches_batch (nvidia_kernels.cu:295-319): one thread per (listed row, batch row) pair walks the row's
// escape slice: out[b, row] += sum over entries of (correct - wrong) * x[b, col]; nothing is written when the sum is 0.
// Neighbouring threads take neighbouring listed rows of ONE batch row: the read-modify-write of out[b, row] then covers
// whole cache lines (with neighbouring batch rows per wave every lane touched a line of its own: 24 -> 15 us per launch
// over the tensors of two Llama-width layers and the head at 64 rows).
__global__ __launch_bounds__(256) void patches_batch_kernel(const int32_t* __restrict__ row_off, const int32_t* __restrict__ cols,
                                                            const int16_t* __restrict__ correct, const int16_t* __restrict__ wrong,
                                                            const int32_t* __restrict__ rows, const uint16_t* __restrict__ act,
                                                            int act_stride, float* __restrict__ out, int out_stride, int n_rows,
                                                            int B)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int b = (int)(idx / n_rows), ri = (int)(idx % n_rows);
    if (b >= B) return;
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
