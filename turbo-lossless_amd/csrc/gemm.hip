// Split-12 fused decode + GEMM on CDNA4 matrix cores (gfx950).
//
//   out_s[b*out_stride + m] = sum_k dec(W_s[m,k]) * X[b*act_stride + k]
//
// the function of the reference's split12_fused_gemm V1/V2/V3
// (split12_gemm.cuh:99-288, split12_gemm_v2.cuh:86-240, split12_gemm_v3.cuh:111-253)
// plus nv_apply_patches_batch (nvidia_kernels.cu:295-319), re-designed for
// wave64 MFMA instead of warp-level mma.sync:
//
//   * v_mfma_f32_32x32x16_bf16, activations as the A operand (rows = batch),
//     weights as the B operand (columns = output features), so that an
//     accumulator register holds 32 consecutive m of one batch row and the
//     stores to out[b, m] coalesce without a transpose through LDS.
//   * The whole batch tile (up to 256 rows) lives in one workgroup: every
//     weight byte is fetched once per launch (the reference re-decodes per
//     batch tile, nvidia_kernels.cu:456).
//   * The compressed planes are staged global -> LDS as they are (1.5 B per
//     weight) and rebuilt to bf16 in registers, two weights per VGPR
//     (t12_decode8), straight into the MFMA B operand: no bf16 copy of W ever
//     exists in LDS or HBM.  The activations are staged already paired the way
//     t12_decode8 orders its outputs, so no operand shuffling is needed.
//   * Waves are laid out WB x WM; a wave owns FB x FM 32x32 accumulator tiles.
//     B <= 128 uses 1 x 4 waves (each weight decoded once per workgroup);
//     B <= 256 uses 2 x 2 waves with 4 x 2 tiles (128 accumulator VGPRs).
//   * Few row tiles (small M) are split along K across workgroups; the partial
//     sums go to a workspace and a second kernel adds them in a fixed order
//     (deterministic) together with the escape corrections.
//   * Escapes are EXACT and cost no extra pass: the (column, exact bf16) pairs of
//     the workgroup's 128 rows -- one contiguous slice of the CSR list -- are
//     staged in LDS once; every lane walks its own row's slice in step with the
//     K loop and overwrites the decoded half-word in its MFMA operand register.
//
// Fast path requirements: K % 64 == 0, 0 <= base_exp <= 240, 16-byte aligned
// activation rows.  Everything else goes to the general kernel below.

#include "t12_device.h"
#include "t12_host.h"

namespace {

constexpr int KC = 64;          // K columns staged per pipeline stage
constexpr int TM = 128;         // weight rows per workgroup
constexpr int PCAP = 2048;      // escape entries a workgroup can stage in LDS
constexpr int PATCH_BYTES = PCAP * 4 + (TM + 1) * 4 + 12;
constexpr int NO_ESCAPE = 0x7FFFFFFF;

struct GemmParams {
    T12Segment seg[T12_MAX_SEGMENTS];
    int blk_start[T12_MAX_SEGMENTS + 1];   // first row-tile of each segment
    int seg_row0[T12_MAX_SEGMENTS];        // first row of each segment in the workspace
    int nseg;
    int K, B;
    int act_stride;
    int ksplit;                            // workgroups along K
    int kslice;                            // columns per K split (multiple of KC)
    int m_total;                           // sum of M over segments (workspace row length)
    const uint16_t* act;
    float* ws;                             // [ksplit][B][m_total] partial sums when ksplit > 1
};

// LDS slot of (unit, row) in a [units][rows] array of 16-byte units.  Rows are rotated
// inside their aligned block of eight by the unit index, so that both access patterns are
// bank-conflict free: the staging writes (neighbouring lanes = the units of one row) and
// the fragment reads (neighbouring lanes = consecutive rows of one unit).
__device__ __forceinline__ int lds_slot(int u, int r, int rows) { return u * rows + (r & ~7) + ((r + u) & 7); }

__device__ __forceinline__ int find_segment(const GemmParams& p, int tile)
{
    int s = 0;
#pragma unroll
    for (int i = 1; i < T12_MAX_SEGMENTS; i++)
        if (i < p.nseg && tile >= p.blk_start[i]) s = i;
    return s;
}

// ---------------------------------------------------------------------------
// LDS stage layout (one of two buffers), unit u = (k % 64) / 8 = eight bf16 of one row,
// paired (i, i + 4) per dword the way t12_decode8 / t12_pair_acts order them:
//   act  [8 units][TB rows] x 16 B
//   w    [8 units][TM rows] x 16 B     decoded weights
// MFMA k-step t of a stage covers columns 16t .. 16t+15; the lanes of wave half h take
// unit 2t + h of their row, for both operands.
// ---------------------------------------------------------------------------
// DBG (benchmark probes, 0 in production): bit 0 skips the MFMAs, bit 1 skips the global->LDS
// staging inside the loop, bit 3 skips the escapes.
template <int WB, int WM, int FB, int FM, int DBG>
__device__ __forceinline__ void gemm_mfma_body(const GemmParams& p)
{
    constexpr int TB = WB * FB * 32;                  // batch rows per workgroup
    static_assert(WB * WM == 4, "four waves per workgroup");
    static_assert(WM * FM * 32 == TM, "row tile is 128");
    constexpr int ACT_UNITS = TB * 8;                 // 16-byte units per stage
    constexpr int ACT_LD = ACT_UNITS / 256;           // per thread
    constexpr int STAGE_BYTES = ACT_UNITS * 16 + TM * 128;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wb = wave / WM, wm = wave % WM;
    const int ln = lane & 31, lh = lane >> 5;

    const int tile = blockIdx.x;
    const int s = find_segment(p, tile);
    const T12Segment& sg = p.seg[s];
    const int M = sg.M, K = p.K, B = p.B;
    const int m0 = (tile - p.blk_start[s]) * TM;
    const int b0 = blockIdx.y * TB;
    const int k_begin = blockIdx.z * p.kslice;
    const int k_end = min(K, k_begin + p.kslice);
    const int nstage = (k_end - k_begin) / KC;
    const uint32_t be2 = t12_opaque(((uint32_t)sg.base_exp << 7) | ((uint32_t)sg.base_exp << 23));

    // ---- this thread's share of the global -> LDS staging
    //  acts:   item idx = tid + 256*i -> batch row idx / 8, unit idx % 8 (8 lanes = 128 contiguous bytes)
    //  planes: item idx = tid + 256*i (i < 2) -> weight row idx / 4, 16 columns c = idx % 4
    //          (16 sm bytes + 8 gr bytes -> two decoded units 2c, 2c + 1)
    // rows past the end are clamped: their products are computed and never stored
    const uint16_t* a_src[ACT_LD];
    int a_dst[ACT_LD];
#pragma unroll
    for (int i = 0; i < ACT_LD; i++) {
        const int idx = tid + 256 * i;
        const int r = idx >> 3, u = idx & 7;
        a_src[i] = p.act + (size_t)min(b0 + r, B - 1) * p.act_stride + k_begin + u * 8;
        a_dst[i] = lds_slot(u, r, TB) * 16;
    }
    const int wc = tid & 3;                       // the same 16-column group for both items
    const uint8_t* s_src[2];
    const uint8_t* g_src[2];
    int w_dst[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int r = (tid + 256 * i) >> 2;
        const size_t e = (size_t)min(m0 + r, M - 1) * K + k_begin;
        s_src[i] = sg.sm + e + wc * 16;
        g_src[i] = sg.gr + (e >> 1) + wc * 8;
        w_dst[i][0] = ACT_UNITS * 16 + lds_slot(2 * wc, r, TM) * 16;
        w_dst[i][1] = ACT_UNITS * 16 + lds_slot(2 * wc + 1, r, TM) * 16;
    }

    // Register ring: the global loads of stage st + D are issued while stage st is
    // being multiplied (HBM latency is longer than one stage of MFMAs); a stage is decoded
    // and moved registers -> LDS one iteration before it is consumed (double-buffered LDS).
    constexpr int D = 3;
    uint4 ra[D][ACT_LD];
    uint4 rs[D][2];
    uint2 rg[D][2];
#define T12_LOAD_STAGE(slot, st)                                                        \
    {                                                                                   \
        _Pragma("unroll") for (int i = 0; i < ACT_LD; i++)                              \
            ra[slot][i] = *(const uint4*)(a_src[i] + (size_t)(st) * KC);                \
        _Pragma("unroll") for (int i = 0; i < 2; i++) {                                 \
            rs[slot][i] = t12_ldg_stream16(s_src[i] + (size_t)(st) * KC);               \
            rg[slot][i] = t12_ldg_stream8(g_src[i] + (size_t)(st) * (KC / 2));          \
        }                                                                               \
    }
#define T12_STORE_STAGE(slot, buf)                                                                  \
    {                                                                                               \
        uint8_t* base_ = lds + (buf) * STAGE_BYTES;                                                 \
        _Pragma("unroll") for (int i = 0; i < ACT_LD; i++)                                          \
            *(uint4*)(base_ + a_dst[i]) = t12_pair_acts(ra[slot][i]);                               \
        _Pragma("unroll") for (int i = 0; i < 2; i++) {                                             \
            uint32_t w_[2][4];                                                                      \
            t12_decode8(rs[slot][i].x, rs[slot][i].y, rg[slot][i].x, be2, w_[0]);                   \
            t12_decode8(rs[slot][i].z, rs[slot][i].w, rg[slot][i].y, be2, w_[1]);                   \
            *(uint4*)(base_ + w_dst[i][0]) = make_uint4(w_[0][0], w_[0][1], w_[0][2], w_[0][3]);    \
            *(uint4*)(base_ + w_dst[i][1]) = make_uint4(w_[1][0], w_[1][1], w_[1][2], w_[1][3]);    \
        }                                                                                           \
    }

    t12_f32x16 acc[FB][FM];
#pragma unroll
    for (int i = 0; i < FB; i++)
#pragma unroll
        for (int j = 0; j < FM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // ---- escape list of this workgroup's rows -> LDS.  The rows are consecutive, so
    //      their entries are one contiguous slice [e0, e1) of cols[] / correct[].
    //      esc_mode: 0 none, 1 staged (exact values written over the decoded ones in LDS),
    //      2 too many for LDS (or K > 65536): wrong values multiplied, corrected in the epilogue.
    uint32_t* lpat = (uint32_t*)(lds + 2 * STAGE_BYTES);       // col | correct << 16
    int* lrow = (int*)(lpat + PCAP);                           // [TM + 1] offsets into lpat
    int esc_mode = 0;
    if (sg.row_off && !(DBG & 8)) {
        const int e0 = sg.row_off[min(m0, M)], e1 = sg.row_off[min(m0 + TM, M)];
        esc_mode = (e1 - e0 <= PCAP && K <= 65536) ? 1 : 2;
        if (esc_mode == 1) {
            for (int t = tid; t < e1 - e0; t += 256)
                lpat[t] = (uint32_t)sg.cols[e0 + t] | ((uint32_t)(uint16_t)sg.correct[e0 + t] << 16);
            for (int t = tid; t <= TM; t += 256) lrow[t] = sg.row_off[min(m0 + t, M)] - e0;
        }
    }
    // Per staging item: cursor into its row's slice and the column of the next entry.  The
    // thread that decoded 16 columns of a row into LDS also overwrites the escapes among them
    // there (same wave, LDS executes its writes in order: no barrier needed in between).
    int pp[2] = {0, 0}, pe[2] = {0, 0}, nc[2] = {NO_ESCAPE, NO_ESCAPE};
#define T12_PATCH_STAGE(buf, kabs)                                                                  \
    if (esc_mode == 1) {                                                                            \
        uint8_t* base_ = lds + (buf) * STAGE_BYTES + ACT_UNITS * 16;                                \
        _Pragma("unroll") for (int i = 0; i < 2; i++) {                                             \
            while (nc[i] < (kabs) + KC) {                                                           \
                const int e_ = nc[i] - (kabs) - 16 * wc;            /* 0..15: one of this item's */ \
                if ((unsigned)e_ < 16u) {                                                           \
                    const int r_ = (tid + 256 * i) >> 2;                                            \
                    const int off_ = lds_slot(2 * wc + (e_ >> 3), r_, TM) * 16 + (e_ & 3) * 4 + ((e_ >> 2) & 1) * 2; \
                    *(uint16_t*)(base_ + off_) = (uint16_t)(lpat[pp[i]] >> 16);                     \
                }                                                                                   \
                pp[i]++;                                                                            \
                nc[i] = pp[i] < pe[i] ? (int)(lpat[pp[i]] & 0xFFFFu) : NO_ESCAPE;                   \
            }                                                                                       \
        }                                                                                           \
    }

    auto load_frags = [&](const uint4* lact, const uint4* lw, int t, uint4 (&A)[FB], uint4 (&W)[FM]) {
#pragma unroll
        for (int i = 0; i < FB; i++) A[i] = lact[lds_slot(2 * t + lh, (wb * FB + i) * 32 + ln, TB)];
#pragma unroll
        for (int j = 0; j < FM; j++) W[j] = lw[lds_slot(2 * t + lh, (wm * FM + j) * 32 + ln, TM)];
    };
    auto mma = [&](const uint4 (&A)[FB], const uint4 (&W)[FM]) {
#pragma unroll
        for (int i = 0; i < FB; i++) {
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if (DBG & 1) acc[i][j][0] += __builtin_bit_cast(float, A[i].x ^ W[j].x ^ W[j].y ^ W[j].z ^ W[j].w);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(t12_bf16x8, A[i]),
                                                                        __builtin_bit_cast(t12_bf16x8, W[j]),
                                                                        acc[i][j], 0, 0, 0);
            }
        }
    };
    // one stage = 64 columns = 4 MFMA k-steps; fragment loads run one k-step ahead
    auto compute_stage = [&](int buf) {
        const uint8_t* base = lds + buf * STAGE_BYTES;
        const uint4* lact = (const uint4*)base;
        const uint4* lw = (const uint4*)(base + ACT_UNITS * 16);
        uint4 A0[FB], A1[FB], W0[FM], W1[FM];
        load_frags(lact, lw, 0, A0, W0);
        load_frags(lact, lw, 1, A1, W1);
        mma(A0, W0);
        load_frags(lact, lw, 2, A0, W0);
        mma(A1, W1);
        load_frags(lact, lw, 3, A1, W1);
        mma(A0, W0);
        mma(A1, W1);
    };

    // prologue: stages 0..D-1 in flight, escape list visible, stage 0 into LDS
#pragma unroll
    for (int d = 0; d < D; d++)
        if (d < nstage) T12_LOAD_STAGE(d, d)
    __syncthreads();
    if (esc_mode == 1) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int r = (tid + 256 * i) >> 2;
            pp[i] = lrow[r];
            pe[i] = lrow[r + 1];
            while (pp[i] < pe[i] && (int)(lpat[pp[i]] & 0xFFFFu) < k_begin) pp[i]++;   // K split: skip earlier columns
            if (pp[i] < pe[i]) nc[i] = (int)(lpat[pp[i]] & 0xFFFFu);
        }
    }
    if (nstage > 0) {
        T12_STORE_STAGE(0, 0)
        T12_PATCH_STAGE(0, k_begin)
    }
    __syncthreads();

    int st = 0;
    // steady state, unrolled by D so that ring slots are compile-time; no guards inside
    for (; st + 2 * D <= nstage; st += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (!(DBG & 2)) T12_LOAD_STAGE(d, st + d + D)    // slot d held stage st + d: already in LDS
            compute_stage((st + d) & 1);
            if (!(DBG & 2)) T12_STORE_STAGE((d + 1) % D, (st + d + 1) & 1)
            T12_PATCH_STAGE((st + d + 1) & 1, k_begin + (st + d + 1) * KC)
            __syncthreads();
        }
    }
    // drain
    for (; st < nstage; st += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (st + d < nstage) {
                if (st + d + D < nstage) T12_LOAD_STAGE(d, st + d + D)
                compute_stage((st + d) & 1);
                if (st + d + 1 < nstage) {
                    T12_STORE_STAGE((d + 1) % D, (st + d + 1) & 1)
                    T12_PATCH_STAGE((st + d + 1) & 1, k_begin + (st + d + 1) * KC)
                }
                __syncthreads();
            }
        }
    }
#undef T12_LOAD_STAGE
#undef T12_STORE_STAGE
#undef T12_PATCH_STAGE

    // ---- overflow path only (more escapes than the LDS list holds): the streamed value of an
    //      escape was its "wrong" decode, so acc[b, m] += (correct - wrong) * X[b, col], added by
    //      the K split that owns column 0
    if (blockIdx.z == 0 && esc_mode == 2) {
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int m = m0 + (wm * FM + j) * 32 + ln;
            if (m < M) {
                const int beg = sg.row_off[m], end = sg.row_off[m + 1];
                for (int pp = beg; pp < end; pp++) {
                    const float delta = t12_bf16_to_f32((uint16_t)sg.correct[pp]) -
                                        t12_bf16_to_f32((uint16_t)sg.wrong[pp]);
                    const uint16_t* xc = p.act + sg.cols[pp];
#pragma unroll
                    for (int i = 0; i < FB; i++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int bb = b0 + (wb * FB + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                            if (bb < B) acc[i][j][r] += delta * t12_bf16_to_f32(xc[(size_t)bb * p.act_stride]);
                        }
                }
            }
        }
    }

    // ---- store: accumulator register r of lane (ln, lh) is
    //      D[row = 8*(r/4) + 4*lh + r%4][col = ln]   (row = batch, col = m)
    float* dst;
    size_t ld;
    int col_off;
    if (p.ksplit > 1) {
        dst = p.ws + (size_t)blockIdx.z * B * p.m_total;
        ld = p.m_total;
        col_off = p.seg_row0[s];
    } else {
        dst = sg.out;
        ld = sg.out_stride;
        col_off = 0;
    }
#pragma unroll
    for (int i = 0; i < FB; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int m = m0 + (wm * FM + j) * 32 + ln;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int b = b0 + (wb * FB + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (m < M && b < B) dst[(size_t)b * ld + col_off + m] = acc[i][j][r];
            }
        }
}

// One workgroup per CU (batch tile 256: 128 accumulator registers + the load ring) ...
template <int WB, int WM, int FB, int FM, int DBG = 0>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const GemmParams p)
{
    gemm_mfma_body<WB, WM, FB, FM, DBG>(p);
}
// ... or two (batch tiles <= 128): at most 256 registers per lane, so that two waves share a SIMD
// and one wave's decode / LDS traffic runs under the other's MFMAs.
template <int WB, int WM, int FB, int FM, int DBG = 0>
__global__ __launch_bounds__(256, 2) void gemm_mfma_kernel_occ2(const GemmParams p)
{
    gemm_mfma_body<WB, WM, FB, FM, DBG>(p);
}

// ---------------------------------------------------------------------------
// K-split reduction: out[b, m] = sum over splits z of ws[z][b][m], in ascending z
// (a fixed order: the result does not depend on which workgroup finished first).
// Grid: (blocks of 256 workspace columns, B).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmParams p)
{
    const int col = blockIdx.x * 256 + threadIdx.x;
    const int b = blockIdx.y;
    if (col >= p.m_total) return;
    int s = 0;
#pragma unroll
    for (int i = 1; i < T12_MAX_SEGMENTS; i++)
        if (i < p.nseg && col >= p.seg_row0[i]) s = i;
    float v = 0.0f;
    for (int z = 0; z < p.ksplit; z++) v += p.ws[((size_t)z * p.B + b) * p.m_total + col];
    const T12Segment& sg = p.seg[s];
    sg.out[(size_t)b * sg.out_stride + (col - p.seg_row0[s])] = v;
}

// ---------------------------------------------------------------------------
// General path: any K, any base_exp, any alignment.  One wave per (row, 8
// batch rows); scalar decode rule; escapes exact from the CSR list.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_general_kernel(const GemmParams p)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tile = blockIdx.x;            // blk_start counts 4-row blocks
    const int s = find_segment(p, tile);
    const T12Segment& sg = p.seg[s];
    const int row = (tile - p.blk_start[s]) * 4 + wave;
    if (row >= sg.M) return;
    const int b0 = blockIdx.y * 8;
    const int nb = min(8, p.B - b0);
    const int K = p.K;
    const size_t base = (size_t)row * K;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int k = lane; k < K; k += T12_WAVE) {
        const size_t i = base + k;
        const uint32_t g = (sg.gr[i >> 1] >> (4 * (i & 1))) & 0xFu;
        if (g == 0 && sg.row_off) continue;            // taken from the list below
        const float w = t12_bf16_to_f32(t12_decode_scalar(sg.sm[i], g, sg.base_exp));
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (j < nb) acc[j] += w * t12_bf16_to_f32(p.act[(size_t)(b0 + j) * p.act_stride + k]);
    }
    if (sg.row_off) {
        const int beg = sg.row_off[row], end = sg.row_off[row + 1];
        for (int q = beg + lane; q < end; q += T12_WAVE) {
            const float w = t12_bf16_to_f32((uint16_t)sg.correct[q]);
            const int k = sg.cols[q];
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (j < nb) acc[j] += w * t12_bf16_to_f32(p.act[(size_t)(b0 + j) * p.act_stride + k]);
        }
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float v = t12_wave_sum(acc[j]);
        if (lane == 0 && j < nb) sg.out[(size_t)(b0 + j) * sg.out_stride + row] = v;
    }
}

// ---- workspace for the K-split partial sums (grown on demand, per device) ----
float* g_ws[16] = {};
size_t g_ws_bytes[16] = {};

float* workspace(size_t bytes)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    if (g_ws_bytes[dev] < bytes) {
        if (g_ws[dev]) (void)hipFree(g_ws[dev]);
        g_ws[dev] = nullptr;
        g_ws_bytes[dev] = 0;
        if (hipMalloc((void**)&g_ws[dev], bytes) != hipSuccess) return nullptr;
        g_ws_bytes[dev] = bytes;
    }
    return g_ws[dev];
}

int g_gemm_ksplit = 0;   // 0 = choose by shape

int g_gemm_dbg = 0;

template <int WB, int WM, int FB, int FM, int DBG = 0, bool OCC2 = false>
int launch_mfma(GemmParams& p, int tiles, hipStream_t st)
{
    constexpr int TB = WB * FB * 32;
    constexpr int STAGE_BYTES = TB * 8 * 16 + TM * 128;
    const dim3 grid(tiles, (p.B + TB - 1) / TB, p.ksplit);   // batch tiles of one row tile are neighbours in time
    auto kfn = OCC2 ? gemm_mfma_kernel_occ2<WB, WM, FB, FM, DBG> : gemm_mfma_kernel<WB, WM, FB, FM, DBG>;
    static bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                2 * STAGE_BYTES + PATCH_BYTES) !=
            hipSuccess) {
            t12_set_error("t12_gemm: cannot reserve %d bytes of LDS", 2 * STAGE_BYTES);
            return T12_ELAUNCH;
        }
        attr_set = true;
    }
    hipLaunchKernelGGL(kfn, grid, dim3(256), 2 * STAGE_BYTES + PATCH_BYTES, st, p);
    T12_CHECK_LAUNCH("t12_gemm");
    return T12_OK;
}

}  // namespace

extern "C" {

// Pins the number of K splits of the MFMA path (benchmark sweeps); 0 = by shape.
int t12_tune_gemm(int ksplit)
{
    g_gemm_ksplit = ksplit;
    return T12_OK;
}

// Benchmark probe: runs the B > 128 kernel with parts of its loop removed (wrong results).
int t12_debug_gemm(int mask)
{
    g_gemm_dbg = mask;
    return T12_OK;
}

int t12_gemm(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K, int B,
             void* stream)
{
    T12_REQUIRE(segs && nseg >= 1 && nseg <= T12_MAX_SEGMENTS, "t12_gemm: nseg must be 1..%d (got %d)",
                T12_MAX_SEGMENTS, nseg);
    T12_REQUIRE(act_bf16 && K >= 1 && B >= 1, "t12_gemm: activations null or K/B < 1 (K=%d B=%d)", K, B);
    T12_REQUIRE(act_stride >= K, "t12_gemm: act_stride %d < K %d", act_stride, K);
    hipStream_t st = (hipStream_t)stream;
    GemmParams p;
    p.nseg = nseg;
    p.K = K;
    p.B = B;
    p.act_stride = act_stride;
    p.act = (const uint16_t*)act_bf16;
    p.ws = nullptr;
    bool fast = (K % KC == 0) && (act_stride % 8 == 0) && ((uintptr_t)act_bf16 % 16 == 0);
    int m_total = 0;
    for (int i = 0; i < nseg; i++) {
        const T12Segment& g = segs[i];
        T12_REQUIRE(g.M >= 1 && g.sm && g.gr && g.out, "t12_gemm: segment %d has M < 1 or a null pointer", i);
        T12_REQUIRE(!g.row_off || (g.cols && g.correct && g.wrong), "t12_gemm: segment %d: row_off without lists", i);
        T12_REQUIRE(g.base_exp >= -1 && g.base_exp <= 254, "t12_gemm: segment %d: base_exp %d out of range", i,
                    g.base_exp);
        if (g.base_exp < 0 || g.base_exp > 240) fast = false;
        p.seg[i] = g;
        if (p.seg[i].out_stride == 0) p.seg[i].out_stride = out_stride;
        T12_REQUIRE(p.seg[i].out_stride >= g.M, "t12_gemm: out_stride %d < M %d of segment %d", p.seg[i].out_stride,
                    g.M, i);
        p.seg_row0[i] = m_total;
        m_total += g.M;
    }
    p.m_total = m_total;

    if (!fast) {
        int tiles = 0;
        for (int i = 0; i < nseg; i++) {
            p.blk_start[i] = tiles;
            tiles += (segs[i].M + 3) / 4;
        }
        p.blk_start[nseg] = tiles;
        p.ksplit = 1;
        p.kslice = K;
        hipLaunchKernelGGL(gemm_general_kernel, dim3(tiles, (B + 7) / 8), dim3(256), 0, st, p);
        T12_CHECK_LAUNCH("t12_gemm(general)");
        return T12_OK;
    }

    int tiles = 0;
    for (int i = 0; i < nseg; i++) {
        p.blk_start[i] = tiles;
        tiles += (segs[i].M + TM - 1) / TM;
    }
    p.blk_start[nseg] = tiles;
    // K split: fill the chip.  A 256-row batch tile needs a whole CU (LDS, accumulators);
    // smaller batch tiles fit 2-4 workgroups per CU.  Every split keeps >= 4 stages.
    const bool big = B > 128 && !(g_gemm_dbg & 64);
    const int btiles = big ? (B + 255) / 256 : (B + 127) / 128;
    const int per_cu = big ? 1 : (B > 64 ? 2 : 4);
    const int want = 256 * per_cu;
    int ks = 1;
    if (g_gemm_ksplit > 0) ks = g_gemm_ksplit;
    else
        while (tiles * btiles * ks * 4 < want * 3 && K / (ks * 2) >= 4 * KC && ks < 16) ks *= 2;
    int kslice = ((K / KC + ks - 1) / ks) * KC;
    ks = (K + kslice - 1) / kslice;
    p.ksplit = ks;
    p.kslice = kslice;
    if (ks > 1) {
        p.ws = workspace((size_t)ks * B * m_total * sizeof(float));
        if (!p.ws) {
            t12_set_error("t12_gemm: cannot allocate %zu bytes of K-split workspace",
                          (size_t)ks * B * m_total * sizeof(float));
            return T12_ELAUNCH;
        }
    }
    int rc;
    if (B <= 32) rc = launch_mfma<1, 4, 1, 1, 0, true>(p, tiles, st);
    else if (B <= 64) rc = launch_mfma<1, 4, 2, 1, 0, true>(p, tiles, st);
    else if (B <= 128 || (g_gemm_dbg & 64)) {
        if ((g_gemm_dbg & 63) == 0) rc = launch_mfma<1, 4, 4, 1, 0, true>(p, tiles, st);
        else if ((g_gemm_dbg & 63) == 1) rc = launch_mfma<1, 4, 4, 1, 1, true>(p, tiles, st);
        else if ((g_gemm_dbg & 63) == 2) rc = launch_mfma<1, 4, 4, 1, 2, true>(p, tiles, st);
        else if ((g_gemm_dbg & 63) == 8) rc = launch_mfma<1, 4, 4, 1, 8, true>(p, tiles, st);
        else if ((g_gemm_dbg & 63) == 16) rc = launch_mfma<1, 4, 4, 1, 0, false>(p, tiles, st);
        else rc = launch_mfma<1, 4, 4, 1, 10, true>(p, tiles, st);
    }
    else if (g_gemm_dbg == 1) rc = launch_mfma<2, 2, 4, 2, 1>(p, tiles, st);
    else if (g_gemm_dbg == 2) rc = launch_mfma<2, 2, 4, 2, 2>(p, tiles, st);
    else if (g_gemm_dbg == 8) rc = launch_mfma<2, 2, 4, 2, 8>(p, tiles, st);
    else if (g_gemm_dbg == 10) rc = launch_mfma<2, 2, 4, 2, 10>(p, tiles, st);
    else rc = launch_mfma<2, 2, 4, 2>(p, tiles, st);
    if (rc) return rc;

    if (ks > 1) {
        hipLaunchKernelGGL(gemm_reduce_kernel, dim3((m_total + 255) / 256, B), dim3(256), 0, st, p);
        T12_CHECK_LAUNCH("t12_gemm(reduce)");
    }
    return T12_OK;
}

}  // extern "C"
