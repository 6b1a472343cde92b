// Split-12 fused decode-GEMV for one activation vector (B = 1), gfx950.
//
// Computes, for every segment s of a fused launch,
//     out_s[m] = sum_k dec(W_s[m,k]) * x[k]
// the function of the reference's split12_matvec_v2 / _multirow / _dual
// (decompress_v2.hip:148-227, 234-380, 387-523) followed by apply_patches_v2
// (:78-99), in ONE launch and with a different mapping:
//   * a lane streams 16 consecutive weights per step with one 128-bit load of
//     the sign/mantissa plane and one 64-bit load of the nibble plane (a wave
//     covers 1024 consecutive K of a row), instead of byte loads;
//   * two weights are rebuilt per 32-bit register (t12_decode8) and multiplied
//     with v_dot2_f32_bf16 against activations that were paired to match when
//     they were staged into LDS, once per workgroup;
//   * escapes: the streamed value of a group-0 weight is the "wrong" value; the
//     wave that owns the row adds (correct - wrong) * x[col] from the CSR list
//     before its reduction (wave-level patch, no second launch).
// Bandwidth bound: 1.5 B per weight from HBM, everything else is L2/LDS.

#include "t12_device.h"
#include "t12_host.h"

namespace {

constexpr int GEMV_SEGS = 16;              // a mixture-of-experts launch carries (gate, up) of up to eight experts

struct GemvParams {
    T12Segment seg[GEMV_SEGS];
    int blk_start[T12_MAX_SEGMENTS + 1];   // first workgroup of each segment
    int nseg;
    int K;
    const uint16_t* act;
    uint16_t* out_bf16;                    // SwiGLU mode only
    const float* add;                      // out[m] = add[m] + sum (single segment), or null
    // RMSNorm prologue (NORM > 0): activations = bf16(rmsnorm(nx [+ nres]) * nw)
    const float* nx;
    const float* nres;
    const float* nw;
    float* hidden_out;                     // nx + nres, written by workgroup 0 (may be null)
    float eps;
    // MOE launches (gridDim.y activation rows, each with the expert the routing gave it):
    const int* slot_expert;                // [gridDim.y] on the device; a negative entry = no row, the workgroup leaves
    int act_stride;                        // bf16 elements between activation rows
    int out_ld;                            // elements between output rows (fp32 outputs and out_bf16)
};

__device__ __forceinline__ int find_segment(const GemvParams& p, int blk)
{
    int s = 0;
#pragma unroll
    for (int i = 1; i < T12_MAX_SEGMENTS; i++)
        if (i < p.nseg && blk >= p.blk_start[i]) s = i;
    return s;
}

// This lane's share of the row's escape corrections.
// DELTA: the streamed sum already holds wrong * x for every escape, so the
// correction is (correct - wrong) * x (wrong is finite whenever base_exp >= 0).
// !DELTA: the streamed sum skipped the escapes, the correction is correct * x.
template <bool DELTA>
__device__ __forceinline__ float patch_partial(const T12Segment& sg, int row, int lane,
                                               const uint16_t* __restrict__ act)
{
    float c = 0.0f;
    if (sg.row_off) {
        const int beg = sg.row_off[row], end = sg.row_off[row + 1];
        for (int q = beg + lane; q < end; q += T12_WAVE) {
            float w = t12_bf16_to_f32((uint16_t)sg.correct[q]);
            if (DELTA) w -= t12_bf16_to_f32((uint16_t)sg.wrong[q]);
            c += w * t12_bf16_to_f32(act[sg.cols[q]]);
        }
    }
    return c;
}

// ---------------------------------------------------------------------------
// Fast path: K % 16 == 0, 0 <= base_exp <= 240.
// Workgroup = NW waves; a wave owns R consecutive rows and walks their full K
// in 1024-column tiles, software pipelined D tiles deep through a register
// ring: every lane keeps D*R 128-bit + D*R 64-bit loads in flight.
// Order inside a wave, arranged so that no dependent load chain is exposed:
//   (0) the activations (bf16 input: up to SU 16-byte pieces per thread),
//   (1) CSR row pointers of the R rows (one vector load, lanes 0..R),
//   (2) the first D tiles of weight loads,
//   (3) the workgroup stages the activations into LDS, barrier,
//   (4) the rows' first 64 escape entries each (cols / correct / wrong) are
//       requested; they arrive while
//   (5) the tile stream is consumed and refilled,
//   (6) escape corrections: (correct - wrong) * x[col], x read back from LDS,
//   (7) DPP wave reduction, lane 63 stores.
// LDS: activations, paired (t12_pair_acts), laid out per 1024-column chunk as
// [half j = 0,1][lane 0..63] x 16 B so that both ds_read_b128 of a lane are
// conflict free.  Columns >= K are stored as zeros.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float lds_act_at(const uint4* lds_act, int k)
{
    // inverse of the staging layout: column k -> its bf16 inside the paired tiles
    const int q = k >> 3, i = k & 7;
    const int slot = (q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1);
    const uint16_t* h = (const uint16_t*)(lds_act + slot);
    return t12_bf16_to_f32(h[(i & 3) * 2 + (i >> 2)]);
}

// SWIGLU (R must be 2): row 0 of a wave is row m of segment 0 (gate), row 1 is row m of
// segment 1 (up); the wave writes bf16( silu(gate.x) * (up.x) ) to p.out_bf16[m] instead of two
// fp32 sums -- the reference's split12_matvec_v2_dual (decompress_v2.hip:387-523) with its
// silu_mul_bf16 kernel (engine/kernels.hip:447-459) folded into the epilogue.
// NORM (1: RMSNorm, 2: residual add + RMSNorm): instead of reading bf16 activations, every
// workgroup rebuilds them from the fp32 residual stream while its first weight tiles are in
// flight -- the reference's (add_)rms_norm_bf16_batch kernels (engine/kernels.hip:355-442) as a
// prologue.  K <= 16 * NW * 64.  Workgroup 0 also stores nx + nres for the residual path.
// MOE: one activation row per blockIdx.y, multiplied with the tensors of the expert slot_expert[blockIdx.y] names --
// segment e (SWIGLU: segments 2e and 2e + 1); rows of activations and outputs are act_stride / out_ld apart.
template <int NW, int R, int D, int MINB, bool SWIGLU = false, int NORM = 0, bool MOE = false>
__global__ __launch_bounds__(NW * 64, MINB) void gemv_stream_kernel(const GemvParams p)
{
    static_assert(!SWIGLU || R == 2, "the SwiGLU epilogue pairs exactly two rows");
    static_assert(!MOE || NORM == 0, "expert launches take bf16 activations");
    int expert = 0;
    if (MOE) {
        expert = __builtin_amdgcn_readfirstlane(p.slot_expert[blockIdx.y]);
        if (expert < 0) return;                // (the whole workgroup: no barrier has been reached)
    }
    const uint16_t* const act_row = MOE ? p.act + (size_t)blockIdx.y * p.act_stride : p.act;
    extern __shared__ uint4 lds_act[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = p.K;
    const int T = K >> 10;                     // whole 1024-column tiles
    const int nchunk = (K + 1023) >> 10;

    const int blk = blockIdx.x;
    const int s = MOE ? (SWIGLU ? 2 * expert : expert) : (SWIGLU ? 0 : find_segment(p, blk));
    const T12Segment& sg = p.seg[s];
    const int M = sg.M;
    // row r of this wave: tensor SEG(r), matrix row ROW(r)
#define SEG(r) (SWIGLU ? p.seg[(MOE ? s : 0) + (r)] : sg)
#define ROW(r) (SWIGLU ? row0 : row0 + (r))
    const int row0 = SWIGLU ? blk * NW + wave : (blk - (MOE ? 0 : p.blk_start[s])) * (NW * R) + wave * R;
    const bool live = row0 < M;                // wave-uniform
    uint32_t be2r[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        be2r[r] = t12_opaque(((uint32_t)SEG(r).base_exp << 7) | ((uint32_t)SEG(r).base_exp << 23));

    // The activations are requested FIRST: they come out of the L2 (every workgroup reads the same vector) and so
    // arrive before the weight tiles requested behind them; loads complete in order, so requested after the tiles
    // they would wait for HBM, and staged in a loop they would cost one round trip per pass.  Piece q = 8 columns.
    constexpr int SU = 4;                      // pieces per thread requested up front (16 * NW * 64 * SU / 8 columns)
    uint4 xpre[SU];
    if (NORM == 0) {
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const int k = (tid + u * NW * 64) * 8;
            xpre[u] = make_uint4(0, 0, 0, 0);
            if (u == 0 || u * NW * 64 * 8 < K)                       // workgroup-uniform
                xpre[u] = *(const uint4*)(act_row + min(k, K - 8));  // (clamped: columns >= K are zeroed below)
        }
    }

    // NORM: the same for the fp32 residual stream, its addend and the norm weights (8 columns per piece, 2 pieces per thread)
    float4 npre[NORM ? 2 : 1][2], rpre[NORM == 2 ? 2 : 1][2], wpre[NORM ? 2 : 1][2];
    if (NORM != 0) {
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const int k = min((tid + gi * NW * 64) * 8, K - 8);      // (clamped: pieces beyond K are not used)
            if (gi == 0 || NW * 64 * 8 < K) {                        // workgroup-uniform
                npre[gi][0] = *(const float4*)(p.nx + k);
                npre[gi][1] = *(const float4*)(p.nx + k + 4);
                if (NORM == 2) {
                    rpre[gi][0] = *(const float4*)(p.nres + k);
                    rpre[gi][1] = *(const float4*)(p.nres + k + 4);
                }
                wpre[gi][0] = *(const float4*)(p.nw + k);
                wpre[gi][1] = *(const float4*)(p.nw + k + 4);
            }
        }
    }

    // CSR row pointers: lane 2r holds the begin and lane 2r+1 the end of row r's escape slice
    int ro = 0;
    if (live && lane < 2 * R) {
        const T12Segment& g = SEG(lane >> 1);
        if (g.row_off) ro = g.row_off[min(ROW(lane >> 1) + (lane & 1), M)];
    }

    const uint8_t* smp[R];
    const uint8_t* grp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const size_t e = (size_t)min(ROW(r), M - 1) * K;        // clamp: loads stay in bounds
        smp[r] = SEG(r).sm + e + lane * 16;
        grp[r] = SEG(r).gr + (e >> 1) + lane * 8;
    }

    constexpr int DR = D > 0 ? D : 1;          // the K tail borrows slot 0
    uint4 ringS[DR][R];
    uint2 ringG[DR][R];
#define T12_FETCH(slot, tile)                                                   \
    _Pragma("unroll") for (int r = 0; r < R; r++) {                             \
        ringS[slot][r] = t12_ldg_stream16(smp[r] + (size_t)(tile) * 1024);      \
        ringG[slot][r] = t12_ldg_stream8(grp[r] + (size_t)(tile) * 512);        \
    }
#define T12_CONSUME(slot, tile)                                                                        \
    {                                                                                                  \
        const uint4 a0 = lds_act[(tile) * 128 + lane];                                                 \
        const uint4 a1 = lds_act[(tile) * 128 + 64 + lane];                                            \
        _Pragma("unroll") for (int r = 0; r < R; r++) {                                                \
            acc[r] = t12_decode_dot8(ringS[slot][r].x, ringS[slot][r].y, ringG[slot][r].x, be2r[r], a0, acc[r]); \
            acc[r] = t12_decode_dot8(ringS[slot][r].z, ringS[slot][r].w, ringG[slot][r].y, be2r[r], a1, acc[r]); \
        }                                                                                              \
    }

    // the host picks D <= T, so the first D tiles always exist (rows are clamped)
#pragma unroll
    for (int d = 0; d < D; d++) {
        T12_FETCH(d, d)
        __builtin_amdgcn_sched_barrier(0);   // issue in ring order: waits can then be partial
    }

    if (NORM == 0) {
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const int q = tid + u * NW * 64;
            if (q < nchunk * 128)
                lds_act[(q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1)] =
                    t12_pair_acts(q * 8 < K ? xpre[u] : make_uint4(0, 0, 0, 0));
        }
        for (int q = tid + SU * NW * 64; q < nchunk * 128; q += NW * 64) {     // K beyond the pieces requested up front
            const int k = q * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (k < K) v = *(const uint4*)(act_row + k);
            lds_act[(q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1)] = t12_pair_acts(v);
        }
    } else {
        __shared__ float red[NW];
        float v[2][8];
        float ss = 0.0f;
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const int k = (tid + gi * NW * 64) * 8;
#pragma unroll
            for (int e = 0; e < 8; e++) v[gi][e] = 0.0f;
            if (k < K) {
                const float4 a = npre[gi][0], b = npre[gi][1];
                v[gi][0] = a.x; v[gi][1] = a.y; v[gi][2] = a.z; v[gi][3] = a.w;
                v[gi][4] = b.x; v[gi][5] = b.y; v[gi][6] = b.z; v[gi][7] = b.w;
                if (NORM == 2) {
                    const float4 c = rpre[gi][0], d = rpre[gi][1];
                    v[gi][0] += c.x; v[gi][1] += c.y; v[gi][2] += c.z; v[gi][3] += c.w;
                    v[gi][4] += d.x; v[gi][5] += d.y; v[gi][6] += d.z; v[gi][7] += d.w;
                    if (blockIdx.x == 0 && p.hidden_out) {
                        *(float4*)(p.hidden_out + k) = make_float4(v[gi][0], v[gi][1], v[gi][2], v[gi][3]);
                        *(float4*)(p.hidden_out + k + 4) = make_float4(v[gi][4], v[gi][5], v[gi][6], v[gi][7]);
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; e++) ss += v[gi][e] * v[gi][e];
            }
        }
        ss = t12_wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; w++) tot += red[w];
        const float rn = rsqrtf(tot / (float)K + p.eps);
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const int q = tid + gi * NW * 64;
            const int k = q * 8;
            if (q < nchunk * 128) {
                uint4 y = make_uint4(0, 0, 0, 0);
                if (k < K) {
                    const float4 wa = wpre[gi][0], wb = wpre[gi][1];
                    y.x = t12_f32_to_bf16(v[gi][0] * rn * wa.x) | ((uint32_t)t12_f32_to_bf16(v[gi][1] * rn * wa.y) << 16);
                    y.y = t12_f32_to_bf16(v[gi][2] * rn * wa.z) | ((uint32_t)t12_f32_to_bf16(v[gi][3] * rn * wa.w) << 16);
                    y.z = t12_f32_to_bf16(v[gi][4] * rn * wb.x) | ((uint32_t)t12_f32_to_bf16(v[gi][5] * rn * wb.y) << 16);
                    y.w = t12_f32_to_bf16(v[gi][6] * rn * wb.z) | ((uint32_t)t12_f32_to_bf16(v[gi][7] * rn * wb.w) << 16);
                }
                lds_act[(q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1)] = t12_pair_acts(y);
            }
        }
    }
    __syncthreads();
    if (!live) return;

    // escape entries: lane l takes entry beg + l of each row
    // (kept as loaded until the row's sum is formed: arithmetic on a requested value right here would make the wave
    // wait for it, a full memory latency, before it consumes its first tile)
    int pcol[R];
    int pcorrect[R], pwrong[R];              // (the arrays' own 16-bit integers, widened by the load itself)
    int pend[R], pnext[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int beg = __builtin_amdgcn_readlane(ro, 2 * r), end = __builtin_amdgcn_readlane(ro, 2 * r + 1);
        pend[r] = end;
        pnext[r] = beg + T12_WAVE;
        pcol[r] = -1;
        pcorrect[r] = pwrong[r] = 0;
        if (beg + lane < end) {                          // end > beg only when the tensor has a list
            pcol[r] = SEG(r).cols[beg + lane];
            pcorrect[r] = SEG(r).correct[beg + lane];
            pwrong[r] = SEG(r).wrong[beg + lane];
        }
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;

    int t = 0;
    // steady state: whole ring rotations in which every slot is refilled
    for (; D > 0 && t + 2 * D <= T; t += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            T12_CONSUME(d, t + d)
            T12_FETCH(d, t + d + D)
            __builtin_amdgcn_sched_barrier(0);   // keep the refill right behind its consumer
        }
    }
    // drain: the last (up to 2D - 1) tiles
    for (; D > 0 && t < T; t += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (t + d < T) {
                T12_CONSUME(d, t + d)
                if (t + d + D < T) { T12_FETCH(d, t + d + D) }
            }
        }
    }
    if (T < nchunk && T * 1024 + lane * 16 < K) {   // K tail: whole 16-column pieces
        T12_FETCH(0, T)
        T12_CONSUME(0, T)
    }
#undef T12_FETCH
#undef T12_CONSUME

    float tot[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        tot[r] = 0.0f;
        if (ROW(r) < M) {                                // wave-uniform
            float v = acc[r];
            if (pcol[r] >= 0) v += (t12_bf16_to_f32((uint16_t)pcorrect[r]) - t12_bf16_to_f32((uint16_t)pwrong[r])) * lds_act_at(lds_act, pcol[r]);
            for (int q = pnext[r] + lane; q < pend[r]; q += T12_WAVE)     // rows with > 64 escapes
                v += (t12_bf16_to_f32((uint16_t)SEG(r).correct[q]) - t12_bf16_to_f32((uint16_t)SEG(r).wrong[q])) *
                     lds_act_at(lds_act, SEG(r).cols[q]);
            tot[r] = t12_wave_sum_lane63(v);
            if (!SWIGLU && lane == 63) {
                if (MOE) sg.out[(size_t)blockIdx.y * p.out_ld + row0 + r] = tot[r];
                else sg.out[row0 + r] = p.add ? tot[r] + p.add[row0 + r] : tot[r];
            }
        }
    }
    if (SWIGLU && lane == 63) {
        const float g = tot[0];
        (MOE ? p.out_bf16 + (size_t)blockIdx.y * p.out_ld : p.out_bf16)[row0] = t12_f32_to_bf16(g / (1.0f + expf(-g)) * tot[R - 1]);
    }
#undef SEG
#undef ROW
}

// ---------------------------------------------------------------------------
// General path: any K (odd included: nibble parity follows the flat element
// index), any base_exp (-1 included, where the "wrong" value of an escape is a
// NaN/Inf pattern).  One wave per row, scalar decode rule.  With an escape list
// the group-0 elements are skipped in the stream and taken exactly from the
// list; without one they decode to the wrong value like the reference's
// unpatched kernels.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemv_general_kernel(const GemvParams p)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int blk = blockIdx.x;
    const int s = find_segment(p, blk);
    const T12Segment& sg = p.seg[s];
    const int row = (blk - p.blk_start[s]) * 4 + wave;
    if (row >= sg.M) return;
    const int K = p.K;
    const size_t base = (size_t)row * K;
    float acc = 0.0f;
    for (int k = lane; k < K; k += T12_WAVE) {
        const size_t i = base + k;
        const uint32_t g = (sg.gr[i >> 1] >> (4 * (i & 1))) & 0xFu;
        const uint16_t w = t12_decode_scalar(sg.sm[i], g, sg.base_exp);
        if (g != 0 || !sg.row_off) acc += t12_bf16_to_f32(w) * t12_bf16_to_f32(p.act[k]);
    }
    acc += patch_partial<false>(sg, row, lane, p.act);
    acc = t12_wave_sum(acc);
    if (lane == 0) sg.out[row] = p.add ? acc + p.add[row] : acc;
}

// Only the escape corrections (the reference's separate patch kernels): out[row] += sum over the row's entries of
// (correct - wrong) * x[col].  Eight lanes per row (a row of an LLM tensor holds a handful of entries: one step), 32
// rows per workgroup; the eight partial sums are folded with three xor exchanges, in an order that does not depend on
// timing.  A row without entries is not written.
constexpr int PATCH_LANES = 8;
constexpr int PATCH_ROWS = 256 / PATCH_LANES;          // rows per workgroup; blk_start counts such groups
__global__ __launch_bounds__(256) void patches_kernel(const GemvParams p)
{
    const int sub = threadIdx.x & (PATCH_LANES - 1), rloc = threadIdx.x / PATCH_LANES;
    const int blk = blockIdx.x;
    const int s = find_segment(p, blk);
    const T12Segment& sg = p.seg[s];
    const int row = (blk - p.blk_start[s]) * PATCH_ROWS + rloc;
    float c = 0.0f;
    bool any = false;
    if (row < sg.M) {
        const int beg = sg.row_off[row], end = sg.row_off[row + 1];
        any = end > beg;
        for (int q = beg + sub; q < end; q += PATCH_LANES)
            c += (t12_bf16_to_f32((uint16_t)sg.correct[q]) - t12_bf16_to_f32((uint16_t)sg.wrong[q])) *
                 t12_bf16_to_f32(p.act[sg.cols[q]]);
    }
#pragma unroll
    for (int off = PATCH_LANES / 2; off > 0; off >>= 1) c += __shfl_xor(c, off, T12_WAVE);
    if (sub == 0 && any && c != 0.0f) sg.out[row] += c;
}

template <int NW, int R, int D, int MINB = 1>
int launch_stream(GemvParams& p, const T12Segment* segs, int nseg, hipStream_t st)
{
    int total = 0;
    for (int i = 0; i < nseg; i++) {
        p.blk_start[i] = total;
        total += (segs[i].M + NW * R - 1) / (NW * R);
    }
    p.blk_start[nseg] = total;
    const size_t lds = (size_t)((p.K + 1023) / 1024) * 2048;
    hipLaunchKernelGGL((gemv_stream_kernel<NW, R, D, MINB>), dim3(total), dim3(NW * 64), lds, st, p);
    T12_CHECK_LAUNCH("t12_gemv");
    return T12_OK;
}

template <int NORM>
int launch_swiglu(GemvParams& p, hipStream_t st)
{
    const int NW = 8;
    const int total = (p.seg[0].M + NW - 1) / NW;
    p.blk_start[0] = 0;
    p.blk_start[1] = p.blk_start[2] = total;
    const size_t lds = (size_t)((p.K + 1023) / 1024) * 2048;
    const int T = p.K / 1024;
    if (T >= 2)
        hipLaunchKernelGGL((gemv_stream_kernel<8, 2, 2, 1, true, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    else if (T == 1)
        hipLaunchKernelGGL((gemv_stream_kernel<8, 2, 1, 1, true, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    else
        hipLaunchKernelGGL((gemv_stream_kernel<8, 2, 0, 1, true, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    T12_CHECK_LAUNCH("t12_gemv_swiglu");
    return T12_OK;
}

template <int NORM>
int launch_plain_norm(GemvParams& p, const T12Segment* segs, int nseg, hipStream_t st)
{
    const int NW = 8;
    int total = 0;
    for (int i = 0; i < nseg; i++) {
        p.blk_start[i] = total;
        total += (segs[i].M + NW - 1) / NW;
    }
    p.blk_start[nseg] = total;
    const size_t lds = (size_t)((p.K + 1023) / 1024) * 2048;
    const int T = p.K / 1024;
    if (T >= 2)
        hipLaunchKernelGGL((gemv_stream_kernel<8, 1, 2, 1, false, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    else if (T == 1)
        hipLaunchKernelGGL((gemv_stream_kernel<8, 1, 1, 1, false, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    else
        hipLaunchKernelGGL((gemv_stream_kernel<8, 1, 0, 1, false, NORM>), dim3(total), dim3(NW * 64), lds, st, p);
    T12_CHECK_LAUNCH("t12_gemv_norm");
    return T12_OK;
}

int check_norm_operands(const char* who, const T12Segment* segs, int nseg, const float* x, const float* residual,
                        const float* norm_w, const float* hidden_out, int K)
{
    T12_REQUIRE(x && norm_w, "%s: x / norm weight is null", who);
    T12_REQUIRE(K % 16 == 0 && K <= 8192, "%s: K %d must be a multiple of 16 and <= 8192", who, K);
    T12_REQUIRE(!hidden_out || (hidden_out != x && hidden_out != residual), "%s: hidden_out may not alias x or residual", who);
    for (int i = 0; i < nseg; i++)
        T12_REQUIRE(segs[i].base_exp >= 0 && segs[i].base_exp <= 240, "%s: segment %d base_exp %d outside 0..240", who, i,
                    segs[i].base_exp);
    return T12_OK;
}

int validate(const T12Segment* segs, int nseg, const void* act, int K, bool need_out)
{
    T12_REQUIRE(segs && nseg >= 1 && nseg <= T12_MAX_SEGMENTS, "nseg must be 1..%d (got %d)", T12_MAX_SEGMENTS, nseg);
    T12_REQUIRE(act && K >= 1, "activations null or K < 1 (K=%d)", K);
    for (int i = 0; i < nseg; i++) {
        const T12Segment& g = segs[i];
        T12_REQUIRE(g.M >= 1, "segment %d: M must be >= 1 (got %d)", i, g.M);
        T12_REQUIRE(g.sm && g.gr, "segment %d: sm/gr plane is null", i);
        T12_REQUIRE(!need_out || g.out, "segment %d: output is null", i);
        T12_REQUIRE(!g.row_off || (g.cols && g.correct && g.wrong),
                    "segment %d: row_off given without cols/correct/wrong", i);
        T12_REQUIRE(g.base_exp >= -1 && g.base_exp <= 254, "segment %d: base_exp %d out of range", i, g.base_exp);
    }
    return T12_OK;
}

int gemv_impl(const T12Segment* segs, int nseg, const void* act_bf16, int K, const float* add, void* stream);

}  // namespace

extern "C" {

int t12_gemv(const T12Segment* segs, int nseg, const void* act_bf16, int K, void* stream)
{
    return gemv_impl(segs, nseg, act_bf16, K, nullptr, stream);
}

// out[m] = residual[m] + W[m,:] . act : the residual add that follows wo / w_down in a decoder layer
// (the first half of add_rms_norm_bf16_batch, engine/kernels.hip:399-442) folded into the GEMV's store.
int t12_gemv_add(const T12Segment* seg, const void* act_bf16, int K, const float* residual, void* stream)
{
    T12_REQUIRE(residual, "t12_gemv_add: residual is null");
    return gemv_impl(seg, 1, act_bf16, K, residual, stream);
}

}  // extern "C"

namespace {

int gemv_impl(const T12Segment* segs, int nseg, const void* act_bf16, int K, const float* add, void* stream)
{
    int rc = validate(segs, nseg, act_bf16, K, true);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    GemvParams p;
    p.nseg = nseg;
    p.K = K;
    p.act = (const uint16_t*)act_bf16;
    p.out_bf16 = nullptr;
    p.add = add;
    bool fast = (K % 16 == 0) && ((K + 1023) / 1024 * 2048 <= 160 * 1024);
    for (int i = 0; i < nseg; i++) {
        p.seg[i] = segs[i];
        if (segs[i].base_exp < 0 || segs[i].base_exp > 240) fast = false;
    }
    if (!fast) {
        int total = 0;
        for (int i = 0; i < nseg; i++) {
            p.blk_start[i] = total;
            total += (segs[i].M + 3) / 4;
        }
        p.blk_start[nseg] = total;
        hipLaunchKernelGGL(gemv_general_kernel, dim3(total), dim3(256), 0, st, p);
        T12_CHECK_LAUNCH("t12_gemv(general)");
        return T12_OK;
    }
    // 8 waves x 1 row per wave x a ring two tiles deep (as deep as the row has whole 1024-column tiles): measured on
    // MI355X over the Llama-3.1-8B layer shapes against 4-wave workgroups, two and four rows per wave and rings of
    // depth 4, this is the fastest everywhere -- the chip hides HBM latency better with many light waves (62 VGPRs,
    // 8 waves per SIMD) than with deep per-wave rings.
    const int T = K / 1024;
    if (T >= 2) return launch_stream<8, 1, 2>(p, segs, nseg, st);
    if (T == 1) return launch_stream<8, 1, 1>(p, segs, nseg, st);
    return launch_stream<8, 1, 0>(p, segs, nseg, st);
}

}  // namespace

extern "C" {

// out_bf16[m] = bf16( silu(gate[m,:].x) * (up[m,:].x) ), escapes exact, one launch.
int t12_gemv_swiglu(const T12Segment* gate, const T12Segment* up, const void* act_bf16, int K, void* out_bf16,
                    void* stream)
{
    T12_REQUIRE(gate && up && out_bf16, "t12_gemv_swiglu: null operand");
    T12Segment two[2] = {*gate, *up};
    int rc = validate(two, 2, act_bf16, K, false);
    if (rc) return rc;
    T12_REQUIRE(gate->M == up->M, "t12_gemv_swiglu: gate has %d rows, up has %d", gate->M, up->M);
    T12_REQUIRE(K % 16 == 0 && (K + 1023) / 1024 * 2048 <= 160 * 1024, "t12_gemv_swiglu: K %d must be a multiple of 16", K);
    T12_REQUIRE(gate->base_exp >= 0 && gate->base_exp <= 240 && up->base_exp >= 0 && up->base_exp <= 240,
                "t12_gemv_swiglu: base_exp outside 0..240 (use t12_gemv + launch_silu_mul_bf16_batch)");
    GemvParams p;
    p.seg[0] = two[0];
    p.seg[1] = two[1];
    p.nseg = 2;
    p.K = K;
    p.act = (const uint16_t*)act_bf16;
    p.out_bf16 = (uint16_t*)out_bf16;
    p.add = nullptr;
    return launch_swiglu<0>(p, (hipStream_t)stream);
}

// y_s = W_s . bf16(rmsnorm(x [+ residual]) * norm_w) with the norm computed in the kernel's prologue.
int t12_gemv_norm(const T12Segment* segs, int nseg, const float* x, const float* residual, const float* norm_w, float eps,
                  float* hidden_out, int K, void* stream)
{
    int rc = validate(segs, nseg, x, K, true);
    if (rc) return rc;
    rc = check_norm_operands("t12_gemv_norm", segs, nseg, x, residual, norm_w, hidden_out, K);
    if (rc) return rc;
    GemvParams p;
    for (int i = 0; i < nseg; i++) p.seg[i] = segs[i];
    p.nseg = nseg;
    p.K = K;
    p.act = nullptr;
    p.out_bf16 = nullptr;
    p.add = nullptr;
    p.nx = x;
    p.nres = residual;
    p.nw = norm_w;
    p.hidden_out = hidden_out;
    p.eps = eps;
    return residual ? launch_plain_norm<2>(p, segs, nseg, (hipStream_t)stream)
                    : launch_plain_norm<1>(p, segs, nseg, (hipStream_t)stream);
}

int t12_gemv_swiglu_norm(const T12Segment* gate, const T12Segment* up, const float* x, const float* residual,
                         const float* norm_w, float eps, float* hidden_out, int K, void* out_bf16, void* stream)
{
    T12_REQUIRE(gate && up && out_bf16, "t12_gemv_swiglu_norm: null operand");
    T12Segment two[2] = {*gate, *up};
    int rc = validate(two, 2, x, K, false);
    if (rc) return rc;
    T12_REQUIRE(gate->M == up->M, "t12_gemv_swiglu_norm: gate has %d rows, up has %d", gate->M, up->M);
    rc = check_norm_operands("t12_gemv_swiglu_norm", two, 2, x, residual, norm_w, hidden_out, K);
    if (rc) return rc;
    GemvParams p;
    p.seg[0] = two[0];
    p.seg[1] = two[1];
    p.nseg = 2;
    p.K = K;
    p.act = nullptr;
    p.out_bf16 = (uint16_t*)out_bf16;
    p.add = nullptr;
    p.nx = x;
    p.nres = residual;
    p.nw = norm_w;
    p.hidden_out = hidden_out;
    p.eps = eps;
    return residual ? launch_swiglu<2>(p, (hipStream_t)stream) : launch_swiglu<1>(p, (hipStream_t)stream);
}

// One activation row per slot, each multiplied with the tensors of the expert the routing gave the slot (a device
// table): the few-row step of a mixture-of-experts layer, where every named expert is streamed at the rate of the B = 1
// kernel.  per_expert = 2: segs = (gate, up) per expert, out_bf16[slot, m] = bf16(silu(gate . x) * (up . x));
// per_expert = 1: segs[e].out[slot * out_ld + m] = W_e[m, :] . x_slot.  Returns 1 when the shape has no such kernel
// (K not a multiple of 16 or under two tiles, base_exp outside 0..240, more than sixteen segments, misaligned rows).
__attribute__((visibility("hidden"))) int t12_gemv_experts(const T12Segment* segs, int per_expert, int E, int K,
                                                           const void* act_bf16, int act_stride, const int* slot_expert,
                                                           int slots, void* out_bf16, int out_ld, void* stream)
{
    if (per_expert < 1 || per_expert > 2 || E < 1 || E * per_expert > GEMV_SEGS || slots < 1) return 1;
    if (K % 16 != 0 || K < 2048 || (size_t)((K + 1023) / 1024) * 2048 > 160 * 1024) return 1;
    if (act_stride % 8 != 0 || (uintptr_t)act_bf16 % 16 != 0) return 1;
    const int M = segs[0].M;
    GemvParams p;
    for (int i = 0; i < E * per_expert; i++) {
        const T12Segment& g = segs[i];
        if (g.M != M || !g.sm || !g.gr || g.base_exp < 0 || g.base_exp > 240) return 1;
        if (g.row_off && !(g.cols && g.correct && g.wrong)) return 1;
        if (per_expert == 1 && !g.out) return 1;
        p.seg[i] = g;
    }
    if (per_expert == 2 && !out_bf16) return 1;
    p.nseg = E * per_expert;
    p.K = K;
    p.act = (const uint16_t*)act_bf16;
    p.out_bf16 = (uint16_t*)out_bf16;
    p.add = nullptr;
    p.slot_expert = slot_expert;
    p.act_stride = act_stride;
    p.out_ld = out_ld;
    const int NW = 8;
    const size_t lds = (size_t)((K + 1023) / 1024) * 2048;
    const dim3 grid((M + NW - 1) / NW, slots);
    if (per_expert == 2)
        hipLaunchKernelGGL((gemv_stream_kernel<8, 2, 2, 1, true, 0, true>), grid, dim3(NW * 64), lds, (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL((gemv_stream_kernel<8, 1, 2, 1, false, 0, true>), grid, dim3(NW * 64), lds, (hipStream_t)stream, p);
    T12_CHECK_LAUNCH("t12_moe_ffn(gemv)");
    return T12_OK;
}

// ---- reference-named launchers ---------------------------------------------
int launch_split12_v2_async(const void* sign_mantissa, const void* groups, int base_exp,
                            const void* activations, void* output, int M, int K, void* stream)
{
    T12Segment g = {(const uint8_t*)sign_mantissa, (const uint8_t*)groups, nullptr, nullptr, nullptr, nullptr,
                    (float*)output, M, base_exp, 0, 0};
    return t12_gemv(&g, 1, activations, K, stream);
}

int launch_split12_v2_dual_async(const void* sm_a, const void* gr_a, int base_exp_a,
                                 const void* sm_b, const void* gr_b, int base_exp_b,
                                 const void* activations, void* output_a, void* output_b,
                                 int M, int K, void* stream)
{
    T12Segment g[2] = {
        {(const uint8_t*)sm_a, (const uint8_t*)gr_a, nullptr, nullptr, nullptr, nullptr, (float*)output_a, M, base_exp_a, 0, 0},
        {(const uint8_t*)sm_b, (const uint8_t*)gr_b, nullptr, nullptr, nullptr, nullptr, (float*)output_b, M, base_exp_b, 0, 0}};
    return t12_gemv(g, 2, activations, K, stream);
}

static int launch_patch_descs(const PatchBatchDesc* d, int n, hipStream_t st)
{
    // all descriptors of one call read the same activation vector in the reference's
    // call sites (inference.cpp:263-269, 318-322); different vectors get one launch each
    int i = 0;
    while (i < n) {
        GemvParams p;
        int cnt = 0, total = 0;
        p.act = (const uint16_t*)d[i].activations;
        while (i < n && cnt < T12_MAX_SEGMENTS && (const uint16_t*)d[i].activations == p.act) {
            T12Segment& g = p.seg[cnt];
            g.sm = g.gr = nullptr;
            g.row_off = d[i].row_offsets;
            g.cols = d[i].patch_cols;
            g.correct = d[i].patch_correct;
            g.wrong = d[i].patch_wrong;
            g.out = d[i].output;
            g.M = d[i].M;
            g.base_exp = 0;
            g.out_stride = g.reserved = 0;
            p.blk_start[cnt] = total;
            total += (d[i].M + PATCH_ROWS - 1) / PATCH_ROWS;
            cnt++;
            i++;
        }
        p.blk_start[cnt] = total;
        p.nseg = cnt;
        p.K = 0;
        if (total > 0) {
            hipLaunchKernelGGL(patches_kernel, dim3(total), dim3(256), 0, st, p);
            T12_CHECK_LAUNCH("launch_patches");
        }
    }
    return T12_OK;
}

int launch_patches_v2_async(const void* row_offsets, const void* patch_cols, const void* correct_vals,
                            const void* wrong_vals, const void* activations, void* output, int M, void* stream)
{
    if (M == 0) return 0;
    T12_REQUIRE(row_offsets && patch_cols && correct_vals && wrong_vals && activations && output && M > 0,
                "launch_patches_v2_async: null operand or M < 0");
    PatchBatchDesc d = {(const int32_t*)row_offsets, (const int32_t*)patch_cols, (const int16_t*)correct_vals,
                        (const int16_t*)wrong_vals, (const int16_t*)activations, (float*)output, M};
    return launch_patch_descs(&d, 1, (hipStream_t)stream);
}

int launch_patches_v2(const void* row_offsets, const void* patch_cols, const void* correct_vals,
                      const void* wrong_vals, const void* activations, void* output, int M)
{
    int rc = launch_patches_v2_async(row_offsets, patch_cols, correct_vals, wrong_vals, activations, output, M, nullptr);
    if (rc) return -1;
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}

// descs_gpu is accepted for signature compatibility and left untouched: the
// descriptors travel as kernel arguments, so no host-to-device copy is needed.
int launch_patches_b1_batched_async(void* descs_gpu, const void* descs_cpu, int num_descs, int max_M, void* stream)
{
    (void)descs_gpu;
    if (num_descs == 0 || max_M == 0) return 0;
    T12_REQUIRE(descs_cpu && num_descs > 0 && num_descs <= 8, "launch_patches_b1_batched_async: 1..8 descriptors");
    const PatchBatchDesc* d = (const PatchBatchDesc*)descs_cpu;
    for (int i = 0; i < num_descs; i++)
        T12_REQUIRE(d[i].row_offsets && d[i].patch_cols && d[i].patch_correct && d[i].patch_wrong &&
                        d[i].activations && d[i].output && d[i].M > 0,
                    "launch_patches_b1_batched_async: descriptor %d has a null field", i);
    return launch_patch_descs(d, num_descs, (hipStream_t)stream);
}

}  // extern "C"
