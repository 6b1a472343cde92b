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
//   * The compressed planes are loaded into registers, rebuilt to bf16 there, two
//     weights per VGPR (t12_decode8), and written once per workgroup into a bf16 tile
//     in LDS from which the waves read their MFMA B fragments: every weight is
//     decoded once per workgroup, no bf16 copy of W ever exists in HBM.  The
//     activations are staged already paired the way t12_decode8 orders its
//     outputs, so no operand shuffling is needed.
//   * Eight waves per workgroup (two per SIMD), laid out WB x WM; a wave owns FB x FM 32x32
//     accumulator tiles: batch tiles of 64 (2 x 4 waves, 1 x 1), 128 (2 x 4, 2 x 1) and
//     256 rows (4 x 2, 2 x 2).
//   * Few row tiles (small M) are split along K across workgroups; the partial
//     sums go to a workspace and a second kernel adds them in a fixed order
//     (deterministic) -- or the caller's next kernel does (t12_gemm_deferred).
//   * Escapes are EXACT and cost no extra pass: the (column, exact bf16) pairs of
//     the workgroup's 128 rows -- one contiguous slice of the CSR list -- are
//     staged in LDS once; the thread that decoded 16 columns of a row walks that
//     row's slice in step with the K loop and overwrites the decoded half-words
//     in the LDS tile.
//
// Fast path requirements: K % 64 == 0, 0 <= base_exp <= 240, 16-byte aligned
// activation rows.  Everything else goes to the general kernel below.

#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "t12_device.h"
#include "t12_host.h"
#include "dense16_plan.h"

// library-internal (hidden: not part of the ABI)
extern "C" __attribute__((visibility("hidden"))) void t12_glue_release_stream(hipStream_t st);      // glue.hip
extern "C" __attribute__((visibility("hidden"))) void t12_sampler_release_stream(hipStream_t st);   // engine/sampler.cpp

namespace {

constexpr int KC = 64;          // K columns staged per pipeline stage
constexpr int TM = 128;         // weight rows per workgroup
constexpr int PCAP = 2048;      // escape entries a workgroup can stage in LDS
constexpr int PATCH_BYTES = PCAP * 4 + (TM + 1) * 4 + 12;
constexpr int NO_ESCAPE = 0x7FFFFFFF;

constexpr int GMAX = 16;        // segments of one launch (a grouped launch: gate and up of eight experts)
static_assert(GMAX >= T12_MAX_SEGMENTS, "t12_gemm takes T12_MAX_SEGMENTS segments");

// One launch multiplies up to GMAX tensors.  t12_gemm: all of them with the same activations [B, K]; a grouped
// launch (t12_gemm_grouped): segment i with its own seg_act[i] of seg_B[i] rows.  The tile kernel and the K-split
// reduction read the per-segment fields, which t12_gemm fills with the shared values; the other kernels read
// act / B / act_stride.
struct GemmParams {
    T12Segment seg[GMAX];
    int blk_start[GMAX + 1];               // first row-tile of each segment
    int seg_row0[GMAX];                    // first row of each segment among all rows of the launch
    const uint16_t* seg_act[GMAX];
    int seg_B[GMAX];
    int seg_act_stride[GMAX];
    // partial sums of segment i, split z, element (b, m): ws[z * split_stride + seg_ws0[i] + b * seg_ld[i] + m]
    //   t12_gemm: seg_ws0 = seg_row0, seg_ld = m_total (rows of length m_total, what t12_gemm_deferred describes)
    //   grouped:  seg_ws0 = sum of B * M over the segments before, seg_ld = M
    size_t seg_ws0[GMAX];
    int seg_ld[GMAX];
    size_t split_stride;
    int nseg;
    int K, B;                              // B: t12_gemm's batch; grouped: the largest seg_B
    int act_stride;
    int ksplit;                            // workgroups along K
    int kslice;                            // columns per K split (multiple of KC)
    int m_total;                           // sum of M over segments
    const uint16_t* act;
    float* ws;                             // partial sums when ksplit > 1
    uint16_t* out_bf16;                    // SwiGLU mode: bf16 [B, out_bf16_ld], silu(seg 2i) * seg 2i+1 of pair i
    int out_bf16_ld;
    int npair = 1;                         // SwiGLU mode: (gate, up) pairs of the launch; blk_start[i] = first tile of pair i
    // Rows per group known on the device only (the experts of a mixture-of-experts layer, counted by the routing
    // kernel): group_of_seg[s] picks an entry of dev_counts / dev_base, the segment's batch is dev_counts[.] and its
    // activations, outputs (fp32 and bf16) start dev_base[.] rows into the pointers given.  The grid then has one
    // workgroup per row tile, which walks the group's batch tiles.  nullptr: seg_B as given.
    const int* dev_counts = nullptr;
    const int* dev_base = nullptr;
    int group_of_seg[GMAX];
    int n_first = 0;                       // mixed small-batch launch: segments [0, n_first) take the larger workgroups
};

// LDS slot of (unit, row) in a [units][rows] array of 16-byte units.  Rows are rotated
// inside their aligned block of eight by the unit index, so that both access patterns are
// bank-conflict free: the staging writes (neighbouring lanes = the units of one row) and
// the fragment reads (neighbouring lanes = consecutive rows of one unit).
__device__ __forceinline__ int lds_slot(int u, int r, int rows) { return u * rows + (r & ~7) + ((r + u) & 7); }

// Order in which a thread's staging units are stored: the ndec decode units (18 VALU each) evenly
// among the nact activation units (4 VALU each).  Position pos -> unit index (activation units
// 0 .. nact-1, decode units nact .. nact+ndec-1).
__device__ __forceinline__ constexpr int stage_unit_order(int pos, int nact, int ndec)
{
    const int nu = nact + ndec;
    const int dec_before = pos * ndec / nu;              // decode units placed before pos
    const bool is_dec = (pos + 1) * ndec / nu > dec_before;
    return is_dec ? nact + dec_before : pos - dec_before;
}

__device__ __forceinline__ int find_segment(const GemmParams& p, int tile)
{
    int s = 0;
#pragma unroll
    for (int i = 1; i < GMAX; i++)
        if (i < p.nseg && tile >= p.blk_start[i]) s = i;
    return s;
}
__device__ __forceinline__ int find_pair(const GemmParams& p, int tile)
{
    int s = 0;
#pragma unroll
    for (int i = 1; i < GMAX / 2; i++)
        if (i < p.npair && tile >= p.blk_start[i]) s = i;
    return s;
}

// ---------------------------------------------------------------------------
// LDS stage layout (one of two buffers), unit u = (k % 64) / 8 = eight bf16 of one row,
// paired (i, i + 4) per dword the way t12_decode8 / t12_pair_acts order them:
//   act  [8 units][TB rows] x 16 B
//   w    [8 units][TM rows] x 16 B     decoded weights
// MFMA k-step t of a stage covers columns 16t .. 16t+15; the lanes of wave half h take
// unit 2t + h of their row, for both operands.
//
// Global loads.  A stage is 64 columns: 128 B of an activation row (one cache line) but
// only 64 B of a row's sm plane and 32 B of its gr plane.  Fetching those a stage at a
// time asks HBM for every line twice or more (the rows of a tile are K bytes apart, a
// power of two: they fall into a handful of L2 sets and are evicted before the next
// stage comes back for the other half).  So weights are loaded per WINDOW of two stages
// (128 columns), both halves of a line in back-to-back instructions:
//   piece X (used by the even stage): lanes c8 < 4 take row rr, columns 16*c8 ..;
//                                     lanes c8 >= 4 take row 64 + (rr^1), columns 16*(c8-4) ..
//   piece Y (used by the odd stage) : the other halves of the same two lines, lanes swapped
// where c8 = tid % 8, rr = item / 8 in 0..63.  Every lane decodes one piece per item and
// stage (balanced), every sm line is requested whole within two instructions, and the
// rr^1 keeps the LDS writes of the two lane groups on different banks.
// ---------------------------------------------------------------------------
// SWI (two segments of equal M, gate and up; FM == 2): a tile holds 64 rows of each, interleaved in
// blocks of 32 -- local rows [0,32) gate rows 0..31, [32,64) up rows 0..31, [64,96) gate 32..63, [96,128) up
// 32..63 -- so that the two accumulator tiles of a wave are gate and up of the SAME 32 rows and the epilogue
// writes bf16( silu(gate) * up ) straight from registers: the reference's silu_mul_bf16 kernel
// (engine/kernels.hip:447-459) and the fp32 round trip of both projections folded away.
// bt: batch tile.  Returns false when the tile lies past the segment's rows (nothing was done).
template <int WB, int WM, int FB, int FM, bool SWI = false>
__device__ __forceinline__ bool gemm_mfma_body(const GemmParams& p, const int bt)
{
    static_assert(!SWI || FM == 2, "the SwiGLU epilogue pairs the two row tiles of a wave");
    constexpr int TB = WB * FB * 32;                  // batch rows per workgroup
    constexpr int NT = WB * WM * 64;                  // threads per workgroup
    static_assert(NT == 512, "eight waves per workgroup");
    static_assert(WM * FM * 32 == TM, "row tile is 128");
    constexpr int ACT_UNITS = TB * 8;                 // 16-byte units per stage
    constexpr int ACT_LD = ACT_UNITS / NT;            // per thread
    constexpr int W_LD = TM * 4 / NT;                 // 16-column weight pieces per thread and stage
    static_assert(ACT_LD >= 1 && ACT_LD * NT == ACT_UNITS, "activation tile divides over the threads");
    constexpr int STAGE_BYTES = ACT_UNITS * 16 + TM * 128;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wb = wave / WM, wm = wave % WM;
    const int ln = lane & 31, lh = lane >> 5;

    const int tile = blockIdx.x;
    const int pair = SWI ? find_pair(p, tile) : 0;
    const int s = SWI ? 2 * pair : find_segment(p, tile);          // SWI: the gate segment of the tile's pair
    const T12Segment& sg = p.seg[s];
    const int M = sg.M, K = p.K;
    const int B = p.dev_counts ? p.dev_counts[p.group_of_seg[s]] : p.seg_B[s];
    const int row_base = p.dev_base ? p.dev_base[p.group_of_seg[s]] : 0;     // first row of this group in act / out
    const int act_stride = p.seg_act_stride[s];
    const uint16_t* const act = p.seg_act[s] + (size_t)row_base * act_stride;
    if (bt * (WB * FB * 32) >= B) return false;            // grouped launch: this segment has fewer batch tiles than the grid
    const int m0 = SWI ? (tile - p.blk_start[pair]) * (TM / 2) : (tile - p.blk_start[s]) * TM;
    // local row r of the tile -> segment and matrix row
    auto row_seg = [&](int r) { return SWI ? s + ((r >> 5) & 1) : s; };
    auto row_mat = [&](int r) { return SWI ? m0 + ((r >> 6) << 5) + (r & 31) : m0 + r; };
    const int b0 = bt * TB;
    const int k_begin = blockIdx.z * p.kslice;
    const int k_end = min(K, k_begin + p.kslice);
    const int nstage = (k_end - k_begin) / KC;
    uint32_t be2s[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int be = p.seg[SWI ? s + j : s].base_exp;
        be2s[j] = t12_opaque(((uint32_t)be << 7) | ((uint32_t)be << 23));
    }

    // ---- this thread's share of the global -> LDS staging
    //  acts: item idx = tid + NT*i -> batch row idx / 8, unit idx % 8 (8 lanes = 128 contiguous bytes)
    // rows past the end are clamped: their products are computed and never stored
    const uint16_t* a_src[ACT_LD];
    int a_dst[ACT_LD];
#pragma unroll
    for (int i = 0; i < ACT_LD; i++) {
        const int idx = tid + NT * i;
        const int r = idx >> 3, u = idx & 7;
        a_src[i] = act + (size_t)min(b0 + r, B - 1) * act_stride + k_begin + u * 8;
        a_dst[i] = lds_slot(u, r, TB) * 16;
    }
    //  weights: pieces X / Y of item i (see above); [0] = X, [1] = Y
    const int c8 = tid & 7, hi = c8 >> 2, cc = c8 & 3;
    const uint8_t* s_src[2][W_LD];
    const uint8_t* g_src[2][W_LD];
    int w_row[2][W_LD];
    int w_dst[2][W_LD][2];
    uint32_t w_be2[2][W_LD];
#pragma unroll
    for (int i = 0; i < W_LD; i++) {
        const int rr = (tid + NT * i) >> 3;                   // 0..63
        const int r_lo = rr, r_hi = 64 + (rr ^ 1);
#pragma unroll
        for (int y = 0; y < 2; y++) {
            const int r = (hi ^ y) ? r_hi : r_lo;
            const T12Segment& g = p.seg[row_seg(r)];
            const size_t e = (size_t)min(row_mat(r), M - 1) * K + k_begin + 64 * y + 16 * cc;
            w_row[y][i] = r;
            w_be2[y][i] = be2s[SWI ? (r >> 5) & 1 : 0];
            s_src[y][i] = g.sm + e;
            g_src[y][i] = g.gr + (e >> 1);
            w_dst[y][i][0] = ACT_UNITS * 16 + lds_slot(2 * cc, r, TM) * 16;
            w_dst[y][i][1] = ACT_UNITS * 16 + lds_slot(2 * cc + 1, r, TM) * 16;
        }
    }

    // Register rings.  Activations: 4 slots, stage s + 4 is requested while stage s is
    // multiplied.  Weights: 2 window slots, window w + 2 is requested during the odd stage of
    // window w, when both of the slot's pieces have been decoded.  A stage is decoded and moved
    // registers -> LDS one iteration before it is consumed (double-buffered LDS).
    constexpr int DA = 4;
    uint4 ra[DA][ACT_LD];
    uint4 rs[2][2][W_LD];      // [window slot][X / Y][item]
    uint2 rg[2][2][W_LD];
    // The staging work of a thread is cut into units so that it can be spread between the
    // MFMAs of a stage.  Load units: ACT_LD activation pieces, then (odd stages) 4 per item:
    // sm X, sm Y, gr X, gr Y.  Store units: ACT_LD activation pieces, 2 decode units per item.
    auto load_act = [&](int slot, int stg, int u) { ra[slot][u] = *(const uint4*)(a_src[u] + (size_t)stg * KC); };
    auto load_w = [&](int slot, int win, int u, bool do_x, bool do_y) {
        const int i = u >> 2, y = u & 1;
        if (y == 0 ? !do_x : !do_y) return;
        if ((u & 2) == 0) rs[slot][y][i] = *(const uint4*)(s_src[y][i] + (size_t)win * (2 * KC));
        else rg[slot][y][i] = *(const uint2*)(g_src[y][i] + (size_t)win * KC);
    };
    auto store_unit = [&](int aslot, int wslot, int y, int buf, int u) {
        uint8_t* base_ = lds + buf * STAGE_BYTES;
        if (u < ACT_LD) {
            *(uint4*)(base_ + a_dst[u]) = t12_pair_acts(ra[aslot][u]);
        } else {
            const int i = (u - ACT_LD) >> 1, h = (u - ACT_LD) & 1;
            const uint4 sv = rs[wslot][y][i];
            const uint2 gv = rg[wslot][y][i];
            uint32_t w_[4];
            if (h == 0) t12_decode8(sv.x, sv.y, gv.x, w_be2[y][i], w_);
            else t12_decode8(sv.z, sv.w, gv.y, w_be2[y][i], w_);
            *(uint4*)(base_ + w_dst[y][i][h]) = make_uint4(w_[0], w_[1], w_[2], w_[3]);
        }
    };

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
    int* lrow = (int*)(lpat + PCAP);                           // [TM + 1] offsets into lpat (SWI: [2][TM/2 + 1])
    int esc_mode = 0;
    if (SWI) {
        // two slices: the 64 gate rows, then the 64 up rows
        const T12Segment& g0 = p.seg[s];
        const T12Segment& g1 = p.seg[s + 1];
        const int r_lo = min(m0, M), r_hi = min(m0 + TM / 2, M);
        const int e00 = g0.row_off ? g0.row_off[r_lo] : 0, e10 = g1.row_off ? g1.row_off[r_lo] : 0;
        const int n0 = g0.row_off ? g0.row_off[r_hi] - e00 : 0, n1 = g1.row_off ? g1.row_off[r_hi] - e10 : 0;
        if (g0.row_off || g1.row_off) esc_mode = (n0 + n1 <= PCAP && K <= 65536) ? 1 : 2;
        if (esc_mode == 1) {
            for (int t = tid; t < n0; t += NT)
                lpat[t] = (uint32_t)g0.cols[e00 + t] | ((uint32_t)(uint16_t)g0.correct[e00 + t] << 16);
            for (int t = tid; t < n1; t += NT)
                lpat[n0 + t] = (uint32_t)g1.cols[e10 + t] | ((uint32_t)(uint16_t)g1.correct[e10 + t] << 16);
            for (int t = tid; t <= TM / 2; t += NT) {
                lrow[t] = g0.row_off ? g0.row_off[min(m0 + t, M)] - e00 : 0;
                lrow[TM / 2 + 1 + t] = n0 + (g1.row_off ? g1.row_off[min(m0 + t, M)] - e10 : 0);
            }
        }
    } else if (sg.row_off) {
        const int e0 = sg.row_off[min(m0, M)], e1 = sg.row_off[min(m0 + TM, M)];
        esc_mode = (e1 - e0 <= PCAP && K <= 65536) ? 1 : 2;
        if (esc_mode == 1) {
            for (int t = tid; t < e1 - e0; t += NT)
                lpat[t] = (uint32_t)sg.cols[e0 + t] | ((uint32_t)(uint16_t)sg.correct[e0 + t] << 16);
            for (int t = tid; t <= TM; t += NT) lrow[t] = sg.row_off[min(m0 + t, M)] - e0;
        }
    }
    // Per piece kind and item: cursor into its row's slice and the column of the next entry.  The
    // thread that decoded 16 columns of a row into LDS also overwrites the escapes among them
    // there (same wave, LDS executes its writes in order: no barrier needed in between).  A
    // thread owns its X row in even stages and its Y row in odd ones; entries of the stages in
    // between are stepped over.
    int pp[2][W_LD], pe[2][W_LD], nc[2][W_LD];
#pragma unroll
    for (int y = 0; y < 2; y++)
#pragma unroll
        for (int i = 0; i < W_LD; i++) { pp[y][i] = pe[y][i] = 0; nc[y][i] = NO_ESCAPE; }
    auto patch_stage = [&](int y, int buf, int kabs) {
        if (esc_mode != 1) return;
        uint8_t* base_ = lds + buf * STAGE_BYTES + ACT_UNITS * 16;
#pragma unroll
        for (int i = 0; i < W_LD; i++) {
            while (nc[y][i] < kabs + KC) {
                const int e = nc[y][i] - kabs - 16 * cc;            // 0..15: one of this piece's
                if ((unsigned)e < 16u) {
                    const int off = lds_slot(2 * cc + (e >> 3), w_row[y][i], TM) * 16 + (e & 3) * 4 + ((e >> 2) & 1) * 2;
                    *(uint16_t*)(base_ + off) = (uint16_t)(lpat[pp[y][i]] >> 16);
                }
                pp[y][i]++;
                nc[y][i] = pp[y][i] < pe[y][i] ? (int)(lpat[pp[y][i]] & 0xFFFFu) : NO_ESCAPE;
            }
        }
    };

    // One stage = 64 columns = 4 MFMA k-steps; the fragments of k-step t + 1 are read from LDS
    // at the start of k-step t.  The staging work for later stages is placed between the MFMAs,
    // a unit after every few of them, and pinned there with scheduling barriers: whatever is
    // not issued under a running MFMA is serial time for the wave.
    //   d = stage number modulo 4 (selects ring slots and LDS buffers at compile time)
    constexpr int NMMA = 4 * FB * FM;
    constexpr int NSU = ACT_LD + 2 * W_LD;               // store units per stage
    constexpr int NLU_ODD = ACT_LD + 4 * W_LD;           // load units of an odd stage
    constexpr int NCH = NMMA >= 2 * NSU ? NSU : NMMA;    // chunks of staging work per stage
    auto run_stage = [&](int d, int stg, bool ld_act, bool ld_x, bool ld_y, bool do_store) {
        const int buf = d & 1;
        const bool odd = d & 1;
        const int nlu = odd ? NLU_ODD : ACT_LD;
        // stage stg + 1: activation slot, weight window slot, piece kind
        const int n_aslot = (d + 1) & 3, n_wslot = ((d + 1) >> 1) & 1, n_y = (d + 1) & 1, n_buf = (d + 1) & 1;
        // requests: activations of stage stg + 4 -> slot d; weights of window stg / 2 + 2 -> slot (d >> 1) & 1
        const int l_wslot = (d >> 1) & 1, l_win = (stg >> 1) + 2;
        const uint8_t* base = lds + buf * STAGE_BYTES;
        const uint4* lact = (const uint4*)base;
        const uint4* lw = (const uint4*)(base + ACT_UNITS * 16);
        uint4 A[2][FB], W[2][FM];
        auto load_frags = [&](int t) {
#pragma unroll
            for (int i = 0; i < FB; i++) A[t & 1][i] = lact[lds_slot(2 * t + lh, (wb * FB + i) * 32 + ln, TB)];
#pragma unroll
            for (int j = 0; j < FM; j++) W[t & 1][j] = lw[lds_slot(2 * t + lh, (wm * FM + j) * 32 + ln, TM)];
        };
        load_frags(0);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if (t < 3) load_frags(t + 1);
#pragma unroll
            for (int i = 0; i < FB; i++) {
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(t12_bf16x8, A[t & 1][i]), __builtin_bit_cast(t12_bf16x8, W[t & 1][j]),
                        acc[i][j], 0, 0, 0);
                    const int m = (t * FB + i) * FM + j;
                    // chunk c of the staging work goes after MFMA number (c + 1) * NMMA / NCH - 1
#pragma unroll
                    for (int c = 0; c < NCH; c++) {
                        if ((c + 1) * NMMA / NCH - 1 == m) {
#pragma unroll
                            for (int u = 0; u < NLU_ODD; u++) {
                                if (u < nlu && u * NCH / nlu == c) {
                                    if (u < ACT_LD) {
                                        if (ld_act) load_act(d, stg + DA, u);
                                    } else {
                                        load_w(l_wslot, l_win, u - ACT_LD, ld_x, ld_y);
                                    }
                                }
                            }
#pragma unroll
                            for (int u = 0; u < NSU; u++)
                                if (do_store && u * NCH / NSU == c)
                                    store_unit(n_aslot, n_wslot, n_y, n_buf, stage_unit_order(u, ACT_LD, 2 * W_LD));
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
        }
        if (do_store) patch_stage(n_y, n_buf, k_begin + (stg + 1) * KC);
        __syncthreads();
    };

    // prologue: activation stages 0..3 and weight windows 0, 1 in flight, escape list visible,
    // stage 0 into LDS
#pragma unroll
    for (int d = 0; d < DA; d++)
        if (d < nstage) {
#pragma unroll
            for (int u = 0; u < ACT_LD; u++) load_act(d, d, u);
        }
#pragma unroll
    for (int w = 0; w < 2; w++)
#pragma unroll
        for (int u = 0; u < 4 * W_LD; u++) load_w(w, w, u, 2 * w < nstage, 2 * w + 1 < nstage);
    __syncthreads();
    if (esc_mode == 1) {
#pragma unroll
        for (int y = 0; y < 2; y++)
#pragma unroll
            for (int i = 0; i < W_LD; i++) {
                const int r = w_row[y][i];
                const int li = SWI ? ((r >> 5) & 1) * (TM / 2 + 1) + ((r >> 6) << 5) + (r & 31) : r;
                int q = lrow[li];
                const int qe = lrow[li + 1];
                while (q < qe && (int)(lpat[q] & 0xFFFFu) < k_begin) q++;   // K split: skip earlier columns
                pp[y][i] = q;
                pe[y][i] = qe;
                if (q < qe) nc[y][i] = (int)(lpat[q] & 0xFFFFu);
            }
    }
    // All prologue loads have landed before the loop is entered: the compiler's wait-count
    // bookkeeping then sees only the loop's own loads at the loop head and waits for exactly
    // the ring slot it needs (with loads pending across the entry edge it drains all of them
    // once per trip).
    __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
    if (nstage > 0) {
#pragma unroll
        for (int u = 0; u < NSU; u++) store_unit(0, 0, 0, 0, u);
        patch_stage(0, 0, k_begin);
    }
    __syncthreads();

    int st = 0;
    // steady state, unrolled by 4 so that ring slots and buffers are compile-time; no guards inside
    for (; st + 2 * DA <= nstage; st += DA) {
#pragma unroll
        for (int d = 0; d < DA; d++) run_stage(d, st + d, true, true, true, true);
    }
    // drain
    for (; st < nstage; st += DA) {
#pragma unroll
        for (int d = 0; d < DA; d++) {
            const int sn = st + d;
            if (sn < nstage)
                run_stage(d, sn, sn + DA < nstage, 2 * ((sn >> 1) + 2) < nstage, 2 * ((sn >> 1) + 2) + 1 < nstage,
                          sn + 1 < nstage);
        }
    }

    // ---- overflow path only (more escapes than the LDS list holds): the streamed value of an
    //      escape was its "wrong" decode, so acc[b, m] += (correct - wrong) * X[b, col], added by
    //      the K split that owns column 0
    if (blockIdx.z == 0 && esc_mode == 2) {
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const T12Segment& g = p.seg[SWI ? s + j : s];
            const int m = SWI ? m0 + wm * 32 + ln : m0 + (wm * FM + j) * 32 + ln;
            if (m < M && g.row_off) {
                const int beg = g.row_off[m], end = g.row_off[m + 1];
                for (int pp = beg; pp < end; pp++) {
                    const float delta = t12_bf16_to_f32((uint16_t)g.correct[pp]) -
                                        t12_bf16_to_f32((uint16_t)g.wrong[pp]);
                    const uint16_t* xc = act + g.cols[pp];
#pragma unroll
                    for (int i = 0; i < FB; i++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int bb = b0 + (wb * FB + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                            if (bb < B) acc[i][j][r] += delta * t12_bf16_to_f32(xc[(size_t)bb * act_stride]);
                        }
                }
            }
        }
    }

    // ---- store: accumulator register r of lane (ln, lh) is
    //      D[row = 8*(r/4) + 4*lh + r%4][col = ln]   (row = batch, col = m)
    if (SWI) {
        const int m = m0 + wm * 32 + ln;
        uint16_t* const ob = p.out_bf16 + (size_t)row_base * p.out_bf16_ld;
#pragma unroll
        for (int i = 0; i < FB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int b = b0 + (wb * FB + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                const float g = acc[i][0][r];
                if (m < M && b < B)
                    ob[(size_t)b * p.out_bf16_ld + m] = t12_f32_to_bf16(g / (1.0f + expf(-g)) * acc[i][FM - 1][r]);
            }
        return true;
    }
    float* dst;
    size_t ld;
    if (p.ksplit > 1) {
        dst = p.ws + (size_t)blockIdx.z * p.split_stride + p.seg_ws0[s];
        ld = p.seg_ld[s];
    } else {
        dst = sg.out + (size_t)row_base * sg.out_stride;
        ld = sg.out_stride;
    }
#pragma unroll
    for (int i = 0; i < FB; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int m = m0 + (wm * FM + j) * 32 + ln;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int b = b0 + (wb * FB + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (m < M && b < B) dst[(size_t)b * ld + m] = acc[i][j][r];
            }
        }
    return true;
}

// Eight waves per workgroup, two per SIMD: one wave's decode / LDS traffic runs under the other's MFMAs.
// Batch tiles: one per workgroup (blockIdx.y), except when the rows per group are known on the device only: such
// a launch has one workgroup per row tile, which takes the group's batch tiles one after the other (a group within
// the tile -- the usual case -- is streamed once, a larger one once per tile; no group's rows can fall outside the grid).
template <int WB, int WM, int FB, int FM, bool SWI = false>
__global__ __launch_bounds__(WB * WM * 64) void gemm_mfma_kernel(const GemmParams p)
{
    for (int bt = blockIdx.y;; bt++) {
        if (!gemm_mfma_body<WB, WM, FB, FM, SWI>(p, bt) || !p.dev_counts) break;
        __syncthreads();                                   // the next tile reuses the staging buffers
    }
}

// ---------------------------------------------------------------------------
// K-split reduction: out[b, m] = sum over splits z of the partial sums of (b, m), in ascending z
// (a fixed order: the result does not depend on which workgroup finished first).
// Grid: (blocks of 256 rows of the launch, largest batch).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmParams p)
{
    const int col = blockIdx.x * 256 + threadIdx.x;
    const int b = blockIdx.y;
    if (col >= p.m_total) return;
    int s = 0;
#pragma unroll
    for (int i = 1; i < GMAX; i++)
        if (i < p.nseg && col >= p.seg_row0[i]) s = i;
    if (b >= p.seg_B[s]) return;
    const int m = col - p.seg_row0[s];
    const float* src = p.ws + p.seg_ws0[s] + (size_t)b * p.seg_ld[s] + m;
    float v = 0.0f;
    for (int z = 0; z < p.ksplit; z++) v += src[(size_t)z * p.split_stride];
    const T12Segment& sg = p.seg[s];
    sg.out[(size_t)b * sg.out_stride + m] = v;
}

// The same sums four rows at a time (16-byte loads and stores): thread = rows 4 c .. 4 c + 3 of one batch row.
// Used when every segment's row count, first row, output stride and pointers are multiples of four floats.
__global__ __launch_bounds__(256) void gemm_reduce4_kernel(const GemmParams p)
{
    const int col = (blockIdx.x * 256 + threadIdx.x) * 4;
    const int b = blockIdx.y;
    if (col >= p.m_total) return;
    int s = 0;
#pragma unroll
    for (int i = 1; i < GMAX; i++)
        if (i < p.nseg && col >= p.seg_row0[i]) s = i;
    if (b >= p.seg_B[s]) return;
    const int m = col - p.seg_row0[s];
    const float* src = p.ws + p.seg_ws0[s] + (size_t)b * p.seg_ld[s] + m;
    t12_f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int z = 0; z < p.ksplit; z++) v += *(const t12_f32x4*)(src + (size_t)z * p.split_stride);
    const T12Segment& sg = p.seg[s];
    *(t12_f32x4*)(sg.out + (size_t)b * sg.out_stride + m) = v;
}

// Adds up the partial sums of a K-split launch described by p into the segments' outputs.
void launch_reduce(const GemmParams& p, int max_b, hipStream_t st)
{
    bool vec = p.split_stride % 4 == 0 && (uintptr_t)p.ws % 16 == 0;
    for (int i = 0; i < p.nseg; i++) {
        const T12Segment& g = p.seg[i];
        if (g.M % 4 || p.seg_row0[i] % 4 || p.seg_ws0[i] % 4 || p.seg_ld[i] % 4 || g.out_stride % 4 || (uintptr_t)g.out % 16) vec = false;
    }
    if (vec)
        hipLaunchKernelGGL(gemm_reduce4_kernel, dim3((p.m_total / 4 + 255) / 256, max_b), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(gemm_reduce_kernel, dim3((p.m_total + 255) / 256, max_b), dim3(256), 0, st, p);
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

// ---------------------------------------------------------------------------
// Small batches (B <= 16): the dense-sweep kernel.  At these sizes the product is bound by the weight stream, and
// what the memory system streams fastest is what the B = 1 kernel gives it: workgroups in launch order, each
// sweeping a few whole rows quickly, so that the chip as a whole reads one dense window of the planes.  (Kernels
// whose waves walk many rows slowly in parallel -- a K-split grid of 128-row tiles, a wave per 16 rows -- measure
// 3.5-4.5 TB/s on the same bytes.)
//   * a workgroup owns 16 consecutive weight rows and all of K; its NW waves take the 128-column blocks of the rows
//     in turn (wave w: blocks w, w + NW, ...), so the workgroup as a whole reads its rows' planes front to back;
//   * v_mfma_f32_16x16x32_bf16, activations = A operand (rows = batch), weights = B operand: lane (n, g) =
//     (lane % 16, lane / 16) holds row n, so the planes go straight from HBM into the operand registers -- per
//     block a lane loads 2 x 16 bytes of sign/mantissa (columns 32g .. 32g+15 and 32g+16 .. 32g+31: the four lanes
//     of a row cover its 128-byte line in two back-to-back instructions) and 16 bytes of nibbles, rebuilds them
//     with t12_decode8 and feeds four MFMAs;
//   * the activations are not staged: lane (b, g) reads the 8 columns an MFMA needs straight from memory (they are
//     B x K bf16, resident in L2) and pairs them in registers to match t12_decode8's order;
//   * no barrier until the end, where the waves' partial 16 x 16 tiles are added through LDS in wave order;
//   * escapes: the streamed value of a group-0 weight is its "wrong" value; wave w adds (correct - wrong) * x[b, col]
//     for the entries w, w + NW, ... of each row (the four lanes of a row each for their four batch rows).
// Requires K % 128 == 0, 0 <= base_exp <= 240, B <= 16 NBT (NBT batch tiles of 16 rows share every weight load and
// decode; accumulators, activation registers and the reduction buffer grow with NBT).  blk_start counts the workgroups
// (16 RG rows each) per segment.
// Rows per group known on the device only (dev_counts, the experts of a mixture-of-experts layer at a few tokens):
// the segment's group has dev_counts[g] batch rows starting dev_base[g] rows into the activations and the outputs; a
// workgroup of a group without rows exits at once, one of a group above 16 rows sweeps its weight rows once per 16.
// ---------------------------------------------------------------------------
// SWI (a launch of ONE gate / up pair, segments 0 and 1 of equal row count): the first RG / 2 row groups of a workgroup
// are 16 RG / 2 rows of gate, the others the same rows of up, and the thread that finishes an element of both stores
// bf16( silu(gate) * up ) to out_bf16 instead of the two sums (the arithmetic of silu_mul_kernel, so the result is
// what t12_gemm + launch_silu_mul_bf16_batch give, bit for bit).
template <int NW, int D, int RG, bool DEV, int NBT = 1, bool SWI = false>
__device__ __forceinline__ void gemm_dense16_body(const GemmParams& p, t12_f32x4 (*red)[NW][64])
{
    static_assert(!SWI || (RG % 2 == 0 && !DEV && NBT == 1), "the SwiGLU form pairs row groups");
    constexpr int RH = SWI ? RG / 2 : RG;             // row groups of one tensor
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;

    const int blk = blockIdx.x;
    const int s = SWI ? 0 : find_segment(p, blk);
    const T12Segment& sg = p.seg[s];
    const int M = sg.M, K = p.K;
    // DEV: the group's rows from the device tables; otherwise one pass over the launch's B <= 16 rows
    const int b_all = DEV ? p.dev_counts[p.group_of_seg[s]] : 1;
    const int row_base = DEV ? p.dev_base[p.group_of_seg[s]] : 0;
    for (int b_first = 0; b_first < b_all; b_first += 16 * NBT) {
    const int B = DEV ? min(16 * NBT, b_all - b_first) : p.B;
    const uint16_t* const act = DEV ? p.act + (size_t)(row_base + b_first) * p.act_stride : p.act;
    float* const outp = DEV ? sg.out + (size_t)(row_base + b_first) * sg.out_stride : sg.out;
    const int m0 = (blk - p.blk_start[s]) * (16 * RH);               // RG groups of 16 rows share every activation load
    const int nblk = K >> 7;                          // 128-column blocks per row
    const int mine = nblk > wave ? (nblk - wave + NW - 1) / NW : 0;      // blocks of this wave
    // A wave without a block (K < NW * 128) still issues the first D fetches below and drops them: it aims them at
    // block 0, because its own first block would lie past the end of the row -- and, in the last rows of a plane or
    // of the activations, past the end of the allocation.
    const int wblk = mine > 0 ? wave : 0;
    uint32_t be2r[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        const int be = p.seg[SWI && rg >= RH ? 1 : s].base_exp;
        be2r[rg] = t12_opaque(((uint32_t)be << 7) | ((uint32_t)be << 23));
    }

    // CSR pointers of this lane's rows (used after the stream)
    int e_beg[RG], e_end[RG];
    const uint8_t* smp[RG];
    const uint8_t* grp[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        const T12Segment& sr = p.seg[SWI && rg >= RH ? 1 : s];      // (SWI: gate for the first half, up for the second)
        const int row = m0 + 16 * (rg % RH) + n;
        e_beg[rg] = e_end[rg] = 0;
        if (sr.row_off && row < M) {
            e_beg[rg] = sr.row_off[row];
            e_end[rg] = sr.row_off[row + 1];
        }
        const size_t e0 = (size_t)min(row, M - 1) * K;              // rows past the end are clamped, never stored
        smp[rg] = sr.sm + e0 + 32 * g + (size_t)wblk * 128;
        grp[rg] = sr.gr + (e0 >> 1) + 16 * g + (size_t)wblk * 64;
    }
    const uint16_t* xp[NBT];                          // NBT tiles of 16 batch rows share every weight load and decode
#pragma unroll
    for (int t = 0; t < NBT; t++) xp[t] = act + (size_t)min(16 * t + n, B - 1) * p.act_stride + 32 * g + (size_t)wblk * 128;
    uint4 rS[D][RG][2], rG[D][RG], rX[D][NBT][4];
#define T12_DS_FETCH(slot, j)                                                              \
    {                                                                                      \
        _Pragma("unroll") for (int t = 0; t < NBT; t++)                                    \
            _Pragma("unroll") for (int q = 0; q < 4; q++)                                  \
                rX[slot][t][q] = *(const uint4*)(xp[t] + (size_t)(j) * (NW * 128) + 8 * q); \
        _Pragma("unroll") for (int rg = 0; rg < RG; rg++) {                                \
            rS[slot][rg][0] = *(const uint4*)(smp[rg] + (size_t)(j) * (NW * 128));         \
            rS[slot][rg][1] = *(const uint4*)(smp[rg] + (size_t)(j) * (NW * 128) + 16);    \
            rG[slot][rg] = *(const uint4*)(grp[rg] + (size_t)(j) * (NW * 64));             \
        }                                                                                  \
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        T12_DS_FETCH(d, min(d, max(mine - 1, 0)))     // (fewer blocks than slots: the last one again, in bounds)
        __builtin_amdgcn_sched_barrier(0);
    }

    // the first escape entries of the rows: wave w takes entry e_beg + w, requested now and used after the stream
    int pcol[RG], pcorrect[RG], pwrong[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        pcol[rg] = -1;
        pcorrect[rg] = pwrong[rg] = 0;
        if (e_beg[rg] + wave < e_end[rg]) {
            const T12Segment& sr = p.seg[SWI && rg >= RH ? 1 : s];
            pcol[rg] = sr.cols[e_beg[rg] + wave];
            pcorrect[rg] = sr.correct[e_beg[rg] + wave];
            pwrong[rg] = sr.wrong[e_beg[rg] + wave];
        }
    }

    t12_f32x4 acc[NBT][RG];
#pragma unroll
    for (int t = 0; t < NBT; t++)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) acc[t][rg] = t12_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#define T12_DS_CONSUME(slot)                                                                                 \
    _Pragma("unroll") for (int q = 0; q < 4; q++) {                                                          \
        uint4 xa[NBT];                                                                                       \
        _Pragma("unroll") for (int t = 0; t < NBT; t++) xa[t] = t12_pair_acts(rX[slot][t][q]);               \
        _Pragma("unroll") for (int rg = 0; rg < RG; rg++) {                                                  \
            const uint4 sv = rS[slot][rg][q >> 1];                                                           \
            const uint32_t gq = q == 0 ? rG[slot][rg].x : (q == 1 ? rG[slot][rg].y : (q == 2 ? rG[slot][rg].z : rG[slot][rg].w)); \
            uint32_t w_[4];                                                                                  \
            if (q & 1) t12_decode8(sv.z, sv.w, gq, be2r[rg], w_);                                            \
            else t12_decode8(sv.x, sv.y, gq, be2r[rg], w_);                                                  \
            const uint4 wv = make_uint4(w_[0], w_[1], w_[2], w_[3]);                                         \
            _Pragma("unroll") for (int t = 0; t < NBT; t++)                                                  \
                acc[t][rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(t12_bf16x8, xa[t]),  \
                                                                     __builtin_bit_cast(t12_bf16x8, wv), acc[t][rg], 0, 0, 0); \
        }                                                                                                    \
    }
    int j = 0;
    for (; j + 2 * D <= mine; j += D) {               // every slot is refilled
#pragma unroll
        for (int d = 0; d < D; d++) {
            T12_DS_CONSUME(d)
            T12_DS_FETCH(d, j + d + D)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (; j < mine; j += D) {                        // the last (up to 2D - 1) blocks
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (j + d < mine) {
                T12_DS_CONSUME(d)
                if (j + d + D < mine) T12_DS_FETCH(d, j + d + D)
            }
        }
    }
#undef T12_DS_FETCH
#undef T12_DS_CONSUME

    // ---- escapes.  Accumulator register r of lane (n, g) in batch tile t is D[batch 16t + 4g + r][row n].
    {
        const uint16_t* xrow[NBT][4];
#pragma unroll
        for (int t = 0; t < NBT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) xrow[t][r] = act + (size_t)min(16 * t + 4 * g + r, B - 1) * p.act_stride;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            if (pcol[rg] >= 0) {
                const float delta = t12_bf16_to_f32((uint16_t)pcorrect[rg]) - t12_bf16_to_f32((uint16_t)pwrong[rg]);
#pragma unroll
                for (int t = 0; t < NBT; t++)
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[t][rg][r] += delta * t12_bf16_to_f32(xrow[t][r][pcol[rg]]);
            }
            const T12Segment& sr = p.seg[SWI && rg >= RH ? 1 : s];
            for (int e = e_beg[rg] + wave + NW; e < e_end[rg]; e += NW) {        // rows with more than NW escapes
                const int col = sr.cols[e];
                const float delta = t12_bf16_to_f32((uint16_t)sr.correct[e]) - t12_bf16_to_f32((uint16_t)sr.wrong[e]);
#pragma unroll
                for (int t = 0; t < NBT; t++)
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[t][rg][r] += delta * t12_bf16_to_f32(xrow[t][r][col]);
            }
        }
    }

    // ---- the waves' partial tiles, added in wave order; thread (r, l) = (tid / 64, tid % 64) of the first four waves
    //      finishes element D[batch 16 t + 4 (l / 16) + r][row l % 16] of every batch tile and row group
#pragma unroll
    for (int t = 0; t < NBT; t++)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) red[t * RG + rg][wave][lane] = acc[t][rg];
    __syncthreads();
    if (tid < 256) {
        const int r = tid >> 6, l = tid & 63;
#pragma unroll
        for (int t = 0; t < NBT; t++)
#pragma unroll
            for (int rg = 0; rg < RH; rg++) {
                float v = 0.0f, u = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; w++) v += red[t * RG + rg][w][l][r];
                if (SWI) {
#pragma unroll
                    for (int w = 0; w < NW; w++) u += red[RH + rg][w][l][r];
                }
                const int b = 16 * t + 4 * (l >> 4) + r, row = m0 + 16 * rg + (l & 15);
                if (SWI) {
                    if (b < B && row < M)
                        p.out_bf16[(size_t)b * p.out_bf16_ld + row] = t12_f32_to_bf16(v / (1.0f + expf(-v)) * u);
                } else if (b < B && row < M) outp[(size_t)b * sg.out_stride + row] = v;
            }
    }
    if (DEV && b_first + 16 * NBT < b_all) __syncthreads();  // the next batch rows reuse the reduction buffer
    }
}

template <int NW, int D, int RG, bool DEV = false, int NBT = 1>
__global__ __launch_bounds__(NW * 64) void gemm_dense16_kernel(const GemmParams p)
{
    __shared__ t12_f32x4 red[NBT * RG][NW][64];
    gemm_dense16_body<NW, D, RG, DEV, NBT>(p, red);
}

// The sweep over one gate / up pair with the SiLU * mul in its last step (blockIdx.x counts sets of 16 RG / 2 rows).
template <int NW, int D, int RG>
__global__ __launch_bounds__(NW * 64) void gemm_dense16_swiglu_kernel(const GemmParams p)
{
    __shared__ t12_f32x4 red[RG][NW][64];
    gemm_dense16_body<NW, D, RG, false, 1, true>(p, red);
}

// The same sweep with two sizes of workgroup in one launch.  With RGA row groups per workgroup (its registers allow one
// workgroup per CU) a launch is a sequence of rounds of one workgroup per CU, each as long as a workgroup lives, and a
// last round that fills a fraction of the chip costs as much as a full one (gate|up at B = 16: 448 workgroups = 256 +
// 192, two rounds of 23 us).  The host therefore cuts every tensor in two: the first n_first segments of the launch
// are the heads of the tensors, swept RGA groups per workgroup in whole rounds, the others their tails, swept RGB < RGA
// groups per workgroup so that the last round covers the chip once with shorter workgroups.
template <int NW, int D, int RGA, int RGB>
__global__ __launch_bounds__(NW * 64) void gemm_dense16_mixed_kernel(const GemmParams p)
{
    __shared__ t12_f32x4 red[RGA][NW][64];
    if (find_segment(p, blockIdx.x) < p.n_first) gemm_dense16_body<NW, D, RGA, false>(p, red);
    else gemm_dense16_body<NW, D, RGB, false>(p, red);
}

// ---------------------------------------------------------------------------
// Two batch rows: the B = 1 kernel's shape with NB accumulators.  A workgroup = 8 waves = 8 consecutive rows;
// a wave reads its whole row front to back in 1024-column tiles (16 bytes of sign/mantissa + 8 bytes of nibbles per
// lane and tile, nontemporal, ring of two tiles) -- the access pattern that streams fastest on this chip -- rebuilds
// 16 weights per tile and multiplies them with the NB activation rows (v_dot2_f32_bf16), which the workgroup staged
// in LDS, paired the way t12_decode8 orders its outputs, laid out per row and 1024-column chunk as [half][lane] x 16 B.
// The decode is shared by the batch rows; per weight the kernel spends 2.25 + NB x 0.5 VALU operations and NB x 2
// bytes of LDS reads: measured with NB = 4 it is level with the MFMA kernel below, which therefore takes over from
// three rows on.  Escapes: (correct - wrong) * x[b, col] after the stream, x from LDS.  Wave sums by DPP.
// Requires K % 1024 == 0, NB * K * 2 bytes of LDS (K <= 8192), 0 <= base_exp <= 240, aligned activation rows.
// blk_start counts 8-row groups per segment.
// ---------------------------------------------------------------------------
template <int NB, int D>
__global__ __launch_bounds__(512) void gemm_rows_kernel(const GemmParams p)
{
    extern __shared__ uint4 lds_x[];                   // [NB][T * 128]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = p.K, B = p.B;
    const int T = K >> 10;
    const int blk = blockIdx.x;
    const int s = find_segment(p, blk);
    const T12Segment& sg = p.seg[s];
    const int M = sg.M;
    const int row = (blk - p.blk_start[s]) * 8 + wave;
    const bool live = row < M;                         // wave-uniform
    const uint32_t be2 = t12_opaque(((uint32_t)sg.base_exp << 7) | ((uint32_t)sg.base_exp << 23));

    // activations first (they come out of L2 and must not queue behind the weight tiles): piece = 8 columns,
    // NB * K / 8 pieces over 512 threads
    constexpr int XU = NB * 2;                         // pieces per thread at K = 8192
    const int kp = K >> 3;                             // pieces per batch row
    uint4 xpre[XU];
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int idx = tid + 512 * u;
        xpre[u] = make_uint4(0, 0, 0, 0);
        if (idx < NB * kp) {
            const int nb = idx / kp, q = idx - nb * kp;
            xpre[u] = *(const uint4*)(p.act + (size_t)min(nb, B - 1) * p.act_stride + q * 8);   // rows past the batch: clamped, never stored
        }
    }
    int e_beg = 0, e_end = 0;
    if (live && sg.row_off) {
        e_beg = sg.row_off[row];
        e_end = sg.row_off[row + 1];
    }
    const size_t e0 = (size_t)min(row, M - 1) * K;     // rows past the end: clamped, never stored
    const uint8_t* smp = sg.sm + e0 + lane * 16;
    const uint8_t* grp = sg.gr + (e0 >> 1) + lane * 8;
    uint4 rS[D];
    uint2 rG[D];
#pragma unroll
    for (int d = 0; d < D; d++) {
        const int t = min(d, T - 1);
        rS[d] = t12_ldg_stream16(smp + (size_t)t * 1024);
        rG[d] = t12_ldg_stream8(grp + (size_t)t * 512);
    }
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int idx = tid + 512 * u;
        if (idx < NB * kp) {
            const int nb = idx / kp, q = idx - nb * kp;
            lds_x[nb * (T * 128) + (q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1)] = t12_pair_acts(xpre[u]);
        }
    }
    __syncthreads();

    float acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = 0.0f;
    auto consume = [&](int slot, int t) {
        uint32_t w0[4], w1[4];
        t12_decode8(rS[slot].x, rS[slot].y, rG[slot].x, be2, w0);
        t12_decode8(rS[slot].z, rS[slot].w, rG[slot].y, be2, w1);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const uint4 a0 = lds_x[nb * (T * 128) + t * 128 + lane];
            const uint4 a1 = lds_x[nb * (T * 128) + t * 128 + 64 + lane];
            float v = acc[nb];
            v = t12_dot2(w0[0], a0.x, v);
            v = t12_dot2(w0[1], a0.y, v);
            v = t12_dot2(w0[2], a0.z, v);
            v = t12_dot2(w0[3], a0.w, v);
            v = t12_dot2(w1[0], a1.x, v);
            v = t12_dot2(w1[1], a1.y, v);
            v = t12_dot2(w1[2], a1.z, v);
            v = t12_dot2(w1[3], a1.w, v);
            acc[nb] = v;
        }
    };
    for (int t = 0; t < T; t += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (t + d < T) {
                consume(d, t + d);
                if (t + d + D < T) {
                    rS[d] = t12_ldg_stream16(smp + (size_t)(t + d + D) * 1024);
                    rG[d] = t12_ldg_stream8(grp + (size_t)(t + d + D) * 512);
                }
            }
        }
    }
    // escapes: the streamed value of an escaped weight is its "wrong" value
    for (int e = e_beg + lane; e < e_end; e += 64) {
        const int col = sg.cols[e];
        const float delta = t12_bf16_to_f32((uint16_t)sg.correct[e]) - t12_bf16_to_f32((uint16_t)sg.wrong[e]);
        const int q = col >> 3, i = col & 7;
        const int slot = (q >> 7) * 128 + (q & 1) * 64 + ((q & 127) >> 1);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const uint16_t* h = (const uint16_t*)(lds_x + nb * (T * 128) + slot);
            acc[nb] += delta * t12_bf16_to_f32(h[(i & 3) * 2 + (i >> 2)]);
        }
    }
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const float v = t12_wave_sum_lane63(acc[nb]);
        if (lane == 63 && live && nb < B) sg.out[(size_t)nb * sg.out_stride + row] = v;
    }
}

// ---- workspace for the K-split partial sums: one per (device, stream), grown on demand.  Launches on different
//      streams may overlap, so they must not share partial sums; launches on one stream are ordered.
struct Workspace {
    float* ptr = nullptr;
    size_t bytes = 0;
    std::vector<float*> retired;      // outgrown buffers: kernels already in the stream may still write them
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_ws;

float* workspace(size_t bytes, hipStream_t st)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace& w = g_ws[{dev, st}];
    if (w.bytes < bytes) {
        // Grows geometrically, in whole MiB, so a caller whose shapes grow step by step allocates a few times and the
        // outgrown buffers together stay below the live one.  They are kept until release_workspace: hipFree waits
        // for the whole device, which a launch call must not do.
        size_t want = bytes > 2 * w.bytes ? bytes : 2 * w.bytes;
        want = (want + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
        float* fresh = nullptr;
        if (hipMalloc((void**)&fresh, want) != hipSuccess) {
            (void)hipGetLastError();
            // short of memory: give the outgrown buffers back (this waits for the device) and ask for the exact size
            for (float* r : w.retired) (void)hipFree(r);
            w.retired.clear();
            if (w.ptr) (void)hipFree(w.ptr);
            w.ptr = nullptr;
            w.bytes = 0;
            want = bytes;
            if (hipMalloc((void**)&fresh, want) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
        }
        if (w.ptr) w.retired.push_back(w.ptr);
        w.ptr = fresh;
        w.bytes = want;
    }
    return w.ptr;
}

// Frees the K-split workspace of (current device, stream), outgrown buffers included.
void release_workspace(hipStream_t st)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_ws.find({dev, st});
    if (it == g_ws.end()) return;
    for (float* r : it->second.retired) (void)hipFree(r);
    if (it->second.ptr) (void)hipFree(it->second.ptr);
    g_ws.erase(it);
}

// ---- the same workspace for callers that may not allocate: a fixed array in the code object's own device
//      memory.  Every GPU the library runs on holds its own copy at its own address; the name below is only a
//      host-side handle for hipGetSymbolAddress, never a pointer a kernel could use.
constexpr size_t STATIC_WS_BYTES = (size_t)T12_GEMM_NOALLOC_WS_BYTES;
static __device__ __align__(256) float g_static_ws[STATIC_WS_BYTES / sizeof(float)];
std::mutex g_static_ws_mutex;
float* g_static_ws_ptr[16] = {};                       // per device, filled on the first call on that device

float* static_workspace()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_ws_mutex);
    if (!g_static_ws_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_ws)) != hipSuccess || !ptr) return nullptr;
        g_static_ws_ptr[dev] = (float*)ptr;
    }
    return g_static_ws_ptr[dev];
}


template <int WB, int WM, int FB, int FM, bool SWI = false>
int launch_mfma(GemmParams& p, int tiles, hipStream_t st)
{
    constexpr int TB = WB * FB * 32;
    constexpr int STAGE_BYTES = TB * 8 * 16 + TM * 128;
    const dim3 grid(tiles, (p.B + TB - 1) / TB, p.ksplit);   // batch tiles of one row tile are neighbours in time
    auto kfn = gemm_mfma_kernel<WB, WM, FB, FM, SWI>;
    static bool attr_done[16] = {};                    // the attribute is per device
    static std::mutex attr_mutex;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) dev = 0;
    {
        std::lock_guard<std::mutex> attr_lock(attr_mutex);
        bool& attr_set = attr_done[dev];
        if (!attr_set) {
            if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    2 * STAGE_BYTES + PATCH_BYTES) !=
                hipSuccess) {
                t12_set_error("t12_gemm: cannot reserve %d bytes of LDS", 2 * STAGE_BYTES);
                return T12_ELAUNCH;
            }
            attr_set = true;
        }
    }
    hipLaunchKernelGGL(kfn, grid, dim3(WB * WM * 64), 2 * STAGE_BYTES + PATCH_BYTES, st, p);
    T12_CHECK_LAUNCH("t12_gemm");
    return T12_OK;
}


}  // namespace

extern "C" {

int t12_gemm(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K, int B,
             void* stream)
{
    return t12_gemm_deferred(segs, nseg, act_bf16, act_stride, out_stride, K, B, nullptr, stream);
}

// out_bf16[b, m] = bf16( silu(gate[m,:] . X[b,:]) * (up[m,:] . X[b,:]) ): gate|up projection with the SwiGLU
// in the GEMM's epilogue.  Returns T12_OK when launched, 1 when this shape has no fused kernel (the caller
// then runs t12_gemm on the two segments and launch_silu_mul_bf16_batch), negative on bad operands.
int t12_gemm_swiglu(const T12Segment* gate, const T12Segment* up, const void* act_bf16, int act_stride, int K, int B,
                    void* out_bf16, int out_stride, void* stream)
{
    T12_REQUIRE(gate && up && act_bf16 && out_bf16, "t12_gemm_swiglu: null operand");
    T12_REQUIRE(K >= 1 && B >= 1 && act_stride >= K, "t12_gemm_swiglu: K %d, B %d or act_stride %d invalid", K, B, act_stride);
    T12_REQUIRE(gate->M >= 1 && gate->M == up->M, "t12_gemm_swiglu: gate has %d rows, up has %d", gate->M, up->M);
    T12_REQUIRE(out_stride >= gate->M, "t12_gemm_swiglu: out_stride %d < M %d", out_stride, gate->M);
    const T12Segment* two[2] = {gate, up};
    bool fast = (K % KC == 0) && (act_stride % 8 == 0) && ((uintptr_t)act_bf16 % 16 == 0) && B > 64;
    for (const T12Segment* g : two) {
        T12_REQUIRE(g->sm && g->gr, "t12_gemm_swiglu: a plane is null");
        T12_REQUIRE(!g->row_off || (g->cols && g->correct && g->wrong), "t12_gemm_swiglu: row_off without lists");
        T12_REQUIRE(g->base_exp >= -1 && g->base_exp <= 254, "t12_gemm_swiglu: base_exp %d out of range", g->base_exp);
        if (g->base_exp < 0 || g->base_exp > 240) fast = false;
    }
    // 5 .. 8 batch rows: the whole-row sweep over 32 rows of gate and the same rows of up per workgroup.  Measured on
    // 2 x 14336 x 4096 against t12_gemm + launch_silu_mul_bf16_batch: 43.6 / 44.7 us at B = 5 / 8 against 44.3 / 47.1; no
    // gain at B <= 4 (43.9 against 44.2; B = 2: 44.5 against 39) nor above 8, where the unfused launch balances its
    // last round (B = 9 / 12 / 16: 45.3 / 46.7 / 49.0 against 45.5 / 46.6 / 48.4).
    bool sweep = K % 128 == 0 && act_stride % 8 == 0 && (uintptr_t)act_bf16 % 16 == 0 && B >= 5 && B <= 8;
    for (const T12Segment* g : two)
        if (g->base_exp < 0 || g->base_exp > 240) sweep = false;
    if (sweep) {
        const int rg = 4;
        GemmParams p;
        p.seg[0] = *gate;
        p.seg[1] = *up;
        p.nseg = 2;
        p.K = K;
        p.B = B;
        p.act_stride = act_stride;
        p.act = (const uint16_t*)act_bf16;
        p.ws = nullptr;
        p.ksplit = 1;
        p.kslice = K;
        p.m_total = gate->M;
        const int sets = (gate->M + 8 * rg - 1) / (8 * rg);
        p.blk_start[0] = 0;
        p.blk_start[1] = p.blk_start[2] = sets;
        p.out_bf16 = (uint16_t*)out_bf16;
        p.out_bf16_ld = out_stride;
        hipStream_t st = (hipStream_t)stream;
        hipLaunchKernelGGL((gemm_dense16_swiglu_kernel<8, 2, 4>), dim3(sets), dim3(512), 0, st, p);
        T12_CHECK_LAUNCH("t12_gemm_swiglu(dense16)");
        return T12_OK;
    }
    const int tiles = (gate->M + TM / 2 - 1) / (TM / 2);
    const int btiles = B > 128 ? (B + 255) / 256 : 1;
    if (!fast || tiles * btiles * 4 < 256 * 3) return 1;      // would need a K split: partial sums cannot be gated
    GemmParams p;
    p.seg[0] = *gate;
    p.seg[1] = *up;
    p.nseg = 2;
    p.K = K;
    p.B = B;
    p.act_stride = act_stride;
    p.act = (const uint16_t*)act_bf16;
    p.ws = nullptr;
    p.ksplit = 1;
    p.kslice = ((K + 2 * KC - 1) / (2 * KC)) * 2 * KC;
    p.m_total = gate->M;
    p.seg_act[0] = p.act;                  // the SwiGLU tile reads the fields of segment 0
    p.seg_B[0] = B;
    p.seg_act_stride[0] = act_stride;
    p.blk_start[0] = 0;
    p.blk_start[1] = p.blk_start[2] = tiles;
    p.seg_row0[0] = p.seg_row0[1] = 0;
    p.out_bf16 = (uint16_t*)out_bf16;
    p.out_bf16_ld = out_stride;
    // batch tile of 256 rows, or of 128 for 65 .. 128 rows (one accumulator pair per wave)
    if (B <= 128) return launch_mfma<4, 2, 1, 2, true>(p, tiles, (hipStream_t)stream);
    return launch_mfma<4, 2, 2, 2, true>(p, tiles, (hipStream_t)stream);
}

}  // extern "C"

namespace {

// CUs of the current device (a launch of one workgroup per CU is one round of the small-batch kernel).
int device_cus()
{
    static std::mutex mu;
    static int cus[16] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

// The small-batch launch with rg row groups per workgroup whose last round would fill only part of the chip: every
// tensor is cut into a head, swept rg groups per workgroup in whole rounds, and a tail swept in fewer groups per
// workgroup, chosen so that the tails of all tensors together are one round.  p holds the launch as gemm_impl set it up
// (segments, K, B, activations); returns false, with nothing launched, when the plain launch is as good.
bool launch_dense16_mixed(GemmParams p, int nseg, int rg, hipStream_t st)
{
    int rows[GMAX], head_rows[GMAX];
    for (int i = 0; i < nseg; i++) rows[i] = p.seg[i].M;
    const int rgb = t12_plan_dense16_heads(rows, nseg, rg, device_cus(), GMAX, head_rows);
    if (!rgb) return false;
    // heads first, then tails.  A tail is the same tensor from row 16 rg a on: the row pointers of the escape list hold
    // absolute entry numbers, so only the pointer to them moves; 16 rg a rows of K columns are a whole number of bytes of
    // the nibble plane.
    T12Segment src[GMAX];
    for (int i = 0; i < nseg; i++) src[i] = p.seg[i];
    int n = 0, total = 0;
    p.n_first = 0;
    for (int pass = 0; pass < 2; pass++)
        for (int i = 0; i < nseg; i++) {
            const int rows_a = head_rows[i];
            const int m = pass == 0 ? rows_a : src[i].M - rows_a;
            if (m <= 0) continue;
            T12Segment g = src[i];
            if (pass == 1) {
                const size_t e = (size_t)rows_a * p.K;
                g.sm += e;
                g.gr += e / 2;
                if (g.row_off) g.row_off += rows_a;
                g.out += rows_a;
            }
            g.M = m;
            const int per = 16 * (pass == 0 ? rg : rgb);
            p.seg[n] = g;
            p.blk_start[n] = total;
            total += (m + per - 1) / per;
            n++;
            if (pass == 0) p.n_first = n;
        }
    p.blk_start[n] = total;
    p.nseg = n;
    p.ksplit = 1;
    p.kslice = p.K;
    const dim3 grid(total), block(512);
    if (rg == 4 && rgb == 3) hipLaunchKernelGGL((gemm_dense16_mixed_kernel<8, 2, 4, 3>), grid, block, 0, st, p);
    else if (rg == 4 && rgb == 2) hipLaunchKernelGGL((gemm_dense16_mixed_kernel<8, 2, 4, 2>), grid, block, 0, st, p);
    else if (rg == 4 && rgb == 1) hipLaunchKernelGGL((gemm_dense16_mixed_kernel<8, 2, 4, 1>), grid, block, 0, st, p);
    else if (rg == 2 && rgb == 1) hipLaunchKernelGGL((gemm_dense16_mixed_kernel<8, 2, 2, 1>), grid, block, 0, st, p);
    else return false;
    return true;
}

// The body of t12_gemm / t12_gemm_deferred / t12_gemm_noalloc.  static_ws: the K-split partial sums go to the
// library's fixed device array instead of a grown hipMalloc buffer, and a launch that needs more is refused.
int gemm_impl(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K,
              int B, T12GemmPartials* part, void* stream, bool static_ws)
{
    if (part) {
        part->ws = nullptr;
        part->nsplit = 1;
        part->ld = 0;
        part->split_stride = 0;
    }
    const char* who = static_ws ? "t12_gemm_noalloc" : "t12_gemm";
    T12_REQUIRE(segs && nseg >= 1 && nseg <= T12_MAX_SEGMENTS, "%s: nseg must be 1..%d (got %d)", who,
                T12_MAX_SEGMENTS, nseg);
    T12_REQUIRE(act_bf16 && K >= 1 && B >= 1, "%s: activations null or K/B < 1 (K=%d B=%d)", who, K, B);
    T12_REQUIRE(act_stride >= K, "%s: act_stride %d < K %d", who, act_stride, K);
    hipStream_t st = (hipStream_t)stream;
    GemmParams p;
    p.nseg = nseg;
    p.K = K;
    p.B = B;
    p.act_stride = act_stride;
    p.act = (const uint16_t*)act_bf16;
    p.ws = nullptr;
    p.out_bf16 = nullptr;
    p.out_bf16_ld = 0;
    bool fast = (K % KC == 0) && (act_stride % 8 == 0) && ((uintptr_t)act_bf16 % 16 == 0);
    int m_total = 0;
    for (int i = 0; i < nseg; i++) {
        const T12Segment& g = segs[i];
        T12_REQUIRE(g.M >= 1 && g.sm && g.gr && g.out, "%s: segment %d has M < 1 or a null pointer", who, i);
        T12_REQUIRE(!g.row_off || (g.cols && g.correct && g.wrong), "%s: segment %d: row_off without lists", who, i);
        T12_REQUIRE(g.base_exp >= -1 && g.base_exp <= 254, "%s: segment %d: base_exp %d out of range", who, i,
                    g.base_exp);
        if (g.base_exp < 0 || g.base_exp > 240) fast = false;
        p.seg[i] = g;
        if (p.seg[i].out_stride == 0) p.seg[i].out_stride = out_stride;
        T12_REQUIRE(p.seg[i].out_stride >= g.M, "%s: out_stride %d < M %d of segment %d", who, p.seg[i].out_stride,
                    g.M, i);
        p.seg_row0[i] = m_total;
        p.seg_act[i] = p.act;
        p.seg_B[i] = B;
        p.seg_act_stride[i] = act_stride;
        m_total += g.M;
    }
    p.m_total = m_total;
    for (int i = 0; i < nseg; i++) {
        p.seg_ws0[i] = (size_t)p.seg_row0[i];
        p.seg_ld[i] = m_total;
    }
    p.split_stride = (size_t)B * m_total;

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
    if (B == 2 && K % 1024 == 0 && K <= 8192) {
        // two batch rows: whole-row waves with two accumulators (gate|up 32 us against 42 for the kernel below; with
        // four accumulators the same kernel is no faster than the kernel below, 43-48 us, so it stops at two)
        int groups = 0;
        for (int i = 0; i < nseg; i++) {
            p.blk_start[i] = groups;
            groups += (segs[i].M + 7) / 8;
        }
        p.blk_start[nseg] = groups;
        p.ksplit = 1;
        p.kslice = K;
        hipLaunchKernelGGL((gemm_rows_kernel<2, 2>), dim3(groups), dim3(512), (size_t)2 * K * 2, st, p);
        T12_CHECK_LAUNCH("t12_gemm(rows)");
        return T12_OK;
    }
    if (B > 16 && B <= 32 && K % 128 == 0) {
        // 17 .. 32 batch rows on tensors of few rows: the same sweep with two batch tiles per weight load and decode.
        // One round of workgroups takes ~4.5 us + (K / 4096) (3.7 + 0.2 B) us whatever the row count, because every
        // workgroup reads all B activation rows for its 16 (32) weight rows; the tile kernel below needs a K split and a
        // reduction launch on such tensors and takes 15-22 us.  Measured at B = 17 / 24 / 32 (tile kernel in brackets):
        // 4096 x 4096 11.7 / 12.7 / 14.6 us (17.6-18.0), 4096 x 2048 7.6 / 8.5 / 9.1 (15.5), 1024|1024|4096 x 4096 as three
        // segments 16.7 / 17.8 / 19.1 (20.3-21.1), 8192 x 4096 16.3 / 17.6 / 18.8 (20.6), 4096 x 8192 18.8 / 21.6 / 25.2
        // (22.5).  Past one round, or with long rows, the tile kernel wins (4096 x 14336: 32 against 42 us at B = 32).
        const int C = device_cus();
        int groups16 = 0, sets2 = 0;
        for (int i = 0; i < nseg; i++) {
            groups16 += (segs[i].M + 15) / 16;
            sets2 += (segs[i].M + 31) / 32;
        }
        const long long kb = (long long)K * B;
        const int rg = groups16 <= C && kb <= 4096 * 48 ? 1 : (sets2 <= C && kb <= 5120 * 32 ? 2 : 0);
        if (rg) {
            int groups = 0;
            for (int i = 0; i < nseg; i++) {
                p.blk_start[i] = groups;
                groups += (segs[i].M + 16 * rg - 1) / (16 * rg);
            }
            p.blk_start[nseg] = groups;
            p.ksplit = 1;
            p.kslice = K;
            if (rg == 2) hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 2, false, 2>), dim3(groups), dim3(512), 0, st, p);
            else hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 1, false, 2>), dim3(groups), dim3(512), 0, st, p);
            T12_CHECK_LAUNCH("t12_gemm(dense16, two batch tiles)");
            return T12_OK;
        }
    }
    if (B <= 16 && K % 128 == 0) {
        // row groups that share an activation load: as many as leave the launch >= 448 workgroups
        int groups16 = 0;
        for (int i = 0; i < nseg; i++) groups16 += (segs[i].M + 15) / 16;
        // (measured on 28672 x 4096: at B = 16 four groups per load 49 us against 56 with one; at B = 4 45 against 42:
        // rows of a padded batch cost no activation traffic, more rows per wave cost registers)
        const int want = B > 8 ? 4 : (B > 4 ? 2 : 1);
        const int rg = groups16 >= 4 * 448 && want >= 4 ? 4 : (groups16 >= 2 * 448 && want >= 2 ? 2 : 1);
        if (rg > 1 && launch_dense16_mixed(p, nseg, rg, st)) {
            T12_CHECK_LAUNCH("t12_gemm(dense16, two workgroup sizes)");
            return T12_OK;
        }
        int groups = 0;
        for (int i = 0; i < nseg; i++) {
            p.blk_start[i] = groups;
            groups += (segs[i].M + 16 * rg - 1) / (16 * rg);
        }
        p.blk_start[nseg] = groups;
        p.ksplit = 1;
        p.kslice = K;
        if (rg == 4) hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 4>), dim3(groups), dim3(512), 0, st, p);
        else if (rg == 2) hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 2>), dim3(groups), dim3(512), 0, st, p);
        else hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 1>), dim3(groups), dim3(512), 0, st, p);
        T12_CHECK_LAUNCH("t12_gemm(dense16)");
        return T12_OK;
    }
    // K split: as many workgroups as the chip has CUs, not more (measured on the four Llama-8B layer shapes at B = 32 ..
    // 256: 32 row tiles run best as 8 splits, 48 as 4, 224 unsplit -- every doubling past ~one workgroup per CU costs more
    // in partial sums than it gains), every split at least 8 stages long.
    auto splits_for = [&](int btiles) {
        int ks = 1;
        while (tiles * btiles * ks * 2 <= 256 + 32 && K / (ks * 2) >= 8 * KC && ks < T12_MAX_KSPLIT) ks *= 2;
        return ks;
    };
    int ks = splits_for(B > 128 ? (B + 255) / 256 : 1);
    // A 256-row batch tile whose K slice is under 16 stages (O of the Llama layer: 32 row tiles, 8 splits of 512
    // columns) spends its time filling and draining, and leaves twice the partial sums: such a launch takes 128-row
    // batch tiles and half the splits (O at B = 256 32 -> 27.5 us with the reduction; down, whose slices are long,
    // 55 -> 58 us and QKV 34 -> 37 us the same way, so they keep the 256-row tile).
    const bool tb128 = B > 128 && ks > 1 && K / ks < 16 * KC;
    if (tb128) ks = splits_for((B + 127) / 128);
    int kslice = (((K + 2 * KC - 1) / (2 * KC) + ks - 1) / ks) * 2 * KC;      // whole windows of two stages
    ks = (K + kslice - 1) / kslice;
    p.ksplit = ks;
    p.kslice = kslice;
    if (ks > 1 && static_ws) {
        const size_t need = (size_t)ks * B * m_total * sizeof(float);
        T12_REQUIRE(need <= STATIC_WS_BYTES,
                    "t12_gemm_noalloc: this shape splits K %d ways and needs %zu bytes of partial sums, the fixed "
                    "workspace holds %zu (B %d x %d rows): use t12_gemm, or a smaller batch", ks, need, STATIC_WS_BYTES, B,
                    m_total);
        p.ws = static_workspace();
        if (!p.ws) {
            t12_set_error("t12_gemm_noalloc: hipGetSymbolAddress of the fixed workspace failed");
            return T12_ELAUNCH;
        }
    } else if (ks > 1) {
        p.ws = workspace((size_t)ks * B * m_total * sizeof(float), st);
        if (!p.ws) {
            t12_set_error("%s: cannot allocate %zu bytes of K-split workspace", who,
                          (size_t)ks * B * m_total * sizeof(float));
            return T12_ELAUNCH;
        }
    }
    int rc;
    if (B <= 64) rc = launch_mfma<2, 4, 1, 1>(p, tiles, st);
    else if (B <= 128 || tb128) rc = launch_mfma<2, 4, 2, 1>(p, tiles, st);
    else rc = launch_mfma<4, 2, 2, 2>(p, tiles, st);
    if (rc) return rc;

    if (ks > 1 && part) {
        part->ws = p.ws;
        part->nsplit = ks;
        part->ld = m_total;
        part->split_stride = (size_t)B * m_total;
    } else if (ks > 1) {
        launch_reduce(p, B, st);
        T12_CHECK_LAUNCH("t12_gemm(reduce)");
    }
    return T12_OK;
}

}  // namespace

extern "C" {

// t12_gemm whose K-split partial sums may be left in the workspace for the caller's next kernel to add
// up (part != NULL): part->nsplit == 1 means the outputs are complete in segs[].out.
int t12_gemm_deferred(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K,
                      int B, T12GemmPartials* part, void* stream)
{
    return gemm_impl(segs, nseg, act_bf16, act_stride, out_stride, K, B, part, stream, false);
}

// t12_gemm for callers that may not allocate device memory (HIP graph capture, serving loops, harnesses that forbid
// it): same kernels, same K split, same results bit for bit; the partial sums of a split launch live in a fixed
// T12_GEMM_NOALLOC_WS_BYTES array inside the library's device image instead of a buffer grown with hipMalloc.
// Every launch writes each partial sum it later adds, so the array needs no clearing between calls; all calls on
// one GPU share it, whatever their stream: calls that overlap in time on one GPU race.
int t12_gemm_noalloc(const T12Segment* segs, int nseg, const void* act_bf16, int act_stride, int out_stride, int K,
                     int B, void* stream)
{
    return gemm_impl(segs, nseg, act_bf16, act_stride, out_stride, K, B, nullptr, stream, true);
}

// Several products in one launch, each tensor with its own activations and batch: the experts of a mixture-of-experts
// layer (gate and up of expert e over the rows routed to e), where a launch per expert leaves the chip part empty
// and pays a K-split reduction per expert.  The row tiles of all groups fill one grid; a group with fewer rows than
// the largest simply has fewer batch tiles.  Groups the tile kernel does not take (K % 64, base_exp outside 0..240,
// activations not 16-byte aligned) run as t12_gemm calls, one per group.
int t12_gemm_grouped(const T12Group* groups, int ngroups, int K, void* stream)
{
    T12_REQUIRE(groups && ngroups >= 1 && ngroups <= GMAX, "t12_gemm_grouped: 1..%d groups (got %d)", GMAX, ngroups);
    T12_REQUIRE(K >= 1, "t12_gemm_grouped: K %d", K);
    hipStream_t st = (hipStream_t)stream;
    GemmParams p;
    p.K = K;
    p.act = nullptr;
    p.act_stride = 0;
    p.ws = nullptr;
    p.out_bf16 = nullptr;
    p.out_bf16_ld = 0;
    bool fast = K % KC == 0;
    int n = 0, m_total = 0, max_b = 0;
    size_t ws_floats = 0;
    for (int i = 0; i < ngroups; i++) {
        const T12Group& g = groups[i];
        const T12Segment& w = g.seg;
        T12_REQUIRE(g.B >= 0, "t12_gemm_grouped: group %d has B %d", i, g.B);
        if (g.B == 0) continue;                                   // an expert no row was routed to
        T12_REQUIRE(w.M >= 1 && w.sm && w.gr && w.out && g.act_bf16, "t12_gemm_grouped: group %d has M < 1 or a null pointer", i);
        T12_REQUIRE(!w.row_off || (w.cols && w.correct && w.wrong), "t12_gemm_grouped: group %d: row_off without lists", i);
        T12_REQUIRE(w.base_exp >= -1 && w.base_exp <= 254, "t12_gemm_grouped: group %d: base_exp %d out of range", i, w.base_exp);
        T12_REQUIRE(g.act_stride >= K && w.out_stride >= w.M, "t12_gemm_grouped: group %d: act_stride %d < K %d or out_stride %d < M %d",
                    i, g.act_stride, K, w.out_stride, w.M);
        if (w.base_exp < 0 || w.base_exp > 240 || g.act_stride % 8 != 0 || (uintptr_t)g.act_bf16 % 16 != 0) fast = false;
        p.seg[n] = w;
        p.seg_row0[n] = m_total;
        p.seg_act[n] = (const uint16_t*)g.act_bf16;
        p.seg_B[n] = g.B;
        p.seg_act_stride[n] = g.act_stride;
        p.seg_ws0[n] = ws_floats;
        p.seg_ld[n] = w.M;
        ws_floats += (size_t)g.B * w.M;
        m_total += w.M;
        max_b = g.B > max_b ? g.B : max_b;
        n++;
    }
    if (n == 0) return T12_OK;
    if (!fast) {
        for (int i = 0; i < n; i++) {
            const int rc = gemm_impl(&p.seg[i], 1, p.seg_act[i], p.seg_act_stride[i], p.seg[i].out_stride, K, p.seg_B[i],
                                     nullptr, stream, false);
            if (rc) return rc;
        }
        return T12_OK;
    }
    p.nseg = n;
    p.B = max_b;
    p.m_total = m_total;
    p.split_stride = ws_floats;
    // batch tile by the largest group, so that every tensor is streamed once (a Mixtral layer of 256 tokens, 48 .. 75
    // rows per expert: 0.80 ms with tiles of 128, 0.94 with tiles of 64 taken twice by the larger groups, 1.05 with 256)
    const int tb = max_b <= 64 ? 64 : (max_b <= 128 ? 128 : 256);
    int tiles = 0;
    long units = 0;                                               // workgroups per K split
    for (int i = 0; i < n; i++) {
        p.blk_start[i] = tiles;
        const int t = (p.seg[i].M + TM - 1) / TM;
        tiles += t;
        units += (long)t * ((p.seg_B[i] + tb - 1) / tb);
    }
    p.blk_start[n] = tiles;
    int ks = 1;
    while (units * ks * 2 <= 256 + 32 && K / (ks * 2) >= 8 * KC && ks < T12_MAX_KSPLIT) ks *= 2;   // as in t12_gemm
    const int kslice = (((K + 2 * KC - 1) / (2 * KC) + ks - 1) / ks) * 2 * KC;
    ks = (K + kslice - 1) / kslice;
    p.ksplit = ks;
    p.kslice = kslice;
    if (ks > 1) {
        p.ws = workspace((size_t)ks * ws_floats * sizeof(float), st);
        if (!p.ws) {
            t12_set_error("t12_gemm_grouped: cannot allocate %zu bytes of K-split workspace", (size_t)ks * ws_floats * sizeof(float));
            return T12_ELAUNCH;
        }
    }
    int rc;
    if (tb == 64) rc = launch_mfma<2, 4, 1, 1>(p, tiles, st);
    else if (tb == 128) rc = launch_mfma<2, 4, 2, 1>(p, tiles, st);
    else rc = launch_mfma<4, 2, 2, 2>(p, tiles, st);
    if (rc) return rc;
    if (ks > 1) {
        launch_reduce(p, max_b, st);
        T12_CHECK_LAUNCH("t12_gemm_grouped(reduce)");
    }
    return T12_OK;
}

// Library-internal (t12_moe_ffn): the experts of a mixture-of-experts layer in one launch, with the rows per expert
// known on the device only.  pairs = 0: segment i belongs to group first_group + i; 1 or 2: the segments are (gate, up)
// pairs, segment i belongs to group first_group + i / 2.  Group g has dev_counts[g] rows, which start dev_base[g] rows
// into act_bf16 and into the outputs: seg.out (fp32), or for pairs = 1 out_bf16 = bf16( silu(gate) * up ), row stride
// out_bf16_ld.  hint_b is a count few groups exceed: it
// picks the batch tile (a group above it is streamed once per tile it needs).  K is never split.  Returns 1 when the shape has no such kernel (the caller then sizes launches on the host).
__attribute__((visibility("hidden"))) int t12_gemm_experts(const T12Segment* segs, int nseg, int K, const void* act_bf16,
                                                           int act_stride, const int* dev_counts, const int* dev_base,
                                                           int first_group, int hint_b, int pairs,
                                                           void* out_bf16, int out_bf16_ld, void* stream)
{
    const bool swiglu = pairs == 1;
    if (nseg < 1 || nseg > GMAX || (pairs && nseg % 2)) return 1;
    if (K % KC || act_stride % 8 || (uintptr_t)act_bf16 % 16) return 1;
    for (int i = 0; i < nseg; i++)
        if (segs[i].base_exp < 0 || segs[i].base_exp > 240 || !segs[i].sm || !segs[i].gr) return 1;
    GemmParams p;
    p.K = K;
    p.act = (const uint16_t*)act_bf16;
    p.act_stride = act_stride;
    p.ws = nullptr;
    p.ksplit = 1;
    p.kslice = ((K + 2 * KC - 1) / (2 * KC)) * 2 * KC;
    p.out_bf16 = (uint16_t*)out_bf16;
    p.out_bf16_ld = out_bf16_ld;
    p.dev_counts = dev_counts;
    p.dev_base = dev_base;
    p.nseg = nseg;
    p.B = 1;                               // one workgroup per row tile (it walks the group's batch tiles itself)
    p.split_stride = 0;
    int tiles = 0, m_total = 0;
    for (int i = 0; i < nseg; i++) {
        p.seg[i] = segs[i];
        p.seg_row0[i] = m_total;
        p.seg_act[i] = p.act;
        p.seg_B[i] = 0;
        p.seg_act_stride[i] = act_stride;
        p.seg_ws0[i] = 0;
        p.seg_ld[i] = segs[i].M;
        p.group_of_seg[i] = first_group + (pairs ? i / 2 : i);
        m_total += segs[i].M;
        if (!swiglu) {
            p.blk_start[i] = tiles;
            tiles += (segs[i].M + TM - 1) / TM;
        } else if (i % 2 == 0) {
            if (segs[i].M != segs[i + 1].M) return 1;
            p.blk_start[i / 2] = tiles;
            tiles += (segs[i].M + TM / 2 - 1) / (TM / 2);
        }
    }
    p.m_total = m_total;
    p.npair = swiglu ? nseg / 2 : 1;
    if (!swiglu) p.blk_start[nseg] = tiles;
    hipStream_t st = (hipStream_t)stream;
    if (!swiglu && hint_b <= 8 && K % 128 == 0) {
        // a few rows per group (a decode step of a mixture-of-experts model): bound by the weight stream, so the kernel
        // that sweeps 16 whole rows per workgroup; groups without rows cost a workgroup's exit.  (Measured on the
        // Mixtral shape: 1 token 0.16 ms against 0.25 through the tile kernel, 4 tokens 0.46 against 0.52; at 16
        // tokens -- 4 rows per expert, hint 12 -- the tile kernel is level again: 0.52 against 0.55.)
        int groups = 0;
        for (int i = 0; i < nseg; i++) {
            p.blk_start[i] = groups;
            groups += (segs[i].M + 15) / 16;
        }
        p.blk_start[nseg] = groups;
        p.kslice = K;
        hipLaunchKernelGGL((gemm_dense16_kernel<8, 2, 1, true>), dim3(groups), dim3(512), 0, st, p);
        T12_CHECK_LAUNCH("t12_moe_ffn(dense16)");
        return T12_OK;
    }
    if (swiglu) {
        if (hint_b <= 128) return launch_mfma<4, 2, 1, 2, true>(p, tiles, st);
        return launch_mfma<4, 2, 2, 2, true>(p, tiles, st);
    }
    if (hint_b <= 64) return launch_mfma<2, 4, 1, 1>(p, tiles, st);
    if (hint_b <= 128) return launch_mfma<2, 4, 2, 1>(p, tiles, st);
    return launch_mfma<4, 2, 2, 2>(p, tiles, st);
}

// The library keeps device buffers per (device, stream): the K-split partial sums of t12_gemm*, the argmax partials and the
// context-split buffers of the glue kernels, the sampler's result ids.  A caller about to destroy a stream hands them back here (waits for the
// stream first); a stream that is used again afterwards simply gets new ones.
int t12_release_stream(void* stream)
{
    hipStream_t st = (hipStream_t)stream;
    if (hipStreamSynchronize(st) != hipSuccess) {
        t12_set_error("t12_release_stream: hipStreamSynchronize failed: %s", hipGetErrorString(hipGetLastError()));
        return T12_ELAUNCH;
    }
    release_workspace(st);
    t12_glue_release_stream(st);
    t12_sampler_release_stream(st);
    return T12_OK;
}

}  // extern "C"
