// GPU-side split-12 packer (gfx950): bf16 matrix in HBM -> planes + CSR escape
// list, byte-identical to what the reference's CPU packer emits.
//
//   t12_pack_histogram + t12_pack_base_exp   = split12_find_base_exp (split12_pack.c:18-37)
//   t12_pack_planes / _row_offsets / _escapes = pack_split12          (split12_pack.c:47-128)
//
// The reference makes two O(M*K) passes on one CPU thread; here the first pass
// is a streaming kernel (16 weights per lane, 32 B in, 24 B out), the CSR pointers
// come from a single-workgroup scan of the per-row escape counts, and the
// second pass compacts each row's escapes in ascending column order with one
// wave per row (ballot + prefix popcount), so the order inside a row is the
// reference's.

#include "t12_device.h"
#include "t12_host.h"

namespace {

__device__ __forceinline__ uint32_t group_of(uint32_t v, int base_exp)
{
    const int g = (int)((v >> 7) & 0xFFu) - base_exp;
    return (g >= 1 && g <= 15) ? (uint32_t)g : 0u;
}

// Exponent histogram.  The exponents of a weight matrix fall into a handful of bins, so 64 lanes adding into one
// 256-bin table serialise on those bins (LDS atomics to one address execute one lane at a time: measured 0.8 TB/s).
// Sixteen copies of the table, picked by lane % 16 and laid out [bin][copy] (the copies of a bin are sixteen
// neighbouring banks), leave at most four lanes of a wave on one counter.
constexpr int HIST_COPIES = 16;
__global__ __launch_bounds__(256) void histogram_kernel(const uint16_t* __restrict__ w, size_t n,
                                                        unsigned long long* __restrict__ hist)
{
    __shared__ unsigned int h[256 * HIST_COPIES];
    for (int i = threadIdx.x; i < 256 * HIST_COPIES; i += 256) h[i] = 0;
    __syncthreads();
    const int copy = threadIdx.x & (HIST_COPIES - 1);
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t n8 = n / 8;
    // four 16-byte pieces per lane in flight (the grid is small, see the launcher)
    for (size_t q0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q0 < n8; q0 += 4 * stride) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const size_t q = q0 + u * stride;
            v[u] = q < n8 ? *(const uint4*)(w + q * 8) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (q0 + u * stride >= n8) break;
            const uint32_t d[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                atomicAdd(&h[(((d[i] >> 7) & 0xFFu) * HIST_COPIES) | copy], 1u);
                atomicAdd(&h[(((d[i] >> 23) & 0xFFu) * HIST_COPIES) | copy], 1u);
            }
        }
    }
    if (blockIdx.x == 0)
        for (size_t i = n8 * 8 + threadIdx.x; i < n; i += blockDim.x) atomicAdd(&h[(((uint32_t)w[i] >> 7) & 0xFFu) * HIST_COPIES], 1u);
    __syncthreads();
    unsigned int sum = 0;
#pragma unroll
    for (int c = 0; c < HIST_COPIES; c++) sum += h[threadIdx.x * HIST_COPIES + ((c + threadIdx.x) & (HIST_COPIES - 1))];
    if (sum) atomicAdd(&hist[threadIdx.x], (unsigned long long)sum);
}

// Planes for the whole 16-element pieces of the flat array.
__global__ __launch_bounds__(256) void planes_kernel(const uint16_t* __restrict__ w, size_t n16, int K,
                                                     int base_exp, uint8_t* __restrict__ sm,
                                                     uint8_t* __restrict__ gr, int32_t* __restrict__ row_cnt)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < n16; q += stride) {
        const uint4 lo = *(const uint4*)(w + q * 16);
        const uint4 hi = *(const uint4*)(w + q * 16 + 8);
        const uint32_t d[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        uint32_t s[4] = {0, 0, 0, 0};
        uint32_t g[2] = {0, 0};
        uint32_t esc = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t v = (d[i >> 1] >> (16 * (i & 1))) & 0xFFFFu;
            const uint32_t gi = group_of(v, base_exp);
            s[i >> 2] |= (((v >> 15) << 7) | (v & 0x7Fu)) << (8 * (i & 3));
            g[i >> 3] |= gi << (4 * (i & 7));
            esc |= (gi == 0u) << i;
        }
        *(uint4*)(sm + q * 16) = make_uint4(s[0], s[1], s[2], s[3]);
        *(uint2*)(gr + q * 8) = make_uint2(g[0], g[1]);
        while (esc) {                                   // rare: ~0.05 % of the weights
            const int i = __builtin_ctz(esc);
            esc &= esc - 1;
            atomicAdd(&row_cnt[(q * 16 + i) / (size_t)K], 1);
        }
    }
}

// The last n % 16 elements, by one lane (an odd count leaves the high nibble 0).
__global__ void planes_tail_kernel(const uint16_t* __restrict__ w, size_t first, size_t n, int K, int base_exp,
                                   uint8_t* __restrict__ sm, uint8_t* __restrict__ gr,
                                   int32_t* __restrict__ row_cnt)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    for (size_t i = first; i < n; i++) {
        const uint32_t v = w[i];
        const uint32_t gi = group_of(v, base_exp);
        sm[i] = (uint8_t)(((v >> 15) << 7) | (v & 0x7Fu));
        if (i & 1) gr[i >> 1] = (uint8_t)(gr[i >> 1] | (gi << 4));
        else gr[i >> 1] = (uint8_t)gi;
        if (gi == 0u) atomicAdd(&row_cnt[i / (size_t)K], 1);
    }
}

// row_off[0] = 0, row_off[r+1] = sum of cnt[0..r]; one workgroup of 1024 lanes.
__global__ __launch_bounds__(1024) void scan_kernel(const int32_t* __restrict__ cnt, int M,
                                                    int32_t* __restrict__ row_off)
{
    __shared__ int part[1024];
    const int t = threadIdx.x;
    const int per = (M + 1023) / 1024;
    const int lo = min(t * per, M), hi = min(lo + per, M);
    int s = 0;
    for (int r = lo; r < hi; r++) s += cnt[r];
    part[t] = s;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {          // Hillis-Steele inclusive scan
        const int v = t >= off ? part[t - off] : 0;
        __syncthreads();
        part[t] += v;
        __syncthreads();
    }
    int run = part[t] - s;                              // exclusive prefix of this lane's chunk
    if (t == 0) row_off[0] = 0;
    for (int r = lo; r < hi; r++) {
        run += cnt[r];
        row_off[r + 1] = run;
    }
}

// One wave per row: ordered compaction of the row's escapes.  K % 8 == 0 (rows start 16-byte aligned): a lane takes
// eight consecutive columns per step with one 128-bit load and the wave skips a step without escapes after one
// ballot; the order of the list (ascending column) is lane-major within a step, so an entry's place is the count of
// escapes in lower lanes plus the lane's own earlier ones.  Other K: one column per lane and step.
__global__ __launch_bounds__(256) void escapes_kernel(const uint16_t* __restrict__ w, int M, int K, int base_exp,
                                                      const int32_t* __restrict__ row_off,
                                                      int32_t* __restrict__ cols, int16_t* __restrict__ correct,
                                                      int16_t* __restrict__ wrong)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int lane = threadIdx.x & 63;
    int base = row_off[row];
    if (row_off[row + 1] == base) return;               // nothing to write in this row
    const uint16_t* wr = w + (size_t)row * K;
    if ((K & 7) == 0 && ((uintptr_t)w & 15) == 0) {
        const unsigned long long below = (1ull << lane) - 1ull;
        for (int k0 = 0; k0 < K; k0 += T12_WAVE * 8) {
            const int k = k0 + lane * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (k < K) v = *(const uint4*)(wr + k);
            const uint32_t d[4] = {v.x, v.y, v.z, v.w};
            uint32_t mine = 0;                           // bit j: column k + j is an escape
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t e = (d[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                if (k < K && group_of(e, base_exp) == 0u) mine |= 1u << j;
            }
            if (__ballot(mine != 0u) == 0ull) continue;
            // escapes in lower lanes: a wave prefix sum of the lanes' counts, by one ballot per bit of the count (<= 8)
            const int cnt = __popc(mine);
            int before = 0;
#pragma unroll
            for (int bit = 0; bit < 4; bit++)
                before += __popcll(__ballot((cnt >> bit) & 1) & below) << bit;
            int total = 0;
#pragma unroll
            for (int bit = 0; bit < 4; bit++) total += __popcll(__ballot((cnt >> bit) & 1)) << bit;
            int pos = base + before;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (mine & (1u << j)) {
                    const uint32_t e = (d[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                    cols[pos] = k + j;
                    correct[pos] = (int16_t)e;
                    wrong[pos] = (int16_t)t12_decode_scalar(((e >> 15) << 7) | (e & 0x7Fu), 0u, base_exp);
                    pos++;
                }
            }
            base += total;
        }
        return;
    }
    for (int k0 = 0; k0 < K; k0 += T12_WAVE) {
        const int k = k0 + lane;
        const uint32_t v = k < K ? wr[k] : 0u;
        const bool esc = k < K && group_of(v, base_exp) == 0u;
        const unsigned long long m = __ballot(esc);
        if (esc) {
            const int pos = base + __popcll(m & ((1ull << lane) - 1ull));
            cols[pos] = k;
            correct[pos] = (int16_t)v;
            wrong[pos] = (int16_t)t12_decode_scalar(((v >> 15) << 7) | (v & 0x7Fu), 0u, base_exp);
        }
        base += __popcll(m);
    }
}

int blocks_for(size_t items)
{
    const size_t want = (items + 255) / 256;
    return (int)(want < 1 ? 1 : (want < 256 * 32 ? want : 256 * 32));
}

}  // namespace

extern "C" {

int t12_pack_histogram(const void* w_bf16, size_t n, void* hist_u64x256, void* stream)
{
    T12_REQUIRE(hist_u64x256 && (w_bf16 || n == 0), "t12_pack_histogram: null operand");
    T12_REQUIRE((uintptr_t)w_bf16 % 16 == 0, "t12_pack_histogram: input must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (hipMemsetAsync(hist_u64x256, 0, 256 * sizeof(unsigned long long), st) != hipSuccess) return T12_ELAUNCH;
    if (n == 0) return T12_OK;
    // few workgroups, long strides: every workgroup ends with one 64-bit atomic per bin it met, and those all land on
    // the same dozen addresses (8192 workgroups spent 130 us there, whatever the size of the matrix)
    const int blocks = blocks_for(n / 8) < 512 ? blocks_for(n / 8) : 512;
    hipLaunchKernelGGL(histogram_kernel, dim3(blocks), dim3(256), 0, st, (const uint16_t*)w_bf16, n,
                       (unsigned long long*)hist_u64x256);
    T12_CHECK_LAUNCH("t12_pack_histogram");
    return T12_OK;
}

// Host: the window rule of split12_find_base_exp on a 256-bin histogram.
int t12_pack_base_exp(const uint64_t* hist_host)
{
    uint64_t best = 0, run = 0;
    int best_start = 0;
    for (int j = 0; j < 15; j++) run += hist_host[j];
    for (int s = 0; s <= 241; s++) {
        if (s > 0) run += hist_host[s + 14] - hist_host[s - 1];
        if (run > best) { best = run; best_start = s; }
    }
    return best_start - 1;
}

int t12_pack_planes(const void* w_bf16, int M, int K, int base_exp, void* sm, void* gr, void* row_cnt,
                    void* stream)
{
    T12_REQUIRE(M >= 1 && K >= 1 && w_bf16 && sm && gr && row_cnt, "t12_pack_planes: bad operands");
    T12_REQUIRE(base_exp >= -1 && base_exp <= 240, "t12_pack_planes: base_exp %d out of range", base_exp);
    T12_REQUIRE((uintptr_t)w_bf16 % 16 == 0 && (uintptr_t)sm % 16 == 0 && (uintptr_t)gr % 8 == 0,
                "t12_pack_planes: buffers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const size_t n = (size_t)M * K, n16 = n / 16;
    if (hipMemsetAsync(row_cnt, 0, (size_t)M * sizeof(int32_t), st) != hipSuccess) return T12_ELAUNCH;
    if (n16) {
        hipLaunchKernelGGL(planes_kernel, dim3(blocks_for(n16)), dim3(256), 0, st, (const uint16_t*)w_bf16, n16, K,
                           base_exp, (uint8_t*)sm, (uint8_t*)gr, (int32_t*)row_cnt);
        T12_CHECK_LAUNCH("t12_pack_planes");
    }
    if (n16 * 16 < n) {
        hipLaunchKernelGGL(planes_tail_kernel, dim3(1), dim3(64), 0, st, (const uint16_t*)w_bf16, n16 * 16, n, K,
                           base_exp, (uint8_t*)sm, (uint8_t*)gr, (int32_t*)row_cnt);
        T12_CHECK_LAUNCH("t12_pack_planes(tail)");
    }
    return T12_OK;
}

int t12_pack_row_offsets(const void* row_cnt, int M, void* row_off, void* stream)
{
    T12_REQUIRE(M >= 1 && row_cnt && row_off, "t12_pack_row_offsets: bad operands");
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const int32_t*)row_cnt, M,
                       (int32_t*)row_off);
    T12_CHECK_LAUNCH("t12_pack_row_offsets");
    return T12_OK;
}

int t12_pack_escapes(const void* w_bf16, int M, int K, int base_exp, const void* row_off, void* cols,
                     void* correct, void* wrong, void* stream)
{
    T12_REQUIRE(M >= 1 && K >= 1 && w_bf16 && row_off, "t12_pack_escapes: bad operands");
    if (!cols || !correct || !wrong) return T12_OK;     // P == 0: nothing to fill
    hipLaunchKernelGGL(escapes_kernel, dim3((M + 3) / 4), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)w_bf16, M, K, base_exp, (const int32_t*)row_off, (int32_t*)cols,
                       (int16_t*)correct, (int16_t*)wrong);
    T12_CHECK_LAUNCH("t12_pack_escapes");
    return T12_OK;
}

}  // extern "C"
