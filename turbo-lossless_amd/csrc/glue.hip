// Engine glue kernels for gfx950: embedding lookup, RMSNorm (+ residual add) ->
// bf16, SiLU*mul -> bf16, RoPE, INT8 KV store, decode attention over the INT8
// cache, argmax.  Same C signatures and arithmetic as the reference's launch
// layer (engine/kernels.hip; cited per function), different kernels:
//   * RoPE and the INT8 KV store of the B = 1 path are one launch (the reference
//     uses two, kernels.hip:308-333);
//   * one decode-attention kernel serves both of the reference's variants
//     (attention_all_heads, kernels.hip:499-586, and flash_attention, :883-993):
//     online softmax over 256-position tiles, all query heads of a KV group in
//     one workgroup so the INT8 cache is read once per group, not once per head;
//   * argmax is two-phase (many workgroups per row, then one) so that a single
//     row of 128256 logits is not read by one CU.
// All math is fp32; bf16 is produced with round-to-nearest-even exactly as
// float_to_bf16 (kernels.hip:21-27).

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "t12_device.h"
#include "t12_host.h"

extern "C" void t12_rope_freqs(int head_dim, float theta, float factor, float low_freq_factor, float high_freq_factor,
                               float original_ctx, float* out);

namespace {

// Wave-wide maximum, valid in every lane: six DPP row operations fold the wave into lane 63 (lanes a step does not
// reach keep their own value), one v_readlane hands it to everybody.  (Six exchanges through ds_bpermute take several
// times as long; the attention kernels do three to five such reductions one after the other per tile.)
__device__ __forceinline__ float wave_max(float v)
{
#define T12_DPP_MAX(ctrl, rmask)                                                                                   \
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v),                 \
                                                                       __builtin_bit_cast(int, v), (ctrl), (rmask), \
                                                                       0xF, false)))
    T12_DPP_MAX(0xB1, 0xF);    // quad_perm [1,0,3,2]
    T12_DPP_MAX(0x4E, 0xF);    // quad_perm [2,3,0,1]
    T12_DPP_MAX(0x141, 0xF);   // row_half_mirror
    T12_DPP_MAX(0x140, 0xF);   // row_mirror: every lane of a 16-lane row holds the row maximum
    T12_DPP_MAX(0x142, 0xA);   // row_bcast15 into rows 1 and 3
    T12_DPP_MAX(0x143, 0xC);   // row_bcast31 into rows 2 and 3
#undef T12_DPP_MAX
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Wave-wide sum by the same route (the order of the additions differs from t12_wave_sum's butterfly).
__device__ __forceinline__ float wave_sum_dpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t12_wave_sum_lane63(v)), 63));
}

// Block-wide sum / max over up to 16 waves; every thread gets the result.
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* red /* >= 17 floats */)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = IS_MAX ? wave_max(v) : t12_wave_sum(v);
    __syncthreads();                       // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < nw; w++) r = IS_MAX ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// ---------------------------------------------------------------- embedding
// hidden[b, i] = f32(embd[token_b, i]); an out-of-range id gives zeros (kernels.hip:57-73).
__global__ __launch_bounds__(256) void embed_kernel(const uint16_t* __restrict__ embd, const int* __restrict__ tok,
                                                    float* __restrict__ out, int n_embd, int n_vocab)
{
    const int b = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_embd) return;
    const int t = tok[b];
    out[(size_t)b * n_embd + i] =
        (t >= 0 && t < n_vocab) ? t12_bf16_to_f32(embd[(size_t)t * n_embd + i]) : 0.0f;
}

// ------------------------------------------------------------------ RMSNorm
// y = bf16(x * rsqrt(mean(x^2) + eps) * w); with ADD: x += residual first, written back
// (kernels.hip:355-392 and :399-442).  One workgroup per row, values kept in registers
// between the two passes.
// PART: x[row] is first rebuilt as the sum of nsplit partial rows (ascending, the order of the GEMM's
// own reduction kernel) -- the K-split decode+GEMM leaves them for this kernel to add up.
template <bool ADD, bool PART = false>
__global__ __launch_bounds__(1024) void rms_norm_kernel(float* __restrict__ x, const float* __restrict__ res,
                                                        const float* __restrict__ w, uint16_t* __restrict__ y,
                                                        int n, float eps, const float* __restrict__ part = nullptr,
                                                        int nsplit = 0, size_t split_stride = 0, int ld = 0)
{
    __shared__ float red[17];
    const size_t off = (size_t)blockIdx.x * n;
    const float* prow = PART ? part + (size_t)blockIdx.x * ld : nullptr;
    auto value = [&](int i) {
        float t;
        if (PART) {
            // all partial loads of the element in flight together, then the sum in ascending order
            float pz[T12_MAX_KSPLIT];
#pragma unroll
            for (int z = 0; z < T12_MAX_KSPLIT; z++) pz[z] = z < nsplit ? prow[(size_t)z * split_stride + i] : 0.0f;
            t = 0.0f;
#pragma unroll
            for (int z = 0; z < T12_MAX_KSPLIT; z++)
                if (z < nsplit) t += pz[z];
        } else {
            t = x[off + i];
        }
        if (ADD) t += res[off + i];
        if (ADD || PART) x[off + i] = t;
        return t;
    };
    constexpr int MAXV = 8;                // up to 8 values per thread in registers (n <= 8 * blockDim)
    float v[MAXV];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; j++) {
        const int i = threadIdx.x + j * blockDim.x;
        v[j] = 0.0f;
        if (i < n) {
            const float t = value(i);
            v[j] = t;
            ss += t * t;
        }
    }
    for (int i = threadIdx.x + MAXV * blockDim.x; i < n; i += blockDim.x) {   // very wide rows
        const float t = value(i);
        ss += t * t;
    }
    ss = block_reduce<false>(ss, red);
    const float r = rsqrtf(ss / (float)n + eps);
#pragma unroll
    for (int j = 0; j < MAXV; j++) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < n) y[off + i] = t12_f32_to_bf16(v[j] * r * w[i]);
    }
    for (int i = threadIdx.x + MAXV * blockDim.x; i < n; i += blockDim.x)
        y[off + i] = t12_f32_to_bf16(x[off + i] * r * w[i]);
}

// The same for rows of 4 n' <= 8192 values with 16-byte aligned operands: every thread owns one or two pieces of four
// neighbouring values and requests everything it needs for them -- all partial rows, the residual, the norm weights --
// in one go as 128-bit loads, so the row costs one memory round trip, a block sum and the stores.  NZ = most partial
// rows the instance unrolls.  Sums per element are formed exactly as above (ascending partials, then the residual).
template <bool ADD, bool PART, int NZ>
__global__ __launch_bounds__(1024) void rms_norm_vec_kernel(float* __restrict__ x, const float* __restrict__ res,
                                                            const float* __restrict__ w, uint16_t* __restrict__ y,
                                                            int n, float eps, const float* __restrict__ part,
                                                            int nsplit, size_t split_stride, int ld)
{
    __shared__ float red[17];
    constexpr int NP = 2;
    const size_t off = (size_t)blockIdx.x * n;
    const float* prow = PART ? part + (size_t)blockIdx.x * ld : nullptr;
    float4 v[NP], wv[NP];
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < NP; u++) {
        const int i = (threadIdx.x + u * blockDim.x) * 4;
        v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        wv[u] = v[u];
        if (i < n) {
            float4 pz[PART ? NZ : 1], r4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f), t;
            if (PART) {
#pragma unroll
                for (int z = 0; z < NZ; z++)
                    pz[z] = z < nsplit ? *(const float4*)(prow + (size_t)z * split_stride + i) : r4;
            } else {
                pz[0] = *(const float4*)(x + off + i);
            }
            if (ADD) r4 = *(const float4*)(res + off + i);
            wv[u] = *(const float4*)(w + i);
            if (PART) {
                t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
                for (int z = 0; z < NZ; z++)
                    if (z < nsplit) { t.x += pz[z].x; t.y += pz[z].y; t.z += pz[z].z; t.w += pz[z].w; }
            } else {
                t = pz[0];
            }
            if (ADD) { t.x += r4.x; t.y += r4.y; t.z += r4.z; t.w += r4.w; }
            if (ADD || PART) *(float4*)(x + off + i) = t;
            v[u] = t;
            ss += t.x * t.x + t.y * t.y + t.z * t.z + t.w * t.w;
        }
    }
    ss = block_reduce<false>(ss, red);
    const float r = rsqrtf(ss / (float)n + eps);
#pragma unroll
    for (int u = 0; u < NP; u++) {
        const int i = (threadIdx.x + u * blockDim.x) * 4;
        if (i < n)
            *(uint2*)(y + off + i) =
                make_uint2(t12_f32_to_bf16(v[u].x * r * wv[u].x) | ((uint32_t)t12_f32_to_bf16(v[u].y * r * wv[u].y) << 16),
                           t12_f32_to_bf16(v[u].z * r * wv[u].z) | ((uint32_t)t12_f32_to_bf16(v[u].w * r * wv[u].w) << 16));
    }
}

// ----------------------------------------------------------------- SiLU*mul
// out = bf16( g / (1 + exp(-g)) * up )   (kernels.hip:447-459)
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       uint16_t* __restrict__ out, size_t total)
{
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < total) {
        const float4 g = *(const float4*)(gate + i);
        const float4 u = *(const float4*)(up + i);
        const uint32_t lo = t12_f32_to_bf16(g.x / (1.0f + expf(-g.x)) * u.x) |
                            ((uint32_t)t12_f32_to_bf16(g.y / (1.0f + expf(-g.y)) * u.y) << 16);
        const uint32_t hi = t12_f32_to_bf16(g.z / (1.0f + expf(-g.z)) * u.z) |
                            ((uint32_t)t12_f32_to_bf16(g.w / (1.0f + expf(-g.w)) * u.w) << 16);
        *(uint2*)(out + i) = make_uint2(lo, hi);
    } else {
        for (size_t j = i; j < total; j++) {
            const float g = gate[j];
            out[j] = t12_f32_to_bf16(g / (1.0f + expf(-g)) * up[j]);
        }
    }
}

__global__ __launch_bounds__(256) void add_kernel(float* __restrict__ y, const float* __restrict__ x, size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < total) y[i] += x[i];
}

// --------------------------------------------------------- RoPE + KV store
// Rotate-half RoPE: pairs (d, d + hd/2), angle = pos * freq[d]  (kernels.hip:174-213, 717-754).
// INT8 store per (position, kv head): scale = absmax / 127,
// q = clamp(rint(v * (127 / absmax)), +-127)                    (kernels.hip:220-304, 760-845).
// Grid: (n_head + 2 * n_head_kv, B); one wave per head.
//   blocks [0, n_head)                     rotate a Q head in place
//   blocks [n_head, n_head + nkv)          rotate a K head in place, then quantise + store it
//   blocks [n_head + nkv, n_head + 2 nkv)  quantise + store a V head
// MODE bit 0: do the rotations; bit 1: do the stores.
// Rotate-half RoPE of one pair (kernels.hip:244-262): two products and one add / subtract each, never
// contracted into fused multiply-adds, so that every kernel that rotates gives the same bits.
__device__ __forceinline__ void rope_rotate(float x0, float x1, float sn, float cs, float& r0, float& r1)
{
#pragma clang fp contract(off)
    const float a = x0 * cs, b = x1 * sn, c = x0 * sn, d = x1 * cs;
    r0 = a - b;
    r1 = c + d;
}

// Partial sums of a K-split q|k|v projection (t12_gemm_deferred): element (b, col) of the fused
// [q | k | v] row is the ascending sum over z < nsplit of ws[z * split_stride + b * ld + col].
// nsplit == 0: the values are complete in the q / k / v buffers.
struct QkvPartials {
    const float* ws;
    int nsplit;
    int ld;
    size_t split_stride;
};

template <int MODE>
__global__ __launch_bounds__(64) void rope_kv_kernel(float* __restrict__ q, float* __restrict__ k,
                                                     const float* __restrict__ v, int8_t* __restrict__ ck,
                                                     int8_t* __restrict__ cv, float* __restrict__ sk,
                                                     float* __restrict__ sv, const float* __restrict__ freqs,
                                                     const int* __restrict__ positions, int position,
                                                     int head_dim, int n_head, int n_head_kv, int q_stride,
                                                     int k_stride, QkvPartials part = QkvPartials{nullptr, 0, 0, 0},
                                                     size_t kv_stride = 0, int hm = 0)
{
    const int b = blockIdx.y;
    const int pos = positions ? positions[b] : position;
    const int lane = threadIdx.x;
    const int half = head_dim >> 1;
    int blk = blockIdx.x;
    float* rot = nullptr;
    const float* src = nullptr;
    int8_t* dst = nullptr;
    float* sdst = nullptr;
    int kvh = 0;
    int pcol = 0;                       // first column of this head in the fused [q | k | v] row
    if (blk < n_head) {
        rot = q + (size_t)b * q_stride + (size_t)blk * head_dim;
        pcol = blk * head_dim;
    } else if (blk < n_head + n_head_kv) {
        kvh = blk - n_head;
        rot = k + (size_t)b * k_stride + (size_t)kvh * head_dim;
        src = rot;
        dst = ck;
        sdst = sk;
        pcol = (n_head + kvh) * head_dim;
    } else {
        kvh = blk - n_head - n_head_kv;
        src = v + (size_t)b * k_stride + (size_t)kvh * head_dim;
        dst = cv;
        sdst = sv;
        pcol = (n_head + n_head_kv + kvh) * head_dim;
    }
    // value i of this head: from its buffer, or rebuilt from the K-split partial sums
    auto value = [&](const float* buf, int i) {
        if (part.nsplit == 0) return buf[i];
        const float* pr = part.ws + (size_t)b * part.ld + pcol + i;
        float pz[T12_MAX_KSPLIT];
#pragma unroll
        for (int z = 0; z < T12_MAX_KSPLIT; z++) pz[z] = z < part.nsplit ? pr[(size_t)z * part.split_stride] : 0.0f;
        float t = 0.0f;
#pragma unroll
        for (int z = 0; z < T12_MAX_KSPLIT; z++)
            if (z < part.nsplit) t += pz[z];
        return t;
    };
    // lane owns the pair (lane, lane + half); head_dim <= 128 so one pair per lane
    const bool own = lane < half;
    float r0 = 0.0f, r1 = 0.0f;
    if ((MODE & 1) && rot) {
        if (own) {
            const float ang = (float)pos * freqs[lane];
            float sn, cs;
            sincosf(ang, &sn, &cs);
            const float x0 = value(rot, lane), x1 = value(rot, lane + half);
            rope_rotate(x0, x1, sn, cs, r0, r1);
            rot[lane] = r0;
            rot[lane + half] = r1;
        }
    } else if (src && own) {
        r0 = value(src, lane);
        r1 = value(src, lane + half);
    }
    if ((MODE & 2) && dst) {
        const float amax = wave_max(fmaxf(fabsf(r0), fabsf(r1)));
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        const size_t kv_dim = (size_t)n_head_kv * head_dim;
        // per-sequence caches: sequence b's region starts kv_stride elements (kv_stride / head_dim scales) further on
        // hm != 0: head-major regions, [kv head][hm positions][head_dim] (scales [kv head][hm]); else [position][kv head][head_dim]
        int8_t* row = dst + (size_t)b * kv_stride +
                      (hm ? ((size_t)kvh * hm + pos) * head_dim : (size_t)pos * kv_dim + (size_t)kvh * head_dim);
        if (own) {
            row[lane] = (int8_t)(int)fminf(fmaxf(rintf(r0 * inv), -127.0f), 127.0f);
            row[lane + half] = (int8_t)(int)fminf(fmaxf(rintf(r1 * inv), -127.0f), 127.0f);
        }
        if (lane == 0)
            sdst[(size_t)b * (kv_stride / head_dim) + (hm ? (size_t)kvh * hm + pos : (size_t)pos * n_head_kv + kvh)] = amax / 127.0f;
    }
}

// ------------------------------------------------------- decode attention
// out[b, h, :] = bf16( softmax_t( q[b,h] . (K8[t] * sk[t]) * scale ) . (V8[t] * sv[t]) ),
// t in [0, seq_len), GQA: kv head = h / ratio.
// Workgroup = (kv head, sequence b), 256 lanes; the `ratio` query heads of the
// group are processed together.  Per 256-position tile:
//   phase 1  lane = position: dot(q_h, K[t]) for every head of the group (K row read once)
//   phase 2  online softmax bookkeeping per head (running max m, sum l)
//   phase 3  wave = head (round robin), lane = 2 output dims: acc += p[t] * V[t]
constexpr int ATT_TILE = 256;
constexpr int ATT_MAX_RATIO = 16;

__global__ __launch_bounds__(256) void attn_decode_kernel(const float* __restrict__ q, const int8_t* __restrict__ ck,
                                                          const int8_t* __restrict__ cv, const float* __restrict__ sk,
                                                          const float* __restrict__ sv, uint16_t* __restrict__ out,
                                                          const int* __restrict__ positions, int seq_len_arg,
                                                          int n_head, int n_head_kv, int head_dim, float scale,
                                                          size_t kv_stride, int hm)
{
    extern __shared__ float smem[];
    const int ratio = n_head / n_head_kv;
    float* qs = smem;                                   // [ratio][head_dim]
    float* ps = qs + ratio * head_dim;                  // [ratio][ATT_TILE] scores / probabilities
    float* red = ps + ratio * ATT_TILE;                 // [17]
    float* stat = red + 17;                             // [ratio][2]: running max, tile rescale
    const int kvh = blockIdx.x, b = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int seq_len = positions ? positions[b] + 1 : seq_len_arg;
    const size_t kv_dim = hm ? (size_t)head_dim : (size_t)n_head_kv * head_dim;   // distance between the rows of consecutive positions
    const size_t hoff = hm ? (size_t)kvh * hm * head_dim : (size_t)kvh * head_dim;
    const int ssr = hm ? 1 : n_head_kv;                  // distance between the scales of consecutive positions
    const int8_t* kbase = ck + (size_t)b * kv_stride + hoff;
    const int8_t* vbase = cv + (size_t)b * kv_stride + hoff;
    const size_t sstride = kv_stride / head_dim;        // scale arrays: kv_stride / head_dim per sequence
    const float* skb = sk + (size_t)b * sstride + (hm ? (size_t)kvh * hm : (size_t)kvh);
    const float* svb = sv + (size_t)b * sstride + (hm ? (size_t)kvh * hm : (size_t)kvh);
    const float* qb = q + (size_t)b * n_head * head_dim + (size_t)kvh * ratio * head_dim;

    for (int i = tid; i < ratio * head_dim; i += 256) qs[i] = qb[i];
    if (tid < ratio) stat[2 * tid] = -1e30f;
    __syncthreads();

    // per-head running sums live in the lanes that own the output: wave w owns heads w, w+4, ...
    constexpr int MAX_OWN = ATT_MAX_RATIO / 4;
    float o0[MAX_OWN], o1[MAX_OWN], lsum[MAX_OWN];
#pragma unroll
    for (int j = 0; j < MAX_OWN; j++) o0[j] = o1[j] = lsum[j] = 0.0f;
    const int nd2 = head_dim >> 1;                      // lanes cover dims 2*lane, 2*lane+1 (+128 per extra pass)

    for (int t0 = 0; t0 < seq_len; t0 += ATT_TILE) {
        const int tl = min(ATT_TILE, seq_len - t0);
        // phase 1: scores
        if (tid < tl) {
            const int t = t0 + tid;
            const int8_t* kr = kbase + (size_t)t * kv_dim;
            const float kscale = skb[(size_t)t * ssr] * scale;
            float dot[ATT_MAX_RATIO];
#pragma unroll
            for (int h = 0; h < ATT_MAX_RATIO; h++) dot[h] = 0.0f;
            for (int d = 0; d < head_dim; d += 16) {
                const uint4 kk = *(const uint4*)(kr + d);
                const uint32_t w4[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const float kv = (float)(int8_t)((w4[e >> 2] >> (8 * (e & 3))) & 0xFF);
#pragma unroll
                    for (int h = 0; h < ATT_MAX_RATIO; h++)
                        if (h < ratio) dot[h] += qs[h * head_dim + d + e] * kv;
                }
            }
#pragma unroll
            for (int h = 0; h < ATT_MAX_RATIO; h++)
                if (h < ratio) ps[h * ATT_TILE + tid] = dot[h] * kscale;
        }
        __syncthreads();
        // phase 2: per head tile max -> new running max, rescale factor, probabilities
        for (int h = 0; h < ratio; h++) {
            const float sc = tid < tl ? ps[h * ATT_TILE + tid] : -1e30f;
            const float tmax = block_reduce<true>(sc, red);
            const float m_old = stat[2 * h];
            const float m_new = fmaxf(m_old, tmax);
            if (tid < tl) ps[h * ATT_TILE + tid] = expf(sc - m_new);
            __syncthreads();                             // everyone has read m_old
            if (tid == 0) {
                stat[2 * h] = m_new;
                stat[2 * h + 1] = expf(m_old - m_new);
            }
        }
        __syncthreads();
        // phase 3: P.V for the heads this wave owns
#pragma unroll
        for (int j = 0; j < MAX_OWN; j++) {
            const int h = wave + 4 * j;
            if (h < ratio) {
                const float corr = stat[2 * h + 1];
                float a0 = o0[j] * corr, a1 = o1[j] * corr, ls = lsum[j] * corr;
                if (lane < nd2) {
                    for (int t = 0; t < tl; t++) {
                        const float pv = ps[h * ATT_TILE + t];
                        const float w = pv * svb[(size_t)(t0 + t) * ssr];
                        const uint16_t two = *(const uint16_t*)(vbase + (size_t)(t0 + t) * kv_dim + 2 * lane);
                        a0 += w * (float)(int8_t)(two & 0xFF);
                        a1 += w * (float)(int8_t)(two >> 8);
                        ls += pv;
                    }
                }
                o0[j] = a0;
                o1[j] = a1;
                lsum[j] = ls;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < MAX_OWN; j++) {
        const int h = wave + 4 * j;
        if (h < ratio && lane < nd2) {
            const float inv = 1.0f / lsum[j];
            uint16_t* o = out + (size_t)b * n_head * head_dim + (size_t)(kvh * ratio + h) * head_dim + 2 * lane;
            *(uint32_t*)o = t12_f32_to_bf16(o0[j] * inv) | ((uint32_t)t12_f32_to_bf16(o1[j] * inv) << 16);
        }
    }
}

// ---- fast decode attention for the common shapes (head_dim 64 / 128, GQA ratio 1/2/4/8) ----
// Same function as attn_decode_kernel, per tile of 256 positions, in one of two forms.
// WIDE = true (the default), both products on the matrix cores with INT8 operands:
//   phase 1  Q split into three INT8 limbs per element (rows 8 * limb + head of the A operand), K rows
//            as stored = B operand; v_mfma_i32_32x32x32_i8, exact int32 sums, 64 positions per wave;
//   phase 2  one wave per query head: tile max, exp, sum with wave reductions only; the weights
//            p * v_scale of the tile go to LDS as two INT8 limbs;
//   phase 3  out[head, dim] += w . V: V staged 128 positions at a time in LDS and read back
//            transposed (ds_read_b64_tr_b8), one wave per 32 dims, again v_mfma_i32_32x32x32_i8;
//   every tile's K rows, V rows and scales are requested one tile ahead.
// WIDE = false, the first form, kept for comparison (t12_tune_attention(3)):
//   phase 1  lane = position: the K row is fetched with HD/16 128-bit loads issued together,
//            then dotted with the RATIO query vectors broadcast from LDS (fp32 FMAs);
//   phase 2  as above, without the limbs;
//   phase 3  the same wave: P.V with 128-bit V loads -- 8 (HD=128) or 4 (HD=64) lanes span one
//            position, so one load instruction covers 8 / 16 positions; each lane keeps 16
//            output dims for its position class, classes are folded by xor shuffles at the end.
// SPLIT: see AttnSplit.
// FUSE: the kernel first does what rope_kv_kernel<3> does for its own heads -- rotates the
// RATIO query heads while loading them, rotates this KV head's new K, quantises K and V to
// INT8 and stores them at position pos -- and only then attends over positions 0..pos.
// (All B workgroups of a shared cache, kv_stride = 0, store identical values into one slot.)
// hm (all cache-touching kernels): 0 = a cache region is [position][kv head][dim] with scales [position][kv head], the
// reference's layout; hm > 0 = head-major regions of hm positions, [kv head][hm][dim] with scales [kv head][hm], in which
// the rows one workgroup reads are contiguous.
struct AttnFuse {
    const float* k_new;      // [B, n_head_kv * HD] fp32, unrotated
    const float* v_new;
    int8_t* ck_w;            // writable views of the caches / scales
    int8_t* cv_w;
    float* sk_w;
    float* sv_w;
    const float* freqs;      // [HD / 2]
};

// Context split (gridDim.z > 1): workgroup z attends over positions [z * chunk_len, (z + 1) * chunk_len) only and
// leaves, per query head, its running maximum m, its sum l and its unnormalised 128 outputs in
// ws[((b * n_head_kv + kvh) * nchunk + z) * RATIO + h][HD + 4] (m at [HD], l at [HD + 1]); the workgroup that finishes last for (b, kvh)
// (counter[b * n_head_kv + kvh], which it resets to 0) folds the chunks: out = sum_z e^(m_z - M) acc_z /
// sum_z e^(m_z - M) l_z.  One sequence at a long context otherwise occupies n_head_kv workgroups of the chip.
struct AttnSplit {
    float* ws;
    int* counter;
    int chunk_len;
};

template <int HD, int RATIO, bool FUSE = false, bool SPLIT = false, bool WIDE = false>
__global__ __launch_bounds__(256, FUSE ? 1 : (WIDE ? 3 : 4)) void attn_fast_kernel(const float* __restrict__ q, const int8_t* __restrict__ ck,
                                                        const int8_t* __restrict__ cv, const float* __restrict__ sk,
                                                        const float* __restrict__ sv, uint16_t* __restrict__ out,
                                                        const int* __restrict__ positions, int seq_len_arg,
                                                        int n_head_kv, float scale, size_t kv_stride, AttnFuse fz,
                                                        AttnSplit sp, int hm)
{
    constexpr int CH = HD / 16;                 // lanes per position in phase 3
    constexpr int PG = 64 / CH;                 // positions per load instruction
    constexpr int OWN = (RATIO + 3) / 4;        // heads per wave
    __shared__ float qs[RATIO * HD];
    __shared__ float ps[RATIO * ATT_TILE];
    const int kvh = blockIdx.x, b = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int seq_len = positions ? positions[b] + 1 : seq_len_arg;
    const int n_head = n_head_kv * RATIO;
    const size_t kv_dim = (size_t)n_head_kv * HD;
    const size_t rstride = hm ? (size_t)HD : kv_dim;     // distance between the cache rows of consecutive positions
    const size_t hoff = hm ? (size_t)kvh * hm * HD : (size_t)kvh * HD;
    const int ssr = hm ? 1 : n_head_kv;                  // distance between the scales of consecutive positions
    const int8_t* kbase = ck + (size_t)b * kv_stride + hoff;
    const int8_t* vbase = cv + (size_t)b * kv_stride + hoff;
    const size_t sstride = kv_stride / HD;
    const float* skb = sk + (size_t)b * sstride + (hm ? (size_t)kvh * hm : (size_t)kvh);
    const float* svb = sv + (size_t)b * sstride + (hm ? (size_t)kvh * hm : (size_t)kvh);
    const float* qb = q + (size_t)b * n_head * HD + (size_t)kvh * RATIO * HD;
    // this workgroup's share of the context
    const int nchunk = SPLIT ? gridDim.z : 1;
    const int c0 = SPLIT ? (int)blockIdx.z * sp.chunk_len : 0;
    const int c1 = SPLIT ? min(seq_len, c0 + sp.chunk_len) : seq_len;

    // FUSE: the cache rows of the first tile are requested before anything else, so that their HBM
    // latency runs under the Q / new-K / new-V work instead of behind it: this lane's K row (phase 1)
    // into registers and the V tile through registers into LDS (phase 3 reads it from there).  The row of the position being written (FUSE) is not in memory yet: it comes from LDS.
    constexpr bool VLDS = FUSE && !WIDE;                            // (the long-context form stages V itself, tile by tile)
    constexpr int VPRE = VLDS ? (ATT_TILE * CH) / 256 : 0;          // 16-byte V pieces per thread
    __shared__ __attribute__((aligned(16))) int8_t vt[VLDS ? ATT_TILE * HD : 16];
    __shared__ float vts[VLDS ? ATT_TILE : 1];
    __shared__ __attribute__((aligned(16))) int8_t knew8[FUSE ? HD : 16];
    __shared__ float knew_scale;
    const int tl0 = min(ATT_TILE, c1 - c0);
    const int newpos = FUSE ? seq_len - 1 : -1;
    const bool store_new = FUSE && c1 == seq_len;         // the chunk that holds the position being written
    // one-wave-per-head form: thread = position, the whole K row in registers
    const bool kpre_n = !WIDE && FUSE && tid < tl0 && c0 + tid != newpos;    // (many small workgroups per CU without FUSE: the registers cost more than the latency)
    uint4 kk_pre_n[CH];
    float kscale_pre_n = 0.0f;
    if (kpre_n) {
        const uint4* kr = (const uint4*)(kbase + (size_t)(c0 + tid) * rstride);
#pragma unroll
        for (int u = 0; u < CH; u++) kk_pre_n[u] = kr[u];
        kscale_pre_n = skb[(size_t)(c0 + tid) * ssr] * scale;
    }
    // Phase 1 layout: wave w scores positions 64 w .. 64 w + 63 of a tile in two blocks of 32; lane (ln, lh) of
    // block nb holds half lh of the K row of position 64 w + 32 nb + ln: HD / 2 contiguous bytes = KS pieces
    // of 16, the B operand of KS v_mfma_i32_32x32x32_i8 steps (the dims are consumed in this permuted order on
    // both operands).
    constexpr int KS = HD / 32;
    const int ln = lane & 31, lh = lane >> 5;
    typedef int t12_i32x4 __attribute__((ext_vector_type(4)));
    typedef int t12_i32x16 __attribute__((ext_vector_type(16)));
    uint4 kk_pre[2][KS];
    float kscale_pre[2] = {0.0f, 0.0f};
    bool kpre[2] = {false, false};
    if (FUSE && WIDE) {
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const int tp = wave * 64 + nb * 32 + ln;             // position inside the first tile
            kpre[nb] = tp < tl0 && c0 + tp != newpos;
            if (kpre[nb]) {
                const uint4* kr = (const uint4*)(kbase + (size_t)(c0 + tp) * rstride + lh * (HD / 2));
#pragma unroll
                for (int u = 0; u < KS; u++) kk_pre[nb][u] = kr[u];
                kscale_pre[nb] = skb[(size_t)(c0 + tp) * ssr];     // as stored; multiplied where it is used
            }
        }
    }
    uint4 v_pre[VPRE > 0 ? VPRE : 1];
    float vs_pre = 0.0f;
    if (VLDS) {
#pragma unroll
        for (int x = 0; x < VPRE; x++) {
            const int idx = tid + 256 * x, t = idx / CH, u = idx % CH;
            v_pre[x] = make_uint4(0, 0, 0, 0);
            if (t < tl0 && c0 + t != newpos) v_pre[x] = *(const uint4*)(vbase + (size_t)(c0 + t) * rstride + u * 16);
        }
        if (tid < tl0 && c0 + tid != newpos) vs_pre = svb[(size_t)(c0 + tid) * ssr];
    }

    constexpr int QSTR = HD + 16;               // row pitch of qlimb, for the same reason as WSTR
    // QREG (four query heads of 128 dims): wave w holds head w's 128 values in registers, two per lane -- the fused form
    // has just rotated them there, the other form loads them that way -- and derives the head's limbs there and then,
    // without the round trip through qs and its barrier; the rows it writes are left out of the clearing below (other
    // threads' zeros and this wave's limbs would race).
    constexpr bool QREG = WIDE && RATIO == 4 && HD == 128;
    __shared__ __attribute__((aligned(16))) int8_t qlimb[WIDE ? 32 * QSTR : 16];
    __shared__ float qscale[RATIO];
    constexpr int WSTR = ATT_TILE + 16;         // row pitch of wq: 32 lanes reading 16 bytes of 32 different rows, no bank shared
    __shared__ __attribute__((aligned(16))) int8_t wq[WIDE ? 32 * WSTR : 16];
    if constexpr (WIDE) {
        // both operand buffers are cleared here, under the latency of the requests above (the rows no head writes must
        // read as zero); the barrier behind the Q loads covers them
        for (int i = tid; i < 32 * QSTR / 16; i += 256) {
            const int row = i / (QSTR / 16);
            if (!QREG || (row & 7) >= RATIO || row >= 24) ((uint4*)qlimb)[i] = make_uint4(0, 0, 0, 0);
        }
        for (int i = tid; i < 32 * WSTR / 16; i += 256) ((uint4*)wq)[i] = make_uint4(0, 0, 0, 0);
    }
    // head `wave`, values q0 = dim lane and q1 = dim lane + 64: s_h = max|q_h| / 127 and the three limbs (see below)
    auto limbs_from_registers = [&](float q0, float q1) __attribute__((always_inline)) {
        const int h = wave;
        const float amaxq = wave_max(fmaxf(fabsf(q0), fabsf(q1)));
        const float invq = amaxq > 0.0f ? 127.0f / amaxq : 0.0f;
        auto limbs = [&](float qv, int dd) {
            const float s0 = qv * invq;
            const float a1 = fminf(fmaxf(rintf(s0), -127.0f), 127.0f);
            const float s1 = (s0 - a1) * 254.0f;
            const float a2 = fminf(fmaxf(rintf(s1), -127.0f), 127.0f);
            const float a3 = fminf(fmaxf(rintf((s1 - a2) * 254.0f), -127.0f), 127.0f);
            qlimb[h * QSTR + dd] = (int8_t)(int)a1;
            qlimb[(8 + h) * QSTR + dd] = (int8_t)(int)a2;
            qlimb[(16 + h) * QSTR + dd] = (int8_t)(int)a3;
        };
        limbs(q0, lane);
        limbs(q1, lane + 64);
        if (lane == 0) qscale[h] = amaxq / 127.0f;
    };
    if (!FUSE) {
        if constexpr (QREG) {
            limbs_from_registers(qb[wave * HD + lane], qb[wave * HD + lane + 64]);
        } else {
            for (int i = tid; i < RATIO * HD; i += 256) qs[i] = qb[i];
        }
    } else {
        constexpr int HALF = HD / 2;
        static_assert(256 % HALF == 0, "a thread keeps one rotation angle");
        const int pos = seq_len - 1;
        // everything this part needs is requested in one go -- the frequency of the thread's dim pair d = tid % HALF
        // (the same d in every pass of the Q loop, and the new K row's d in wave 0), the thread's first Q pair, the new
        // K / V row -- and the angle is worked out once: one round trip instead of one per step
        const int d = tid % HALF;
        const float freq = fz.freqs[d];
        const bool qfirst = tid < RATIO * HALF;
        float qx0 = 0.0f, qx1 = 0.0f;
        if (qfirst) {
            qx0 = qb[(tid / HALF) * HD + d];
            qx1 = qb[(tid / HALF) * HD + d + HALF];
        }
        const bool own = lane < HALF;
        float r0 = 0.0f, r1 = 0.0f;
        if (wave < 2 && store_new && own) {
            const float* src = (wave == 0 ? fz.k_new : fz.v_new) + (size_t)b * kv_dim + (size_t)kvh * HD;
            r0 = src[lane];
            r1 = src[lane + HALF];
        }
        float sn, cs;
        sincosf((float)pos * freq, &sn, &cs);
        if constexpr (QREG) {
            float q0, q1;
            rope_rotate(qx0, qx1, sn, cs, q0, q1);
            limbs_from_registers(q0, q1);
        } else if (qfirst) {
            rope_rotate(qx0, qx1, sn, cs, qs[(tid / HALF) * HD + d], qs[(tid / HALF) * HD + d + HALF]);
        }
        for (int i = tid + 256; i < RATIO * HALF; i += 256) {        // (more than 256 pairs: GQA ratios above 4 at head_dim 128)
            const int h = i / HALF;
            const float x0 = qb[h * HD + d], x1 = qb[h * HD + d + HALF];
            rope_rotate(x0, x1, sn, cs, qs[h * HD + d], qs[h * HD + d + HALF]);
        }
        if (wave < 2 && store_new) {                                 // wave 0: K (rotated), wave 1: V
            if (own && wave == 0) {
                const float x0 = r0, x1 = r1;
                rope_rotate(x0, x1, sn, cs, r0, r1);
            }
            const float amax = wave_max(fmaxf(fabsf(r0), fabsf(r1)));
            const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            int8_t* row = (wave == 0 ? fz.ck_w : fz.cv_w) + (size_t)b * kv_stride + hoff + (size_t)pos * rstride;
            const int8_t q0 = (int8_t)(int)fminf(fmaxf(rintf(r0 * inv), -127.0f), 127.0f);
            const int8_t q1 = (int8_t)(int)fminf(fmaxf(rintf(r1 * inv), -127.0f), 127.0f);
            // the new row: to the cache, and (first tile) to LDS where this launch reads it
            const int rel = pos - c0;                                // position inside this chunk
            int8_t* lrow = wave == 0 ? knew8 : vt + (size_t)(VLDS && rel < ATT_TILE ? rel : 0) * HD;
            const bool to_lds = wave == 0 || (VLDS && rel < ATT_TILE);
            if (own) {
                row[lane] = q0;
                row[lane + HALF] = q1;
                if (to_lds) {
                    lrow[lane] = q0;
                    lrow[lane + HALF] = q1;
                }
            }
            if (lane == 0) {
                (wave == 0 ? fz.sk_w : fz.sv_w)[(size_t)b * sstride + (hm ? (size_t)kvh * hm + pos : (size_t)pos * n_head_kv + kvh)] = amax / 127.0f;
                if (wave == 0) knew_scale = amax / 127.0f;
                else if (VLDS && rel < ATT_TILE) vts[rel] = amax / 127.0f;
            }
        }
        // later tiles read the new row back through the cache pointers: only this workgroup does (the chunk that
        // stores the row is the chunk that holds it), so workgroup scope is enough -- a device-scope fence here
        // writes back and invalidates the L2 in every launch
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
        // the prefetched V tile: registers -> LDS (row-major, 16-byte pieces)
#pragma unroll
        for (int x = 0; x < VPRE; x++) {
            const int idx = tid + 256 * x, t = idx / CH;
            if (t < tl0 && c0 + t != newpos) ((uint4*)vt)[idx] = v_pre[x];
        }
        if (VLDS && tid < tl0 && c0 + tid != newpos) vts[tid] = vs_pre;
    }
    __syncthreads();

    // Q as three INT8 limbs per element, q ~ s_h (a1 + a2 / 254 + a3 / 254^2) with s_h = max|q_h| / 127 (error <=
    // 6e-8 max|q_h|: fp32 level, also for heads with outlier dims), laid out as the A operand of the score MFMAs: row
    // 8 * limb + h (the 32 rows of the MFMA are there anyway).
    // INT8 x INT8 products accumulate exactly in int32, so K needs no conversion at all.
    // (qlimb was cleared ahead of the Q loads, under their latency; the barrier above covers it)
    if constexpr (WIDE && !QREG) {
    for (int h = wave; h < RATIO; h += 4) {
        float amax = 0.0f;
        for (int d = lane; d < HD; d += 64) amax = fmaxf(amax, fabsf(qs[h * HD + d]));
        amax = wave_max(amax);
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        for (int d = lane; d < HD; d += 64) {
            const float r0 = qs[h * HD + d] * inv;
            const float a1 = fminf(fmaxf(rintf(r0), -127.0f), 127.0f);
            const float r1 = (r0 - a1) * 254.0f;
            const float a2 = fminf(fmaxf(rintf(r1), -127.0f), 127.0f);
            const float a3 = fminf(fmaxf(rintf((r1 - a2) * 254.0f), -127.0f), 127.0f);
            qlimb[h * QSTR + d] = (int8_t)(int)a1;
            qlimb[(8 + h) * QSTR + d] = (int8_t)(int)a2;
            qlimb[(16 + h) * QSTR + d] = (int8_t)(int)a3;
        }
        if (lane == 0) qscale[h] = amax / 127.0f;
    }
    __syncthreads();
    }
    const int8_t* qa_src = qlimb + ln * QSTR + lh * (HD / 2);      // this lane's A operand pieces (re-read per tile: 4 LDS loads)

    // running maximum / sum of head h live in the wave that owns it (h % 4); the output sums of ALL heads live
    // in every wave, over the 64 positions of each tile that the wave takes in phase 3
    constexpr int NACC = WIDE ? 1 : OWN;
    float m_run[OWN], l_run[OWN], acc[NACC][16];
#pragma unroll
    for (int j = 0; j < OWN; j++) {
        m_run[j] = -1e30f;
        l_run[j] = 0.0f;
    }
#pragma unroll
    for (int h = 0; h < NACC; h++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[h][e] = 0.0f;
    __shared__ float corr_s[RATIO];
    // Long-context form, P.V phase: out[h, d] = sum_t w[h, t] V8[t, d] with w = p * v_scale, again as INT8 MFMAs: w in two
    // INT8 limbs per (head, position) (rows 8 * limb + h of wq), V staged 128 positions at a time in LDS (rows padded to
    // VSTR bytes: conflict-free) and read back TRANSPOSED (ds_read_b64_tr_b8: inside 16 lanes, lane 8 par + c receives
    // byte c of the rows that lanes par, 2 + par, ... 14 + par point at), which is the B operand: 16 consecutive
    // positions of one dim per lane.  Wave w owns dims 32 w .. 32 w + 31; lane (ln, lh) ends with heads 4 lh .. 4 lh + 3 of
    // dim 32 w + ln in o_w[].
    constexpr int VSTR = HD + 16;
    constexpr int NBLK = HD / 32;               // dim blocks = waves busy in this phase
    __shared__ __attribute__((aligned(16))) int8_t vth[WIDE ? 128 * VSTR : 16];
    __shared__ float wscale_s[RATIO];
    float o_w[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int VP = WIDE ? 128 * CH / 256 : 1;   // 16-byte V pieces per thread and half tile
    t12_u32x4 vreg[VP];     // (a native vector type: the compiler keeps this loop-carried array in registers)
    float vsc[OWN][ATT_TILE / 64], vsc_n[OWN][ATT_TILE / 64];
    uint4 kk[2][WIDE ? KS : 1];
    float kscale[2] = {0.0f, 0.0f};      // K scales as loaded: nothing touches a requested value before its tile comes up
    // Requests of the long-context form.  Every tile's K rows, V scales and first 128 V rows are asked for one tile
    // ahead (the registers they land in are free by then), its other 128 V rows during its softmax phase: no
    // memory latency stays exposed inside a workgroup.
    auto issue_k = [&](int t0x, int tlx, bool first) __attribute__((always_inline)) {
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const int tp = wave * 64 + nb * 32 + ln;                 // position inside the tile
            if (wave * 64 + nb * 32 < tlx) {                         // wave-uniform: the block holds positions
                const int t = t0x + min(tp, tlx - 1);                // rows past the end repeat the last one (masked in phase 2)
                if (first && kpre[nb]) {
#pragma unroll
                    for (int u = 0; u < KS; u++) kk[nb][u] = kk_pre[nb][u];
                    kscale[nb] = kscale_pre[nb];
                } else if (FUSE && first && t == newpos) {
#pragma unroll
                    for (int u = 0; u < KS; u++) kk[nb][u] = ((const uint4*)(knew8 + lh * (HD / 2)))[u];
                    kscale[nb] = knew_scale;
                } else {
                    const uint4* kr = (const uint4*)(kbase + (size_t)t * rstride + lh * (HD / 2));
#pragma unroll
                    for (int u = 0; u < KS; u++) kk[nb][u] = kr[u];
                    kscale[nb] = skb[(size_t)t * ssr];
                }
            }
        }
    };
    auto issue_v = [&](int t0x, int tlx, int half) __attribute__((always_inline)) {
#pragma unroll
        for (int x = 0; x < VP; x++) {
            const int idx = tid + 256 * x, t = min(half * 128 + idx / CH, tlx - 1), u = idx % CH;
            vreg[x] = *(const t12_u32x4*)(vbase + (size_t)(t0x + t) * rstride + u * 16);
        }
    };
    auto issue_vsc = [&](int t0x, int tlx, float (&dst)[OWN][ATT_TILE / 64]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < OWN; j++)
#pragma unroll
            for (int i = 0; i < ATT_TILE / 64; i++) {
                const int t = lane + 64 * i;
                dst[j][i] = (wave + 4 * j < RATIO && t < tlx) ? svb[(size_t)(t0x + t) * ssr] : 0.0f;
            }
    };
    const int g = lane / CH, c = lane % CH;     // phase 3: position class, 16-dim chunk
    if constexpr (WIDE) {
        issue_k(c0, tl0, true);
        issue_vsc(c0, tl0, vsc);
        issue_v(c0, tl0, 0);
    }

    // One tile.  full_c = std::true_type: this tile and the next one are complete, so every request of the tile is issued
    // without a condition around it.  (The compiler counts outstanding loads per path: behind a load that sits under a
    // condition it must assume that none of the later ones was issued, and then waits for all of them.)
    auto tile = [&](const int t0, auto full_c) __attribute__((always_inline)) {
        constexpr bool FULLT = decltype(full_c)::value;
        const int tl = FULLT ? ATT_TILE : min(ATT_TILE, c1 - t0);
        const int t0n = t0 + ATT_TILE;
        const bool has_next = FULLT || t0n < c1;
        const int tln = FULLT ? ATT_TILE : min(ATT_TILE, c1 - t0n);
        if constexpr (WIDE) {
        // ---- phase 1: scores of 64 positions per wave, two blocks of 32, KS INT8 MFMAs each
        // (the K rows, V rows and V scales of this tile were requested during the previous tile, or before the loop)
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const int tp = wave * 64 + nb * 32 + ln;
            if (FULLT || wave * 64 + nb * 32 < tl) {
                t12_i32x16 sacc;
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[r] = 0;
#pragma unroll
                for (int u = 0; u < KS; u++)
                    sacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(*(const t12_i32x4*)(qa_src + 16 * u),
                                                                 __builtin_bit_cast(t12_i32x4, kk[nb][u]), sacc, 0, 0, 0);
                // lane (ln, lh) holds column ln = its position; rows 4 lh + r (limb 0), 8 + 4 lh + r (limb 1) and
                // 16 + 4 lh + r (limb 2), r = 0..3: heads 4 lh .. 4 lh + 3
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int h = 4 * lh + r;
                    if (h < RATIO)
                        ps[h * ATT_TILE + tp] = ((float)sacc[r] + ((float)sacc[4 + r] + (float)sacc[8 + r] * (1.0f / 254.0f)) *
                                                                      (1.0f / 254.0f)) * (qscale[h] * (kscale[nb] * scale));
                }
            }
        }
        } else {
        // ---- phase 1
        if (tid < tl) {
            const int t = t0 + tid;
            uint4 kk[CH];
            float kscale;
            if (t0 == c0 && kpre_n) {
#pragma unroll
                for (int u = 0; u < CH; u++) kk[u] = kk_pre_n[u];
                kscale = kscale_pre_n;
            } else if (FUSE && t == newpos && t0 == c0) {
#pragma unroll
                for (int u = 0; u < CH; u++) kk[u] = ((const uint4*)knew8)[u];
                kscale = knew_scale * scale;
            } else {
                const uint4* kr = (const uint4*)(kbase + (size_t)t * rstride);
#pragma unroll
                for (int u = 0; u < CH; u++) kk[u] = kr[u];
                kscale = skb[(size_t)t * ssr] * scale;
            }
            float dot[RATIO];
#pragma unroll
            for (int h = 0; h < RATIO; h++) dot[h] = 0.0f;
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const uint32_t w4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const float kv = (float)(int8_t)((w4[e >> 2] >> (8 * (e & 3))) & 0xFF);
#pragma unroll
                    for (int h = 0; h < RATIO; h++) dot[h] += qs[h * HD + u * 16 + e] * kv;
                }
            }
#pragma unroll
            for (int h = 0; h < RATIO; h++) ps[h * ATT_TILE + tid] = dot[h] * kscale;
        }
        }
        if constexpr (WIDE) {
            // ---- V, first 128 positions of the tile: registers -> LDS (rows past the end repeat the last one; their
            //      weights are zero)
#pragma unroll
            for (int x = 0; x < VP; x++) {
                const int idx = tid + 256 * x;
                *(t12_u32x4*)(vth + (idx / CH) * VSTR + (idx % CH) * 16) = vreg[x];
            }
            // requests, after the wait for this tile's V rows so that it does not cover them: the next tile's K rows and
            // V scales, and this tile's other 128 V rows, travel under the softmax phase
            if constexpr (FULLT) {
#pragma unroll
                for (int nb = 0; nb < 2; nb++) {
                    const int t = t0n + wave * 64 + nb * 32 + ln;
                    const uint4* kr = (const uint4*)(kbase + (size_t)t * rstride + lh * (HD / 2));
#pragma unroll
                    for (int u = 0; u < KS; u++) kk[nb][u] = kr[u];
                    kscale[nb] = skb[(size_t)t * ssr];
                }
#pragma unroll
                for (int j = 0; j < OWN; j++)
#pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const float s = svb[(size_t)(t0n + lane + 64 * i) * ssr];
                        vsc_n[j][i] = (RATIO % 4 == 0 || wave + 4 * j < RATIO) ? s : 0.0f;
                    }
#pragma unroll
                for (int x = 0; x < VP; x++) {
                    const int idx = tid + 256 * x;
                    vreg[x] = *(const t12_u32x4*)(vbase + (size_t)(t0 + 128 + idx / CH) * rstride + (idx % CH) * 16);
                }
            } else {
                if (has_next) {
                    issue_k(t0n, tln, false);
                    issue_vsc(t0n, tln, vsc_n);
                }
                if (128 < tl) issue_v(t0, tl, 1);
                else if (has_next) issue_v(t0n, tln, 0);             // (only the last tile of a chunk can be this short)
            }
            __syncthreads();
            // ---- phase 2, one wave per head: tile maximum, rescale factor, probabilities and their sum; the weights
            //      w = p * v_scale of the tile as two INT8 limbs, w ~ wscale (a1 + a2 / 254)
#pragma unroll
            for (int j = 0; j < OWN; j++) {
                const int h = wave + 4 * j;
                if (h < RATIO) {                                     // wave-uniform
                    float* ph = ps + h * ATT_TILE;
                    float sc[ATT_TILE / 64];
                    float tmax = -1e30f;
#pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const int t = lane + 64 * i;
                        sc[i] = t < tl ? ph[t] : -1e30f;
                        tmax = fmaxf(tmax, sc[i]);
                    }
                    tmax = wave_max(tmax);
                    const float m_new = fmaxf(m_run[j], tmax);
                    const float corr = expf(m_run[j] - m_new);
                    float psum = 0.0f, wv[ATT_TILE / 64], wmax = 0.0f;
#pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const int t = lane + 64 * i;
                        const float pv = t < tl ? expf(sc[i] - m_new) : 0.0f;
                        psum += pv;
                        wv[i] = pv * vsc[j][i];
                        wmax = fmaxf(wmax, wv[i]);
                    }
                    psum = wave_sum_dpp(psum);
                    wmax = wave_max(wmax);
                    const float inv = wmax > 0.0f ? 127.0f / wmax : 0.0f;
#pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const int t = lane + 64 * i;
                        const float r0 = wv[i] * inv;
                        const float a1 = fminf(rintf(r0), 127.0f);
                        const float a2 = fminf(fmaxf(rintf((r0 - a1) * 254.0f), -127.0f), 127.0f);
                        wq[h * WSTR + t] = (int8_t)(int)a1;
                        wq[(8 + h) * WSTR + t] = (int8_t)(int)a2;
                    }
                    l_run[j] = l_run[j] * corr + psum;
                    m_run[j] = m_new;
                    if (lane == 0) {
                        corr_s[h] = corr;
                        wscale_s[h] = wmax / 127.0f;
                    }
                }
            }
            __syncthreads();
            // ---- phase 3: two halves of 128 positions = 4 MFMA steps of 32 positions each
            t12_i32x16 oacc;
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[r] = 0;
            const int s16 = lane & 15;
            // transposed read: lane s16 = 2 j + par points at row j (a position), 8 dims from 8 par on, of its 16-dim group
            const int8_t* vsrc = vth + (s16 >> 1) * VSTR + wave * 32 + ((lane >> 4) & 1) * 16 + (s16 & 1) * 8;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                if (FULLT || half * 128 < tl) {                      // workgroup-uniform
                    if (half == 1) {
                        // second half of the tile through the same LDS rows
                        __syncthreads();                             // every wave is done with the first half
#pragma unroll
                        for (int x = 0; x < VP; x++) {
                            const int idx = tid + 256 * x;
                            *(t12_u32x4*)(vth + (idx / CH) * VSTR + (idx % CH) * 16) = vreg[x];
                        }
                        // the next tile's V scales were requested before the rows just written, so they are here:
                        // taken over now, nothing is left to wait for at the end of the tile
#pragma unroll
                        for (int j = 0; j < OWN; j++)
#pragma unroll
                            for (int i = 0; i < ATT_TILE / 64; i++) vsc[j][i] = vsc_n[j][i];
                        if constexpr (FULLT) {
#pragma unroll
                            for (int x = 0; x < VP; x++) {
                                const int idx = tid + 256 * x;
                                vreg[x] = *(const t12_u32x4*)(vbase + (size_t)(t0n + idx / CH) * rstride + (idx % CH) * 16);
                            }
                        } else if (has_next) issue_v(t0n, tln, 0);    // the next tile's first 128 V rows
                        __syncthreads();
                    }
                    if (wave < NBLK) {
#pragma unroll
                        for (int ks = 0; ks < 4; ks++) {
                            const t12_i32x4 wa = *(const t12_i32x4*)(wq + ln * WSTR + half * 128 + ks * 32 + 16 * lh);
                            typedef int t12_i32x2 __attribute__((ext_vector_type(2)));
                            typedef __attribute__((address_space(3))) t12_i32x2 lds_i32x2;
                            const t12_i32x2 b0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                                (lds_i32x2*)(vsrc + (ks * 32 + 16 * lh) * VSTR));
                            const t12_i32x2 b1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                                (lds_i32x2*)(vsrc + (ks * 32 + 16 * lh + 8) * VSTR));
                            t12_i32x4 vb;
                            vb[0] = b0[0]; vb[1] = b0[1]; vb[2] = b1[0]; vb[3] = b1[1];
                            oacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa, vb, oacc, 0, 0, 0);
                        }
                    }
                }
            }
            // lane (ln, lh): column = dim 32 wave + ln; rows 4 lh + r (limb 0) and 8 + 4 lh + r (limb 1) = heads 4 lh + r
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int h = min(4 * lh + r, RATIO - 1);
                o_w[r] = o_w[r] * corr_s[h] + ((float)oacc[r] + (float)oacc[4 + r] * (1.0f / 254.0f)) * wscale_s[h];
            }
            __syncthreads();                                         // (a tile of 128 positions or fewer is a chunk's last: no scales to take over)
        } else {
            __syncthreads();
            // ---- phases 2 + 3, one wave per head
    #pragma unroll
            for (int j = 0; j < OWN; j++) {
                const int h = wave + 4 * j;
                if (h < RATIO) {                                     // wave-uniform
                    float* ph = ps + h * ATT_TILE;
                    float sc[ATT_TILE / 64];
                    float tmax = -1e30f;
    #pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const int t = lane + 64 * i;
                        sc[i] = t < tl ? ph[t] : -1e30f;
                        tmax = fmaxf(tmax, sc[i]);
                    }
                    tmax = wave_max(tmax);
                    const float m_new = fmaxf(m_run[j], tmax);
                    const float corr = expf(m_run[j] - m_new);
                    float psum = 0.0f;
    #pragma unroll
                    for (int i = 0; i < ATT_TILE / 64; i++) {
                        const int t = lane + 64 * i;
                        const float pv = t < tl ? expf(sc[i] - m_new) : 0.0f;
                        if (t < tl) ph[t] = pv;
                        psum += pv;
                    }
                    psum = wave_sum_dpp(psum);
                    l_run[j] = l_run[j] * corr + psum;
                    m_run[j] = m_new;
    #pragma unroll
                    for (int e = 0; e < 16; e++) acc[j][e] *= corr;
                    // P.V: iteration it covers positions it*PG + g; loads of 4 iterations are issued together
                    for (int it = 0; it * PG < tl; it += 4) {
                        uint4 vv[4];
                        float w[4];
    #pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const int t = (it + x) * PG + g;
                            const bool ok = t < tl;
                            const int tc = ok ? t : 0;
                            if (FUSE && t0 == c0) {
                                vv[x] = ((const uint4*)vt)[tc * CH + c];
                                w[x] = ok ? ph[tc] * vts[tc] : 0.0f;
                            } else {
                                vv[x] = *(const uint4*)(vbase + (size_t)(t0 + tc) * rstride + c * 16);
                                w[x] = ok ? ph[tc] * svb[(size_t)(t0 + tc) * ssr] : 0.0f;
                            }
                        }
    #pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const uint32_t w4[4] = {vv[x].x, vv[x].y, vv[x].z, vv[x].w};
    #pragma unroll
                            for (int e = 0; e < 16; e++)
                                acc[j][e] += w[x] * (float)(int8_t)((w4[e >> 2] >> (8 * (e & 3))) & 0xFF);
                        }
                    }
                }
            }
            __syncthreads();
        }
    };
    {
        int t0 = c0;
        if constexpr (WIDE)
            for (; t0 + 2 * ATT_TILE <= c1; t0 += ATT_TILE) tile(t0, std::true_type{});
        for (; t0 < c1; t0 += ATT_TILE) tile(t0, std::false_type{});
    }
    if constexpr (WIDE) {
        // ---- every lane holds finished sums of its dim for up to four heads; the owners publish maximum and sum
        __shared__ float mstat[RATIO], lstat[RATIO];
#pragma unroll
        for (int j = 0; j < OWN; j++) {
            const int h = wave + 4 * j;
            if (h < RATIO && lane == 0) {
                mstat[h] = m_run[j];
                lstat[h] = l_run[j];
            }
        }
        __syncthreads();
        if (wave < NBLK) {
            const int d = wave * 32 + ln;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int h = 4 * lh + r;
                if (h < RATIO) {
                    if (SPLIT) {
                        float* pw = sp.ws + ((((size_t)b * n_head_kv + kvh) * nchunk + blockIdx.z) * RATIO + h) * (HD + 4);
                        pw[d] = o_w[r];
                        if (d == 0) {
                            pw[HD] = mstat[h];
                            pw[HD + 1] = lstat[h];
                        }
                    } else {
                        out[(size_t)b * n_head * HD + (size_t)(kvh * RATIO + h) * HD + d] = t12_f32_to_bf16(o_w[r] / lstat[h]);
                    }
                }
            }
        }
    } else {
    #pragma unroll
        for (int j = 0; j < OWN; j++) {
            const int h = wave + 4 * j;
            if (h < RATIO) {
    #pragma unroll
                for (int e = 0; e < 16; e++) {
                    float v = acc[j][e];
    #pragma unroll
                    for (int off = CH; off < 64; off <<= 1) v += __shfl_xor(v, off, T12_WAVE);   // fold position classes
                    acc[j][e] = v;
                }
                if (g == 0) {
                    if (SPLIT) {
                        float* pw = sp.ws + ((((size_t)b * n_head_kv + kvh) * nchunk + blockIdx.z) * RATIO + h) * (HD + 4);
    #pragma unroll
                        for (int e = 0; e < 16; e += 4)
                            *(float4*)(pw + c * 16 + e) = make_float4(acc[j][e], acc[j][e + 1], acc[j][e + 2], acc[j][e + 3]);
                        if (c == 0) {
                            pw[HD] = m_run[j];
                            pw[HD + 1] = l_run[j];
                        }
                    } else {
                        const float inv = 1.0f / l_run[j];
                        uint32_t o[8];
    #pragma unroll
                        for (int e = 0; e < 8; e++)
                            o[e] = t12_f32_to_bf16(acc[j][2 * e] * inv) | ((uint32_t)t12_f32_to_bf16(acc[j][2 * e + 1] * inv) << 16);
                        uint4* dst = (uint4*)(out + (size_t)b * n_head * HD + (size_t)(kvh * RATIO + h) * HD + c * 16);
                        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
                        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
                    }
                }
            }
        }
    }
    if (SPLIT) {
        // the workgroup that arrives last for this (sequence, KV head) folds the chunks
        // (one thread publishes for the workgroup: the barrier orders every wave's partial sums before its device-scope
        // release, and the last workgroup's single acquire before every wave's reads -- a device-scope fence writes back or
        // invalidates the L2, so four waves executing one each is four times the cost)
        __shared__ int s_last;
        __syncthreads();
        if (tid == 0)
            s_last = __hip_atomic_fetch_add(sp.counter + (size_t)b * n_head_kv + kvh, 1, __ATOMIC_RELEASE,
                                            __HIP_MEMORY_SCOPE_AGENT) == nchunk - 1;
        __syncthreads();
        if (s_last) {
            if (tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            __syncthreads();
            const float* pb = sp.ws + (((size_t)b * n_head_kv + kvh) * nchunk) * RATIO * (HD + 4);
            // weight of chunk z for head h: e^(m_z - M) / sum_z e^(m_z - M) l_z, built in ps (free by now)
            float* wz = ps;                                          // [RATIO][nchunk] maxima, then weights
            float* lz = ps + RATIO * nchunk;                         // [RATIO][nchunk] sums (2 * nchunk <= ATT_TILE)
            for (int i = tid; i < RATIO * nchunk; i += 256) {
                const int h = i / nchunk, z = i % nchunk;
                const float2 ml = *(const float2*)(pb + ((size_t)z * RATIO + h) * (HD + 4) + HD);
                wz[i] = ml.x;
                lz[i] = ml.y;
            }
            __syncthreads();
            if (tid < RATIO) {
                float mx = -1e30f;
                for (int z = 0; z < nchunk; z++) mx = fmaxf(mx, wz[tid * nchunk + z]);
                float den = 0.0f;
                for (int z = 0; z < nchunk; z++) {
                    const float w = expf(wz[tid * nchunk + z] - mx);
                    den += w * lz[tid * nchunk + z];
                    wz[tid * nchunk + z] = w;
                }
                const float inv = 1.0f / den;
                for (int z = 0; z < nchunk; z++) wz[tid * nchunk + z] *= inv;
            }
            __syncthreads();
            for (int i = tid; i < RATIO * HD / 4; i += 256) {         // four neighbouring outputs per thread
                const int h = i / (HD / 4), d = (i % (HD / 4)) * 4;
                float4 n = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll 8
                for (int z = 0; z < nchunk; z++) {
                    const float4 a = *(const float4*)(pb + ((size_t)z * RATIO + h) * (HD + 4) + d);
                    const float w = wz[h * nchunk + z];
                    n.x += w * a.x; n.y += w * a.y; n.z += w * a.z; n.w += w * a.w;
                }
                *(uint2*)(out + (size_t)b * n_head * HD + (size_t)(kvh * RATIO + h) * HD + d) =
                    make_uint2(t12_f32_to_bf16(n.x) | ((uint32_t)t12_f32_to_bf16(n.y) << 16),
                               t12_f32_to_bf16(n.z) | ((uint32_t)t12_f32_to_bf16(n.w) << 16));
            }
            if (tid == 0) sp.counter[(size_t)b * n_head_kv + kvh] = 0;
        }
    }
}

// ------------------------------------------------------------------ argmax
// Lowest index among equal maxima (the reference's tie rule depends on its
// thread layout, kernels.hip:103-118; exact ties between fp32 logits do not
// occur in practice).  NaN never wins, like the reference's strict '>'.
struct ArgPair {
    float v;
    int i;
};
__device__ __forceinline__ ArgPair better(ArgPair a, ArgPair b)
{
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}
__device__ __forceinline__ ArgPair block_argmax(ArgPair p, ArgPair* sh /* [4] */)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        ArgPair o;
        o.v = __shfl_xor(p.v, off, T12_WAVE);
        o.i = __shfl_xor(p.i, off, T12_WAVE);
        p = better(p, o);
    }
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = p;
    __syncthreads();
    ArgPair r = sh[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); w++) r = better(r, sh[w]);
    return r;
}

constexpr int ARG_CHUNKS = 64;

__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits, int n,
                                                          ArgPair* __restrict__ part)
{
    __shared__ ArgPair sh[4];
    const int row = blockIdx.y, chunk = blockIdx.x;
    const int per = (n + ARG_CHUNKS - 1) / ARG_CHUNKS;
    const int lo = chunk * per, hi = min(n, lo + per);
    const float* x = logits + (size_t)row * n;
    ArgPair p = {-INFINITY, 0x7FFFFFFF};
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const float v = x[i];
        if (v > p.v) { p.v = v; p.i = i; }
    }
    p = block_argmax(p, sh);
    if (threadIdx.x == 0) part[(size_t)row * ARG_CHUNKS + chunk] = p;
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const ArgPair* __restrict__ part, int* __restrict__ result)
{
    __shared__ ArgPair sh[1];
    ArgPair p = part[(size_t)blockIdx.x * ARG_CHUNKS + threadIdx.x];
    p = block_argmax(p, sh);
    if (threadIdx.x == 0) result[blockIdx.x] = p.i == 0x7FFFFFFF ? 0 : p.i;
}

// ---- library-owned device state.  RoPE tables: one per (device, head_dim, theta, scaling rule), built on first
//      use and kept until the process ends (a table is 256 bytes; none is ever freed, so a pointer handed to a launch
//      stays valid whatever other threads do).  Scratch of the argmax and of the context-split attention: one set per
//      (device, stream) -- launches on different streams may overlap and must not share partial results or arrival
//      counters; launches on one stream are ordered.  Guarded for use from several host threads; two host threads
//      that launch on the SAME stream still share that stream's scratch, like any other buffer they would share.
std::mutex g_mu;
struct RopeKey {
    int dev, head_dim;
    float theta, scale[4];
    bool operator<(const RopeKey& o) const { return memcmp(this, &o, sizeof(RopeKey)) < 0; }
};
std::map<RopeKey, float*> g_rope_tables;
struct StreamScratch {
    ArgPair* part = nullptr;       // argmax partials [part_rows][ARG_CHUNKS]
    int part_rows = 0;
    float* split_ws = nullptr;     // context-split attention: partial results
    int* split_cnt = nullptr;      //   and arrival counters (zero between launches)
};
std::map<std::pair<int, hipStream_t>, StreamScratch> g_scratch;

// Frequency scaling of the "llama3" kind (factor <= 0: none); set by launch_rope_scaling
float g_rope_scale[4] = {0.0f, 0.0f, 0.0f, 0.0f};

int current_device()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    return dev;
}

const float* rope_table(int head_dim, float theta)
{
    std::lock_guard<std::mutex> lock(g_mu);
    RopeKey key;
    memset(&key, 0, sizeof key);
    key.dev = current_device();
    key.head_dim = head_dim;
    key.theta = theta;
    memcpy(key.scale, g_rope_scale, sizeof key.scale);
    auto it = g_rope_tables.find(key);
    if (it != g_rope_tables.end()) return it->second;
    const int half = head_dim / 2;
    if (half < 1) return nullptr;
    std::vector<float> h(half);
    t12_rope_freqs(head_dim, theta, g_rope_scale[0], g_rope_scale[1], g_rope_scale[2], g_rope_scale[3], h.data());
    float* d = nullptr;
    if (hipMalloc((void**)&d, half * sizeof(float)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), half * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(d);
        return nullptr;
    }
    g_rope_tables[key] = d;
    return d;
}

// The argmax partial buffer of this (device, stream), grown on demand (the old one is freed: hipFree waits for
// the device, and only launches on this very stream ever read it).
ArgPair* argmax_scratch(int rows, hipStream_t st)
{
    std::lock_guard<std::mutex> lock(g_mu);
    StreamScratch& sc = g_scratch[{current_device(), st}];
    if (sc.part_rows < rows) {
        if (sc.part) (void)hipFree(sc.part);
        sc.part = nullptr;
        sc.part_rows = 0;
        const int want = rows < 256 ? 256 : rows;
        if (hipMalloc((void**)&sc.part, (size_t)want * ARG_CHUNKS * sizeof(ArgPair)) != hipSuccess) return nullptr;
        sc.part_rows = want;
    }
    return sc.part;
}

void report(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        t12_set_error("%s: %s", what, hipGetErrorString(e));
        fprintf(stderr, "turbo12: %s: %s\n", what, hipGetErrorString(e));
    }
}

template <int MODE>
void launch_rope_kv(float* q, float* k, const float* v, int8_t* ck, int8_t* cv, float* sk, float* sv,
                    const int* positions, int position, int head_dim, int n_head, int n_head_kv, int q_stride,
                    int k_stride, float theta, int batch, hipStream_t st, QkvPartials part = QkvPartials{nullptr, 0, 0, 0},
                    size_t kv_stride = 0, int hm = 0)
{
    const float* f = nullptr;
    if (MODE & 1) {
        f = rope_table(head_dim, theta);
        if (!f) { t12_set_error("rope: cannot build the frequency table"); return; }
    }
    if (head_dim > 128 || (head_dim & 1)) {
        t12_set_error("rope/kv-store: head_dim %d unsupported (even, <= 128)", head_dim);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    hipLaunchKernelGGL(rope_kv_kernel<MODE>, dim3(n_head + 2 * n_head_kv, batch), dim3(64), 0, st, q, k, v, ck, cv, sk,
                       sv, f, positions, position, head_dim, n_head, n_head_kv, q_stride, k_stride, part, kv_stride, hm);
    report("rope/kv-store");
}

// The kernel form in use (t12_tune_attention); one word, read once per launch.
//   bits 0..23: context split, fewest positions per chunk (0 = never split); bit 24: specialised kernels allowed;
//   bit 25: their fp32 FMA form instead of the INT8 MFMA form
std::atomic<int> g_attn_mode{256 | (1 << 24)};
#define g_attn_fast ((attn_mode_now & (1 << 24)) != 0)
#define g_attn_chunk (attn_mode_now & 0xFFFFFF)
#define g_attn_wide ((attn_mode_now & (1 << 25)) ? 0x7FFFFFFF : 0)

// Scratch of the context split: partial results of at most ATT_SPLIT_WGS workgroups and one
// counter per (sequence, KV head); the counters start at zero and every launch leaves them there.
constexpr int ATT_SPLIT_WGS = 512;     // also: at most ATT_TILE / 2 chunks per (sequence, KV head)
constexpr int ATT_SPLIT_HEADS = 4096;
constexpr int ATT_SPLIT_TARGET = 256;  // workgroups a split launch aims for

// The context-split scratch of this (device, stream); nullptr when it cannot be allocated.
StreamScratch* attn_split_scratch(hipStream_t st)
{
    std::lock_guard<std::mutex> lock(g_mu);
    StreamScratch& sc = g_scratch[{current_device(), st}];
    if (sc.split_ws) return &sc;
    const size_t ws_bytes = (size_t)ATT_SPLIT_WGS * 8 * (128 + 4) * sizeof(float);     // RATIO <= 8, HD <= 128
    float* ws = nullptr;
    int* cnt = nullptr;
    if (hipMalloc((void**)&ws, ws_bytes) != hipSuccess) return nullptr;
    if (hipMalloc((void**)&cnt, ATT_SPLIT_HEADS * sizeof(int)) != hipSuccess ||
        hipMemset(cnt, 0, ATT_SPLIT_HEADS * sizeof(int)) != hipSuccess) {
        (void)hipFree(ws);
        if (cnt) (void)hipFree(cnt);
        return nullptr;
    }
    sc.split_ws = ws;
    sc.split_cnt = cnt;
    return &sc;
}

}  // namespace

// Frees this file's scratch of (current device, stream): argmax partials, context-split buffers.  The caller has
// made sure that nothing enqueued on the stream still uses them (t12_release_stream waits for the stream).
extern "C" __attribute__((visibility("hidden"))) void t12_glue_release_stream(hipStream_t st)
{
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_scratch.find({current_device(), st});
    if (it == g_scratch.end()) return;
    if (it->second.part) (void)hipFree(it->second.part);
    if (it->second.split_ws) (void)hipFree(it->second.split_ws);
    if (it->second.split_cnt) (void)hipFree(it->second.split_cnt);
    g_scratch.erase(it);
}

namespace {

bool attn_has_fast(int n_head, int n_head_kv, int head_dim)
{
    const int attn_mode_now = g_attn_mode.load(std::memory_order_relaxed);
    if (!g_attn_fast || n_head_kv <= 0 || n_head % n_head_kv) return false;
    const int r = n_head / n_head_kv;
    return (head_dim == 128 && (r == 1 || r == 2 || r == 4 || r == 8)) || (head_dim == 64 && (r == 1 || r == 4));
}

// fuse != nullptr: RoPE + INT8 KV store happen inside the attention kernel (fast shapes only).
void launch_attn(const float* q, const int8_t* ck, const int8_t* cv, const float* sk, const float* sv, int16_t* out,
                 const int* positions, int seq_len, int n_head, int n_head_kv, int head_dim, float scale, int batch,
                 size_t kv_stride, hipStream_t st, const AttnFuse* fuse = nullptr, int hm = 0)
{
    const int attn_mode_now = g_attn_mode.load(std::memory_order_relaxed);
    const int ratio = n_head / n_head_kv;
    if (ratio < 1 || ratio > ATT_MAX_RATIO || n_head % n_head_kv || head_dim % 16 || head_dim > 128) {
        t12_set_error("attention: unsupported heads %d/%d or head_dim %d (needs ratio <= %d, head_dim %% 16 == 0, <= 128)",
                      n_head, n_head_kv, head_dim, ATT_MAX_RATIO);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    // Context split: only when the host knows the length (no per-sequence position array) and the launch
    // would otherwise leave most of the chip idle.
    int nchunk = 1;
    AttnSplit sp = {nullptr, nullptr, 0};
    if (g_attn_fast && g_attn_chunk > 0 && !positions && batch * n_head_kv <= ATT_SPLIT_HEADS) {
        // one workgroup per CU: with more, the fold of the extra partial sums costs more than the shorter chunks gain
        // (4 sequences at 4000 positions: 18.8 us with 256 workgroups, 22.3 us with 512)
        const int room = ATT_SPLIT_TARGET / (batch * n_head_kv);
        int want = std::min(std::min(room, ATT_TILE / 2), (seq_len + g_attn_chunk - 1) / g_attn_chunk);
        StreamScratch* sc = want > 1 ? attn_split_scratch(st) : nullptr;
        if (sc) {
            sp.chunk_len = (((seq_len + want - 1) / want) + 63) & ~63;
            nchunk = (seq_len + sp.chunk_len - 1) / sp.chunk_len;
            sp.ws = sc->split_ws;
            sp.counter = sc->split_cnt;
        }
    }
    // Two forms of the kernel.  First form: scores by fp32 FMAs with one thread per position, P.V with one wave per
    // head (few registers, no set-up).  Second form: both products by INT8 MFMAs (Q split into three INT8 limbs, the softmax
    // weights into two, K used as stored, V read transposed out of LDS), requests one tile ahead.  Measured on
    // per-sequence caches the second is faster at every length (B = 256: 28 against 38 us at 150 positions, 259
    // against 501 us at 2000; B = 1 at 150 positions: 7.0 against 10.3 us), so it is the default; the first stays
    // selectable (t12_tune_attention(3)) and is what the tests compare it with.
    const bool wide = seq_len >= g_attn_wide;
#define T12_ATT_GO(HD_, R_, F_, S_, W_)                                                                         \
    hipLaunchKernelGGL((attn_fast_kernel<HD_, R_, F_, S_, W_>), dim3(n_head_kv, batch, S_ ? nchunk : 1), dim3(256), 0, \
                       st, q, ck, cv, sk, sv, (uint16_t*)out, positions, seq_len, n_head_kv, scale, kv_stride,   \
                       fuse ? *fuse : AttnFuse(), sp, hm)
#define T12_ATT_FAST(HD_, R_)                                                                                   \
    if (head_dim == HD_ && ratio == R_) {                                                                       \
        const int sel = (fuse ? 4 : 0) | (nchunk > 1 ? 2 : 0) | (wide ? 1 : 0);                                 \
        switch (sel) {                                                                                          \
        case 0: T12_ATT_GO(HD_, R_, false, false, false); break;                                                \
        case 1: T12_ATT_GO(HD_, R_, false, false, true); break;                                                 \
        case 2: T12_ATT_GO(HD_, R_, false, true, false); break;                                                 \
        case 3: T12_ATT_GO(HD_, R_, false, true, true); break;                                                  \
        case 4: T12_ATT_GO(HD_, R_, true, false, false); break;                                                 \
        case 5: T12_ATT_GO(HD_, R_, true, false, true); break;                                                  \
        case 6: T12_ATT_GO(HD_, R_, true, true, false); break;                                                  \
        default: T12_ATT_GO(HD_, R_, true, true, true); break;                                                  \
        }                                                                                                       \
        report("attention");                                                                                    \
        return;                                                                                                 \
    }
    if (g_attn_fast) {
        T12_ATT_FAST(128, 4)
        T12_ATT_FAST(128, 1)
        T12_ATT_FAST(128, 2)
        T12_ATT_FAST(128, 8)
        T12_ATT_FAST(64, 1)
        T12_ATT_FAST(64, 4)
    }
#undef T12_ATT_FAST
#undef T12_ATT_GO
    const size_t smem = ((size_t)ratio * head_dim + (size_t)ratio * ATT_TILE + 17 + 2 * ratio) * sizeof(float);
    hipLaunchKernelGGL(attn_decode_kernel, dim3(n_head_kv, batch), dim3(256), smem, st, q, ck, cv, sk, sv,
                       (uint16_t*)out, positions, seq_len, n_head, n_head_kv, head_dim, scale, kv_stride, hm);
    report("attention");
}

}  // namespace

// ---- C launchers: names and signatures of engine/inference.cpp:9-20 / sampler.cpp:4-5 ----
extern "C" {

void launch_rope_init(int head_dim, float theta_base) { (void)rope_table(head_dim, theta_base); }

// freq[d] = theta^(-2d / head_dim) (kernels.hip:133-134), then, for factor > 0, the "llama3" rule
// of the checkpoints' rope_scaling entry: wavelengths above original_ctx / low_freq_factor are
// stretched by factor, those below original_ctx / high_freq_factor are kept, the band between is
// blended linearly in original_ctx / wavelength.  Host arithmetic only.
void t12_rope_freqs(int head_dim, float theta, float factor, float low_freq_factor, float high_freq_factor,
                    float original_ctx, float* out)
{
    const int half = head_dim / 2;
    const float two_pi = 6.283185307179586f;
    for (int d = 0; d < half; d++) {
        float f = 1.0f / powf(theta, (float)(2 * d) / (float)head_dim);
        if (factor > 0.0f) {
            const float wavelen = two_pi / f;
            if (wavelen > original_ctx / low_freq_factor) {
                f = f / factor;
            } else if (!(wavelen < original_ctx / high_freq_factor)) {
                const float smooth = (original_ctx / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor);
                f = (1.0f - smooth) * f / factor + smooth * f;
            }
        }
        out[d] = f;
    }
}

void launch_rope_scaling(float factor, float low_freq_factor, float high_freq_factor, float original_ctx)
{
    std::lock_guard<std::mutex> lock(g_mu);
    if (!(factor > 0.0f)) factor = low_freq_factor = high_freq_factor = original_ctx = 0.0f;
    g_rope_scale[0] = factor;
    g_rope_scale[1] = low_freq_factor;
    g_rope_scale[2] = high_freq_factor;
    g_rope_scale[3] = original_ctx;
}

// 0: always the general kernel; 1 (default): shapes with a specialised kernel use it in its INT8 MFMA form, one
// sequence at a long context split into chunks of at least 256 positions; 2: never split; 3: the specialised
// kernels in their fp32 FMA form (one wave per head); 4: same as 1; n >= 16: chunks of at least n positions.
int t12_tune_attention(int mode)
{
    const int chunk = mode >= 16 ? (mode & 0xFFFFFF) : (mode == 2 ? 0 : 256);
    g_attn_mode.store(chunk | (mode != 0 ? 1 << 24 : 0) | (mode == 3 ? 1 << 25 : 0), std::memory_order_relaxed);
    return 0;
}

void launch_embed_lookup(const int16_t* embd_table, const int* token_ids, float* output, int n_embd, int batch_size,
                         int n_vocab, hipStream_t stream)
{
    hipLaunchKernelGGL(embed_kernel, dim3((n_embd + 255) / 256, batch_size), dim3(256), 0, stream,
                       (const uint16_t*)embd_table, token_ids, output, n_embd, n_vocab);
    report("embed_lookup");
}

// Rows the 128-bit form takes: a multiple of 4 values, at most 8192, every operand 16-byte aligned.
static bool norm_vec_ok(int n, const void* x, const void* res, const void* w, const void* y, const void* part,
                        size_t split_stride, int ld)
{
    auto al = [](const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; };
    return n >= 4 && n % 4 == 0 && n <= 8192 && al(x, 16) && al(res, 16) && al(w, 16) && al(y, 8) && al(part, 16) &&
           split_stride % 4 == 0 && ld % 4 == 0;
}
// Threads per row of the vectorised norm: one 16-byte piece per thread; with many rows in flight two pieces per thread
// (half the waves at the block sum, two independent sets of loads per thread: 7.4 -> 7.05 us at 256 rows of 4096 with
// four partial rows).
static int norm_vec_threads(int n, int batch_size)
{
    const int per = batch_size >= 64 ? 8 : 4;
    const int t = (n / per + 63) / 64 * 64;
    return t < 64 ? 64 : (t > 1024 ? 1024 : t);
}

static int norm_threads(int n)
{
    int t = (n + 7) / 8;                   // 8 values per thread stay in registers
    t = (t + 63) / 64 * 64;
    return t < 64 ? 64 : (t > 1024 ? 1024 : t);
}

void launch_rms_norm_bf16_batch(const float* x, const float* weight, int16_t* y, int n, float eps, int batch_size,
                                hipStream_t stream)
{
    if (norm_vec_ok(n, x, nullptr, weight, y, nullptr, 0, 0))
        hipLaunchKernelGGL((rms_norm_vec_kernel<false, false, 1>), dim3(batch_size), dim3(norm_vec_threads(n, batch_size)), 0, stream,
                           (float*)x, (const float*)nullptr, weight, (uint16_t*)y, n, eps, (const float*)nullptr, 0,
                           (size_t)0, 0);
    else
        hipLaunchKernelGGL(rms_norm_kernel<false>, dim3(batch_size), dim3(norm_threads(n)), 0, stream, (float*)x,
                           (const float*)nullptr, weight, (uint16_t*)y, n, eps);
    report("rms_norm");
}

void launch_add_rms_norm_bf16_batch(float* x, const float* residual, const float* weight, int16_t* y, int n, float eps,
                                    int batch_size, hipStream_t stream)
{
    if (norm_vec_ok(n, x, residual, weight, y, nullptr, 0, 0))
        hipLaunchKernelGGL((rms_norm_vec_kernel<true, false, 1>), dim3(batch_size), dim3(norm_vec_threads(n, batch_size)), 0, stream, x,
                           residual, weight, (uint16_t*)y, n, eps, (const float*)nullptr, 0, (size_t)0, 0);
    else
        hipLaunchKernelGGL(rms_norm_kernel<true>, dim3(batch_size), dim3(norm_threads(n)), 0, stream, x, residual, weight,
                           (uint16_t*)y, n, eps);
    report("add_rms_norm");
}

// x[b] = (sum of the nsplit partial rows) + residual[b] (stored), y[b] = bf16(RMSNorm(x[b]) * weight):
// launch_add_rms_norm_bf16_batch fed by the K-split partial sums of t12_gemm_deferred.
void launch_sum_add_rms_norm_bf16_batch(float* x, const float* partials, int nsplit, size_t split_stride, int ld,
                                        const float* residual, const float* weight, int16_t* y, int n, float eps,
                                        int batch_size, hipStream_t stream)
{
    if (nsplit < 1 || nsplit > T12_MAX_KSPLIT || !partials) {
        t12_set_error("sum_add_rms_norm: nsplit %d outside 1..%d or null partials", nsplit, T12_MAX_KSPLIT);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    if (norm_vec_ok(n, x, residual, weight, y, partials, split_stride, ld)) {
        const dim3 g(batch_size), b(norm_vec_threads(n, batch_size));
        if (nsplit <= 4)
            hipLaunchKernelGGL((rms_norm_vec_kernel<true, true, 4>), g, b, 0, stream, x, residual, weight, (uint16_t*)y, n,
                               eps, partials, nsplit, split_stride, ld);
        else if (nsplit <= 8)
            hipLaunchKernelGGL((rms_norm_vec_kernel<true, true, 8>), g, b, 0, stream, x, residual, weight, (uint16_t*)y, n,
                               eps, partials, nsplit, split_stride, ld);
        else
            hipLaunchKernelGGL((rms_norm_vec_kernel<true, true, T12_MAX_KSPLIT>), g, b, 0, stream, x, residual, weight,
                               (uint16_t*)y, n, eps, partials, nsplit, split_stride, ld);
        report("sum_add_rms_norm");
        return;
    }
    // one workgroup per row has every partial of the row to fetch: as many lanes as the row allows
    int threads = (n + 1) / 2;
    threads = (threads + 63) / 64 * 64;
    threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
    hipLaunchKernelGGL((rms_norm_kernel<true, true>), dim3(batch_size), dim3(threads), 0, stream, x, residual,
                       weight, (uint16_t*)y, n, eps, partials, nsplit, split_stride, ld);
    report("sum_add_rms_norm");
}

void launch_silu_mul_bf16_batch(const float* gate, const float* up, int16_t* out, int n, int batch_size,
                                hipStream_t stream)
{
    const size_t total = (size_t)n * batch_size;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0, stream, gate, up,
                       (uint16_t*)out, total);
    report("silu_mul");
}

void launch_add_batch(float* y, const float* x, int n, int batch_size, hipStream_t stream)
{
    const size_t total = (size_t)n * batch_size;
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, y, x, total);
    report("add");
}

void launch_rope_batch(float* q, float* k, const int* positions, int head_dim, int n_head, int n_head_kv, int q_stride,
                       int k_stride, float theta, int batch_size, hipStream_t stream)
{
    launch_rope_kv<1>(q, k, nullptr, nullptr, nullptr, nullptr, nullptr, positions, 0, head_dim, n_head, n_head_kv,
                      q_stride, k_stride, theta, batch_size, stream);
}

void launch_store_kv_batch(const float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k, float* scale_v,
                           const int* positions, int kv_dim, int max_seq, int n_head_kv, int head_dim, int batch_size,
                           hipStream_t stream)
{
    (void)max_seq;
    launch_rope_kv<2>(nullptr, (float*)k, v, kv_k, kv_v, scale_k, scale_v, positions, 0, head_dim, 0, n_head_kv, 0,
                      kv_dim, 1.0f, batch_size, stream);
}

void launch_rope_store_kv(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                          float* scale_v, int head_dim, int n_head, int n_head_kv, int position, int max_seq,
                          float theta, hipStream_t stream)
{
    (void)max_seq;
    launch_rope_kv<3>(q, k, v, kv_k, kv_v, scale_k, scale_v, nullptr, position, head_dim, n_head, n_head_kv,
                      n_head * head_dim, n_head_kv * head_dim, theta, 1, stream);
}

// Extension of the reference's launch layer: RoPE + INT8 store for a whole batch in one launch.
void launch_rope_store_kv_batch(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                float* scale_v, const int* positions, int head_dim, int n_head, int n_head_kv,
                                int q_stride, int k_stride, float theta, int batch_size, hipStream_t stream)
{
    launch_rope_kv<3>(q, k, v, kv_k, kv_v, scale_k, scale_v, positions, 0, head_dim, n_head, n_head_kv, q_stride,
                      k_stride, theta, batch_size, stream);
}

// Extension of the reference's launch layer: RoPE (Q and K) + INT8 KV store + attention in ONE
// launch, for B >= 1.  positions: device array [batch] (NULL: every sequence is at `position`).
// Shapes without a specialised kernel, and large batches, run the separate launches.  q is scratch: left as
// it was by the fused kernel, rotated in place by the separate RoPE launch.
static void rope_store_attention(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                 float* scale_v, int16_t* output, const int* positions, int position, int n_head,
                                 int n_head_kv, int head_dim, float theta, float scale, int batch_size, int kv_stride,
                                 int hm, hipStream_t stream, bool copies = false)
{
    // Fusing pays when every workgroup stores its own cache slot (one sequence, or per-sequence caches) and
    // the launch is small enough to be a chain of latencies: the fused kernel holds prefetched rows in more
    // registers, so only two of its workgroups fit a CU (measured at B = 256 on per-sequence caches: 35 us
    // fused against 26 + 7 us for the two launches at 150 positions, 256 against 248 + 7 us at 2000).  Lock-step
    // copies on a shared cache (kv_stride = 0, batch > 1) store the same slot from every workgroup: the same bytes when
    // the caller vouches that the rows are copies of one sequence at one position (`copies`), and every workgroup
    // attends to its own new row either way; without that promise the rows may be the positions of one prompt, which
    // need each other's stores, and take the two launches.
    if (attn_has_fast(n_head, n_head_kv, head_dim) &&
        (batch_size == 1 || ((kv_stride != 0 || copies) && batch_size * n_head_kv <= 256))) {
        AttnFuse fz;
        fz.k_new = k;
        fz.v_new = v;
        fz.ck_w = kv_k;
        fz.cv_w = kv_v;
        fz.sk_w = scale_k;
        fz.sv_w = scale_v;
        fz.freqs = rope_table(head_dim, theta);
        if (!fz.freqs) { t12_set_error("rope: cannot build the frequency table"); return; }
        launch_attn(q, kv_k, kv_v, scale_k, scale_v, output, positions, position + 1, n_head, n_head_kv, head_dim,
                    scale, batch_size, (size_t)kv_stride, stream, &fz, hm);
        return;
    }
    launch_rope_kv<3>(q, k, v, kv_k, kv_v, scale_k, scale_v, positions, position, head_dim, n_head, n_head_kv,
                      n_head * head_dim, n_head_kv * head_dim, theta, batch_size, stream, QkvPartials{nullptr, 0, 0, 0},
                      (size_t)kv_stride, hm);
    launch_attn(q, kv_k, kv_v, scale_k, scale_v, output, positions, position + 1, n_head, n_head_kv, head_dim, scale,
                batch_size, (size_t)kv_stride, stream, nullptr, hm);
}

void launch_rope_store_attention(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                 float* scale_v, int16_t* output, const int* positions, int position, int n_head,
                                 int n_head_kv, int head_dim, float theta, float scale, int batch_size, int kv_stride,
                                 hipStream_t stream)
{
    rope_store_attention(q, k, v, kv_k, kv_v, scale_k, scale_v, output, positions, position, n_head, n_head_kv, head_dim,
                         theta, scale, batch_size, kv_stride, 0, stream);
}

// Library-internal (the engine's lock-step batches): launch_rope_store_attention on ONE shared cache region for rows
// that are copies of one sequence, all at `position` -- the reference's batched mode (inference.cpp:430-435: every
// row stores the slot of the shared cache, kernels.hip:785-788).  Small batches then take the fused kernel.
extern "C" __attribute__((visibility("hidden"))) void t12_rope_store_attention_copies(
    float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k, float* scale_v, int16_t* output,
    const int* positions, int position, int n_head, int n_head_kv, int head_dim, float theta, float scale, int batch_size,
    int region_positions, hipStream_t stream)
{
    rope_store_attention(q, k, v, kv_k, kv_v, scale_k, scale_v, output, positions, position, n_head, n_head_kv, head_dim,
                         theta, scale, batch_size, 0, region_positions, stream, true);
}

// The same on head-major cache regions: region_positions > 0 rows per (region, KV head), a region laid out
// [kv head][region_positions][head_dim] (scales [kv head][region_positions]) instead of the reference's
// [position][kv head][head_dim].  Every workgroup then reads one contiguous stream instead of 128-byte pieces of rows
// it shares with the other KV heads' workgroups (B = 256 at 2000 positions: 199 against 254 us).  kv_stride is the
// distance between regions as before.
void launch_rope_store_attention_regions(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v, float* scale_k,
                                         float* scale_v, int16_t* output, const int* positions, int position, int n_head,
                                         int n_head_kv, int head_dim, float theta, float scale, int batch_size,
                                         int kv_stride, int region_positions, hipStream_t stream)
{
    if (region_positions < 1 || position >= region_positions) {
        t12_set_error("rope_store_attention_regions: position %d outside a region of %d positions", position, region_positions);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    rope_store_attention(q, k, v, kv_k, kv_v, scale_k, scale_v, output, positions, position, n_head, n_head_kv, head_dim,
                         theta, scale, batch_size, kv_stride, region_positions, stream);
}

// launch_rope_store_attention for a batch whose q | k | v projection was split along K (t12_gemm_deferred,
// one launch for the three tensors in this order): the RoPE / KV-store kernel adds the partial sums up
// itself.  q and k receive the rotated values; the v buffer is not written.  kv_stride = 0: one shared cache
// region (lock-step copies, or the rows of one sequence's prompt at consecutive positions -- every row's
// K / V is stored before any row attends, so row t sees rows <= t: a causal prefill); otherwise the element
// distance between the regions of consecutive sequences.
static void rope_store_attention_partials(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v,
                                          float* scale_k, float* scale_v, int16_t* output, const int* positions,
                                          int position, int n_head, int n_head_kv, int head_dim, float theta,
                                          float scale, int batch_size, const float* partials, int nsplit,
                                          size_t split_stride, int ld, int kv_stride, int hm, hipStream_t stream)
{
    if (!partials || nsplit < 1 || nsplit > T12_MAX_KSPLIT || ld < (n_head + 2 * n_head_kv) * head_dim) {
        t12_set_error("rope_store_attention_partials: nsplit %d outside 1..%d, null partials or ld %d too small", nsplit,
                      T12_MAX_KSPLIT, ld);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    launch_rope_kv<3>(q, k, v, kv_k, kv_v, scale_k, scale_v, positions, position, head_dim, n_head, n_head_kv,
                      n_head * head_dim, n_head_kv * head_dim, theta, batch_size, stream,
                      QkvPartials{partials, nsplit, ld, split_stride}, (size_t)kv_stride, hm);
    launch_attn(q, kv_k, kv_v, scale_k, scale_v, output, positions, position + 1, n_head, n_head_kv, head_dim, scale,
                batch_size, (size_t)kv_stride, stream, nullptr, hm);
}

void launch_rope_store_attention_partials(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v,
                                          float* scale_k, float* scale_v, int16_t* output, const int* positions,
                                          int position, int n_head, int n_head_kv, int head_dim, float theta,
                                          float scale, int batch_size, const float* partials, int nsplit,
                                          size_t split_stride, int ld, int kv_stride, hipStream_t stream)
{
    rope_store_attention_partials(q, k, v, kv_k, kv_v, scale_k, scale_v, output, positions, position, n_head, n_head_kv,
                                  head_dim, theta, scale, batch_size, partials, nsplit, split_stride, ld, kv_stride, 0, stream);
}

// launch_rope_store_attention_partials on head-major cache regions (see launch_rope_store_attention_regions).
void launch_rope_store_attention_partials_regions(float* q, float* k, const float* v, int8_t* kv_k, int8_t* kv_v,
                                                  float* scale_k, float* scale_v, int16_t* output, const int* positions,
                                                  int position, int n_head, int n_head_kv, int head_dim, float theta,
                                                  float scale, int batch_size, const float* partials, int nsplit,
                                                  size_t split_stride, int ld, int kv_stride, int region_positions,
                                                  hipStream_t stream)
{
    if (region_positions < 1) {
        t12_set_error("rope_store_attention_partials_regions: a region of %d positions", region_positions);
        fprintf(stderr, "turbo12: %s\n", t12_last_error());
        return;
    }
    rope_store_attention_partials(q, k, v, kv_k, kv_v, scale_k, scale_v, output, positions, position, n_head, n_head_kv,
                                  head_dim, theta, scale, batch_size, partials, nsplit, split_stride, ld, kv_stride,
                                  region_positions, stream);
}

void launch_attention_all_heads(const float* q, const int8_t* k_cache, const int8_t* v_cache, const float* scale_k,
                                const float* scale_v, int16_t* output, int n_head, int n_head_kv, int head_dim,
                                int seq_len, int max_seq, float scale, hipStream_t stream)
{
    (void)max_seq;
    launch_attn(q, k_cache, v_cache, scale_k, scale_v, output, nullptr, seq_len, n_head, n_head_kv, head_dim, scale, 1,
                0, stream);
}

void launch_flash_attention(const float* q, const int8_t* k_cache, const int8_t* v_cache, const float* scale_k,
                            const float* scale_v, int16_t* output, int n_head, int n_head_kv, int head_dim, int seq_len,
                            int max_seq, float scale, hipStream_t stream)
{
    launch_attention_all_heads(q, k_cache, v_cache, scale_k, scale_v, output, n_head, n_head_kv, head_dim, seq_len,
                               max_seq, scale, stream);
}

void launch_attention_all_heads_batch(const float* q, const int8_t* kv_k, const int8_t* kv_v, const float* scale_k,
                                      const float* scale_v, int16_t* output, const int* positions, int n_head,
                                      int n_head_kv, int head_dim, int max_seq, float scale, int batch_size,
                                      int kv_stride, hipStream_t stream)
{
    (void)max_seq;
    launch_attn(q, kv_k, kv_v, scale_k, scale_v, output, positions, 0, n_head, n_head_kv, head_dim, scale, batch_size,
                (size_t)kv_stride, stream);
}

void launch_flash_attention_batch(const float* q, const int8_t* kv_k, const int8_t* kv_v, const float* scale_k,
                                  const float* scale_v, int16_t* output, const int* positions, int n_head,
                                  int n_head_kv, int head_dim, int max_seq, float scale, int batch_size, int kv_stride,
                                  hipStream_t stream)
{
    launch_attention_all_heads_batch(q, kv_k, kv_v, scale_k, scale_v, output, positions, n_head, n_head_kv, head_dim,
                                     max_seq, scale, batch_size, kv_stride, stream);
}

void launch_argmax_batch(const float* logits, int* results, int n_vocab, int batch_size, hipStream_t stream)
{
    ArgPair* part = argmax_scratch(batch_size, stream);
    if (!part) { t12_set_error("argmax: cannot allocate scratch"); return; }
    hipLaunchKernelGGL(argmax_part_kernel, dim3(ARG_CHUNKS, batch_size), dim3(256), 0, stream, logits, n_vocab, part);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(batch_size), dim3(64), 0, stream, part, results);
    report("argmax");
}

void launch_argmax(const float* logits, int* result, int n, hipStream_t stream)
{
    launch_argmax_batch(logits, result, n, 1, stream);
}

}  // extern "C"
