// Mixture-of-experts SwiGLU feed-forward layer over split-12 experts (a Mixtral-shaped layer: 8 experts, top-2):
//
//   out[t] = sum_j weights[t, j] * W2_e( silu(W1_e x_t) * (W3_e x_t) ),   e = expert_ids[t, j]
//
// The reference engine has no such layer; its decode+GEMM entry point (nv_launch_split12_fused_gemm_async,
// nvidia_kernels.cu:444) would be called once per expert with that expert's token count as the batch.  Here the
// layer is five launches and the host never waits:
//   1. moe_route_kernel    counting sort of the (token, slot) pairs by expert: counts, first slot per expert,
//                          slot <-> pair tables
//   2. moe_gather_kernel   activation rows in slot order (bf16 [P, n_embd], P = T * k)
//   3. grouped gate|up     (gate, up) of every expert over its slots with the SwiGLU in the epilogue -> bf16 [P, n_ff]
//   4. grouped down        down of every expert over its slots                                      -> fp32 [P, n_embd]
//   5. moe_combine_kernel  out[t] = sum_j weights[t, j] * Y[slot(t, j)]  (j ascending: a fixed order, no atomics)
// The grouped launches read the rows per expert from the routing kernel's tables on the device: one workgroup per row
// tile, which walks the expert's batch tiles (one, unless the expert received more rows than the tile holds).
// A call with at most eight pairs (a decode step of a few sequences) replaces 3 and 4 by two launches of the B = 1
// kernel over (row groups, slots): every slot multiplies its row with the tensors of its expert, read from the table.
// Shapes the tile kernel does not take (K not a multiple of 64, base_exp outside 0..240) size their launches on the
// host instead: one copy of the counts and one wait per call.

#include <cmath>
#include <vector>

#include "t12_device.h"
#include "t12_host.h"

extern "C" void launch_silu_mul_bf16_batch(const float* gate, const float* up, int16_t* out, int n, int batch_size,
                                           hipStream_t stream);
extern "C" __attribute__((visibility("hidden"))) int t12_gemm_experts(const T12Segment* segs, int nseg, int K, const void* act_bf16,
                                                                      int act_stride, const int* dev_counts, const int* dev_base,
                                                                      int first_group, int hint_b, int pairs,
                                                                      void* out_bf16, int out_bf16_ld, void* stream);

extern "C" __attribute__((visibility("hidden"))) int t12_gemv_experts(const T12Segment* segs, int per_expert, int E, int K,
                                                                      const void* act_bf16, int act_stride,
                                                                      const int* slot_expert, int slots, void* out_bf16,
                                                                      int out_ld, void* stream);

namespace {

constexpr int ROUTE_THREADS = 256;
constexpr int FEW_SLOTS = 8;          // up to this many (token, expert) pairs every slot is its own matrix-vector product
constexpr int MAX_EXPERTS = 128;      // the sort keeps a 257-entry count row per expert in LDS (132 KB at 128 experts)

// One workgroup.  Thread i owns the pairs [i * chunk, (i + 1) * chunk); pairs of one expert keep their order
// (pair index ascending), so the grouping is the same on every run.  counts[e] = pairs of expert e, base[e] = its
// first slot (base[E] = pairs placed), expert_of_slot[slot] = the expert whose range holds the slot; slots past the
// placed pairs get pair -1 and expert -1.  *bad = 1 if an id lies outside 0..E-1
// (such a pair gets no slot and contributes nothing).
template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void moe_route_kernel(const IdT* __restrict__ ids, int P, int E,
                                                                  int* __restrict__ counts, int* __restrict__ base,
                                                                  int* __restrict__ pair_of_slot, int* __restrict__ slot_of_pair,
                                                                  int* __restrict__ expert_of_slot, int* __restrict__ bad)
{
    extern __shared__ int route_lds[];
    constexpr int LD = ROUTE_THREADS + 1;
    int* cnt = route_lds;                          // [E][LD]
    int* ebase = route_lds + E * LD;               // [E + 1]
    const int tid = threadIdx.x;
    const int chunk = (P + ROUTE_THREADS - 1) / ROUTE_THREADS;
    const int lo = min(P, tid * chunk), hi = min(P, lo + chunk);
    for (int e = 0; e < E; e++) cnt[e * LD + tid] = 0;
    if (tid == 0) *bad = 0;
    __syncthreads();
    for (int q = lo; q < hi; q++) {
        const long long e = (long long)ids[q];
        if (e >= 0 && e < E) cnt[(int)e * LD + tid]++;
        else *bad = 1;
    }
    __syncthreads();
    // per expert: exclusive prefix over the threads (one wave per expert in turn; 256 values = 4 per lane)
    const int lane = tid & 63, wave = tid >> 6;
    for (int e = wave; e < E; e += ROUTE_THREADS / 64) {
        int v[4], run = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = cnt[e * LD + lane * 4 + i];
            run += v[i];
        }
        int incl = run;                                    // inclusive scan of the lanes' sums
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(incl, d, 64);
            if (lane >= d) incl += o;
        }
        int b = incl - run;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            cnt[e * LD + lane * 4 + i] = b;
            b += v[i];
        }
        if (lane == 63) cnt[e * LD + ROUTE_THREADS] = incl;      // the expert's total
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < E; e++) {
            ebase[e] = run;
            base[e] = run;
            run += cnt[e * LD + ROUTE_THREADS];
            counts[e] = cnt[e * LD + ROUTE_THREADS];
        }
        ebase[E] = run;
        base[E] = run;
    }
    __syncthreads();
    for (int q = lo; q < hi; q++) {
        const long long e = (long long)ids[q];
        if (e >= 0 && e < E) {
            const int slot = ebase[(int)e] + cnt[(int)e * LD + tid]++;
            pair_of_slot[slot] = q;
            slot_of_pair[q] = slot;
            expert_of_slot[slot] = (int)e;
        } else {
            slot_of_pair[q] = -1;
        }
    }
    for (int slot = ebase[E] + tid; slot < P; slot += ROUTE_THREADS) {
        pair_of_slot[slot] = -1;
        expert_of_slot[slot] = -1;
    }
}

// Xg[slot, :] = X[pair_of_slot[slot] / k, :]; one workgroup per slot, 16 bytes per thread and step.
__global__ __launch_bounds__(256) void moe_gather_kernel(const uint16_t* __restrict__ x, int x_stride, const int* __restrict__ pair_of_slot,
                                                         int k, int n, uint16_t* __restrict__ xg)
{
    const int slot = blockIdx.x;
    if (pair_of_slot[slot] < 0) return;                  // past the placed pairs
    const int t = pair_of_slot[slot] / k;
    const uint16_t* src = x + (size_t)t * x_stride;
    uint16_t* dst = xg + (size_t)slot * n;
    if ((n & 7) == 0 && (x_stride & 7) == 0 && ((uintptr_t)x & 15) == 0) {
        for (int c = threadIdx.x * 8; c < n; c += 256 * 8) *(uint4*)(dst + c) = *(const uint4*)(src + c);
    } else {
        for (int c = threadIdx.x; c < n; c += 256) dst[c] = src[c];
    }
}

// out[t, c] = sum_j w[t, j] * Y[slot_of_pair[t * k + j], c]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ slot_of_pair,
                                                          const float* __restrict__ w, int k, int n, float* __restrict__ out,
                                                          int out_stride)
{
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < n; c += 256) {
        float v = 0.0f;
        for (int j = 0; j < k; j++) {
            const int slot = slot_of_pair[t * k + j];
            if (slot >= 0) v += w[t * k + j] * y[(size_t)slot * n + c];
        }
        out[(size_t)t * out_stride + c] = v;
    }
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct MoeLayout {
    size_t bad, counts, base, pair_of_slot, slot_of_pair, expert_of_slot, xg, gate, up, act, y, total;
};

MoeLayout moe_layout(int T, int k, int n_embd, int n_ff, int E)
{
    const size_t P = (size_t)T * k;
    MoeLayout l;
    size_t o = 0;
    l.bad = o;           o = align256(o + sizeof(int));           // first word of the workspace: t12_moe_status reads it
    l.counts = o;        o = align256(o + sizeof(int) * (size_t)E);
    l.base = o;          o = align256(o + sizeof(int) * (size_t)(E + 1));
    l.pair_of_slot = o;  o = align256(o + sizeof(int) * P);
    l.slot_of_pair = o;  o = align256(o + sizeof(int) * P);
    l.expert_of_slot = o; o = align256(o + sizeof(int) * P);
    l.xg = o;            o = align256(o + 2 * P * n_embd);
    l.gate = o;          o = align256(o + 4 * P * n_ff);
    l.up = o;            o = align256(o + 4 * P * n_ff);
    l.act = o;           o = align256(o + 2 * P * n_ff);
    l.y = o;             o = align256(o + 4 * P * n_embd);
    l.total = o;
    return l;
}

// Shapes the tile kernel does not take: the per-expert counts come to the host (one copy, one wait), the grouped
// launches are t12_gemm_grouped calls sized by them (which run such groups as t12_gemm calls), SiLU*mul in between.
int moe_ffn_host_counts(const T12MoeExpert* experts, int E, int T, int n_embd, int n_ff, const int* counts, uint16_t* xg,
                        float* gate, float* up, int16_t* act, float* y, void* stream)
{
    hipStream_t st = (hipStream_t)stream;
    std::vector<int> host(E);
    if (hipMemcpyAsync(host.data(), counts, sizeof(int) * E, hipMemcpyDeviceToHost, st) != hipSuccess ||
        hipStreamSynchronize(st) != hipSuccess) {
        t12_set_error("t12_moe_ffn: reading the per-expert counts failed: %s", hipGetErrorString(hipGetLastError()));
        return T12_ELAUNCH;
    }
    int placed = 0;
    for (int e = 0; e < E; e++) placed += host[e];
    (void)T;
    for (int e0 = 0; e0 < E; e0 += 8) {
        T12Group g[16];
        int n = 0, slot0 = 0;
        for (int e = 0; e < e0; e++) slot0 += host[e];
        for (int e = e0; e < E && e < e0 + 8; e++) {
            for (int j = 0; j < 2; j++) {
                T12Group& q = g[n++];
                q.seg = j == 0 ? experts[e].w1 : experts[e].w3;
                q.seg.out = (j == 0 ? gate : up) + (size_t)slot0 * n_ff;
                q.seg.out_stride = n_ff;
                q.act_bf16 = xg + (size_t)slot0 * n_embd;
                q.act_stride = n_embd;
                q.B = host[e];
            }
            slot0 += host[e];
        }
        const int rc = t12_gemm_grouped(g, n, n_embd, stream);
        if (rc) return rc;
    }
    if (placed > 0) launch_silu_mul_bf16_batch(gate, up, act, n_ff, placed, st);
    T12_CHECK_LAUNCH("t12_moe_ffn(silu_mul)");
    for (int e0 = 0; e0 < E; e0 += 16) {
        T12Group g[16];
        int n = 0, slot0 = 0;
        for (int e = 0; e < e0; e++) slot0 += host[e];
        for (int e = e0; e < E && e < e0 + 16; e++) {
            T12Group& q = g[n++];
            q.seg = experts[e].w2;
            q.seg.out = y + (size_t)slot0 * n_embd;
            q.seg.out_stride = n_embd;
            q.act_bf16 = act + (size_t)slot0 * n_ff;
            q.act_stride = n_ff;
            q.B = host[e];
            slot0 += host[e];
        }
        const int rc = t12_gemm_grouped(g, n, n_ff, stream);
        if (rc) return rc;
    }
    return T12_OK;
}

}  // namespace

extern "C" {

size_t t12_moe_workspace_bytes(int T, int k, int n_embd, int n_ff, int E)
{
    if (T < 1 || k < 1 || n_embd < 1 || n_ff < 1 || E < 1) return 0;
    return moe_layout(T, k, n_embd, n_ff, E).total;
}

int t12_moe_ffn(const T12MoeExpert* experts, int E, const void* x_bf16, int x_stride, const void* expert_ids,
                int id_bytes, const float* weights, int T, int k, int n_embd, int n_ff, void* workspace,
                size_t workspace_bytes, float* out, int out_stride, void* stream)
{
    T12_REQUIRE(experts && x_bf16 && expert_ids && weights && workspace && out, "t12_moe_ffn: null operand");
    T12_REQUIRE(E >= 1 && E <= MAX_EXPERTS, "t12_moe_ffn: 1..%d experts (got %d)", MAX_EXPERTS, E);
    T12_REQUIRE(T >= 1 && k >= 1 && k <= E && n_embd >= 1 && n_ff >= 1, "t12_moe_ffn: T %d, k %d, n_embd %d or n_ff %d invalid",
                T, k, n_embd, n_ff);
    T12_REQUIRE((long long)T * k < (1ll << 24), "t12_moe_ffn: %lld (token, expert) pairs, at most 2^24", (long long)T * k);
    T12_REQUIRE(id_bytes == 4 || id_bytes == 8, "t12_moe_ffn: expert ids are int32 or int64 (id_bytes %d)", id_bytes);
    T12_REQUIRE(x_stride >= n_embd && out_stride >= n_embd, "t12_moe_ffn: x_stride %d or out_stride %d < n_embd %d", x_stride,
                out_stride, n_embd);
    T12_REQUIRE((uintptr_t)workspace % 256 == 0, "t12_moe_ffn: workspace must be 256-byte aligned");
    const MoeLayout l = moe_layout(T, k, n_embd, n_ff, E);
    T12_REQUIRE(workspace_bytes >= l.total, "t12_moe_ffn: workspace of %zu bytes, t12_moe_workspace_bytes says %zu",
                workspace_bytes, l.total);
    for (int e = 0; e < E; e++) {
        const T12MoeExpert& x = experts[e];
        T12_REQUIRE(x.w1.M == n_ff && x.w3.M == n_ff && x.w2.M == n_embd, "t12_moe_ffn: expert %d: w1/w3 need %d rows, w2 %d", e,
                    n_ff, n_embd);
    }
    hipStream_t st = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    int* counts = (int*)(ws + l.counts);
    int* base = (int*)(ws + l.base);
    int* bad = (int*)(ws + l.bad);
    int* pair_of_slot = (int*)(ws + l.pair_of_slot);
    int* slot_of_pair = (int*)(ws + l.slot_of_pair);
    int* expert_of_slot = (int*)(ws + l.expert_of_slot);
    uint16_t* xg = (uint16_t*)(ws + l.xg);
    float* gate = (float*)(ws + l.gate);
    float* up = (float*)(ws + l.up);
    int16_t* act = (int16_t*)(ws + l.act);
    float* y = (float*)(ws + l.y);
    const int P = T * k;

    const size_t route_lds = sizeof(int) * ((size_t)E * (ROUTE_THREADS + 1) + E + 1);
    if (id_bytes == 4) {
        auto fn = moe_route_kernel<int32_t>;
        if (route_lds > 48 * 1024 && hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)route_lds) != hipSuccess) {
            t12_set_error("t12_moe_ffn: cannot reserve %zu bytes of LDS for the routing sort", route_lds);
            return T12_ELAUNCH;
        }
        hipLaunchKernelGGL(fn, dim3(1), dim3(ROUTE_THREADS), route_lds, st, (const int32_t*)expert_ids, P, E, counts, base,
                           pair_of_slot, slot_of_pair, expert_of_slot, bad);
    } else {
        auto fn = moe_route_kernel<long long>;
        if (route_lds > 48 * 1024 && hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)route_lds) != hipSuccess) {
            t12_set_error("t12_moe_ffn: cannot reserve %zu bytes of LDS for the routing sort", route_lds);
            return T12_ELAUNCH;
        }
        hipLaunchKernelGGL(fn, dim3(1), dim3(ROUTE_THREADS), route_lds, st, (const long long*)expert_ids, P, E, counts, base,
                           pair_of_slot, slot_of_pair, expert_of_slot, bad);
    }
    T12_CHECK_LAUNCH("t12_moe_ffn(route)");
    hipLaunchKernelGGL(moe_gather_kernel, dim3(P), dim3(256), 0, st, (const uint16_t*)x_bf16, x_stride, pair_of_slot, k, n_embd, xg);
    T12_CHECK_LAUNCH("t12_moe_ffn(gather)");

    // ---- the grouped launches sized on the device: gate|up of eight experts per launch, down of sixteen.  The batch
    //      tile is picked for a count few experts exceed: mean + 4 standard deviations of an even routing (an expert
    //      above the tile streams its planes once per tile it needs, so a tile below the typical maximum costs more than
    //      a tile above it).  Above 128 rows the SwiGLU goes into the gate|up epilogue; below, the 128-row SwiGLU tile is
    //      slower than two plain groups and the SiLU*mul kernel (Mixtral shape, ~64 rows per expert: 490 against 468 us).
    // ---- a handful of pairs (a decode step of one or a few sequences): every slot is one matrix-vector product with
    //      its expert's tensors, picked on the device -- gate|up with the SwiGLU in the epilogue, then down.  Each named
    //      expert is streamed once per slot that names it, at the rate of the B = 1 kernel (Mixtral shape, one token:
    //      0.16 -> 0.10 ms against the 16-row sweep below, which also starts a workgroup for every row group of every
    //      expert nobody named).
    if (P <= FEW_SLOTS && 2 * E <= 16 && n_embd % 16 == 0 && n_ff % 16 == 0 && n_embd >= 2048 && n_ff >= 2048) {
        T12Segment sg[16];
        bool ok = true;
        for (int e = 0; e < E; e++) {
            sg[2 * e] = experts[e].w1;
            sg[2 * e + 1] = experts[e].w3;
            for (const T12Segment* g : {&experts[e].w1, &experts[e].w3, &experts[e].w2})
                if (g->base_exp < 0 || g->base_exp > 240 || !g->sm || !g->gr) ok = false;
        }
        if (ok) {
            int rc = t12_gemv_experts(sg, 2, E, n_embd, xg, n_embd, expert_of_slot, P, act, n_ff, stream);
            if (rc < 0) return rc;
            if (rc == 0) {
                for (int e = 0; e < E; e++) {
                    sg[e] = experts[e].w2;
                    sg[e].out = y;
                }
                rc = t12_gemv_experts(sg, 1, E, n_ff, act, n_ff, expert_of_slot, P, nullptr, n_embd, stream);
                if (rc < 0) return rc;
                if (rc == 0) {
                    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, slot_of_pair, weights, k, n_embd, out,
                                       out_stride);
                    T12_CHECK_LAUNCH("t12_moe_ffn(combine)");
                    return T12_OK;
                }
                // (the down projection has no such kernel: the grouped path below redoes the layer)
            }
        }
    }

    const double mean = (double)P / E;
    const int hint = (int)fmin((double)P, ceil(mean + 4.0 * sqrt(mean * (1.0 - 1.0 / E))));
    const bool fuse_swiglu = hint > 128;
    bool on_device = true;
    for (int e0 = 0; e0 < E && on_device; e0 += 8) {
        T12Segment sg[16];
        int n = 0;
        for (int e = e0; e < E && e < e0 + 8; e++) {
            sg[n] = experts[e].w1;
            sg[n].out = gate;
            sg[n++].out_stride = n_ff;
            sg[n] = experts[e].w3;
            sg[n].out = up;
            sg[n++].out_stride = n_ff;
        }
        const int rc = t12_gemm_experts(sg, n, n_embd, xg, n_embd, counts, base, e0, hint, fuse_swiglu ? 1 : 2, act, n_ff, stream);
        if (rc < 0) return rc;
        if (rc == 1) on_device = false;                  // this shape has no such kernel
    }
    if (on_device && !fuse_swiglu) {
        launch_silu_mul_bf16_batch(gate, up, act, n_ff, P, st);      // rows past the placed pairs: computed, never read
        T12_CHECK_LAUNCH("t12_moe_ffn(silu_mul)");
    }
    for (int e0 = 0; e0 < E && on_device; e0 += 16) {
        T12Segment sg[16];
        int n = 0;
        for (int e = e0; e < E && e < e0 + 16; e++) {
            sg[n] = experts[e].w2;
            sg[n].out = y;
            sg[n].out_stride = n_embd;
            n++;
        }
        const int rc = t12_gemm_experts(sg, n, n_ff, act, n_ff, counts, base, e0, hint, 0, nullptr, 0, stream);
        if (rc < 0) return rc;
        if (rc == 1) on_device = false;
    }
    if (!on_device) {
        const int rc = moe_ffn_host_counts(experts, E, T, n_embd, n_ff, counts, xg, gate, up, act, y, stream);
        if (rc) return rc;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, slot_of_pair, weights, k, n_embd, out, out_stride);
    T12_CHECK_LAUNCH("t12_moe_ffn(combine)");
    return T12_OK;
}

// Waits for the stream and reports what the routing kernel of the last t12_moe_ffn call on this workspace found:
// T12_OK, or T12_EINVAL when an expert id lay outside 0..E-1 (that pair was left out of the sum).
int t12_moe_status(const void* workspace, void* stream)
{
    T12_REQUIRE(workspace, "t12_moe_status: null workspace");
    int flag = 0;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess ||
        hipMemcpy(&flag, workspace, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) {
        t12_set_error("t12_moe_status: reading the flag failed: %s", hipGetErrorString(hipGetLastError()));
        return T12_ELAUNCH;
    }
    T12_REQUIRE(flag == 0, "t12_moe_ffn: an expert id lay outside the expert table; its pair was left out");
    return T12_OK;
}

}  // extern "C"
