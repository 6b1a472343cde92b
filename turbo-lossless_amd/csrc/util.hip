// Small utility kernels of the engine.

#include <hip/hip_ext.h>

#include <vector>

#include "t12_device.h"
#include "t12_host.h"

namespace {

__global__ void copy_i32_kernel(int* __restrict__ dst, const int* __restrict__ src, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// A kernel that does nothing (hold_ticks == 0): the launch-interval probe below times a chain of them.  With
// hold_ticks > 0 its one wave waits that many ticks of the constant 100 MHz counter first (bounded by an iteration
// count as well): it holds the stream while the host enqueues the chain behind it.
__global__ void idle_kernel(int hold_ticks, int* __restrict__ sink)
{
    if (hold_ticks > 0) {
        const long long t0 = wall_clock64();
        for (int guard = 0; guard < (1 << 24) && wall_clock64() - t0 < hold_ticks; guard++) __builtin_amdgcn_s_sleep(16);
    }
    if (sink && threadIdx.x == 0xFFFF) *sink = 0;      // never true
}

// Shader-clock probe: what the chip clocks at under a given instruction mix.  Every workgroup (eight waves) runs
// `iters` rounds of four independent v_mfma_f32_32x32x16_bf16 per wave on pseudo-random operands; mix = 1 adds, per
// round and wave, what a decode+GEMM stage adds: two packed decodes of eight weights (t12_decode8), two 16-byte LDS
// writes and four 16-byte LDS reads.  Wave 0 of each workgroup reads the shader-clock counter (s_memtime) and the
// constant 100 MHz counter (s_memrealtime) before and after.
template <int MIX>
__global__ __launch_bounds__(512) void probe_clock_kernel(int iters, long long* __restrict__ stamps, float* __restrict__ sink)
{
    __shared__ __attribute__((aligned(16))) uint4 buf[2048];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t h = (blockIdx.x * 512u + tid) * 2654435761u + 12345u;
    auto next = [&]() { h ^= h << 13; h ^= h >> 17; h ^= h << 5; return h; };
    for (int i = tid; i < 2048; i += 512) buf[i] = make_uint4(next(), next(), next(), next());
    // bf16 operands with moderate exponents: sign and mantissa random
    auto operand = [&]() {
        uint4 v;
        v.x = (next() & 0x807F807Fu) | 0x3F003E80u;
        v.y = (next() & 0x807F807Fu) | 0x3E803F00u;
        v.z = (next() & 0x807F807Fu) | 0x3F003F00u;
        v.w = (next() & 0x807F807Fu) | 0x3E803E80u;
        return v;
    };
    uint4 A = operand(), W = operand();
    t12_f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;
    uint32_t s0 = next(), s1 = next(), g = next();
    const uint32_t be2 = t12_opaque((100u << 7) | (100u << 23));
    __syncthreads();
    const long long c0 = clock64(), r0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
        if (MIX) {
#pragma unroll
            for (int d = 0; d < 2; d++) {
                uint32_t w_[4];
                t12_decode8(s0 + d, s1 ^ d, g + it, be2, w_);
                buf[(wave * 128 + d * 64 + lane + it * 64) & 2047] = make_uint4(w_[0], w_[1], w_[2], w_[3]);
            }
            uint4 f = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint4 v = buf[(wave * 256 + d * 64 + lane + it * 192) & 2047];
                f.x ^= v.x; f.y ^= v.y; f.z ^= v.z; f.w ^= v.w;
            }
            W.x = (W.x & 0xFFFF0000u) | (f.x & 0x7Fu) | 0x3E80u;      // keeps the operand finite and the reads alive
            s0 += 0x01010101u;
            s1 ^= s0;
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(t12_bf16x8, A), __builtin_bit_cast(t12_bf16x8, W), acc[i], 0, 0, 0);
        A.y ^= 0x00010001u;
    }
    const long long c1 = clock64(), r1 = wall_clock64();
    float t = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) t += acc[i][r];
    if (t == 1234.5f) sink[tid] = t;                                  // never true: keeps the sums alive
    // wave 0 (served first on its SIMD) gives the clock; the last wave's end gives the duration
    if (tid == 0) {
        stamps[blockIdx.x * 4] = c1 - c0;
        stamps[blockIdx.x * 4 + 1] = r1 - r0;
        stamps[blockIdx.x * 4 + 2] = r0;
    }
    if (lane == 0) atomicMax((unsigned long long*)&stamps[blockIdx.x * 4 + 3], (unsigned long long)r1);
}

}  // namespace

extern "C" {

// Measurement aid (no counterpart in the reference): runs the probe above on `workgroups` workgroups of 512 threads and
// reports the shader clock they saw (GHz, mean over the workgroups) and the MFMA rate they reached (dense bf16
// TFLOP/s of the whole launch).  Synchronous; allocates and frees a few KB.  bench.py prints it next to the MFMA
// roofline: the 2.5 PFLOP/s peak is priced at 2.4 GHz, and the chip lowers its clock under load.
int t12_probe_clock(int workgroups, int iters, int mix, double* ghz, double* tflops, void* stream)
{
    T12_REQUIRE(workgroups >= 1 && workgroups <= 4096 && iters >= 1 && ghz && tflops, "t12_probe_clock: bad operands");
    hipStream_t st = (hipStream_t)stream;
    long long* d = nullptr;
    float* sink = nullptr;
    if (hipMalloc((void**)&d, sizeof(long long) * 4 * workgroups) != hipSuccess || hipMalloc((void**)&sink, 512 * sizeof(float)) != hipSuccess) {
        if (d) (void)hipFree(d);
        t12_set_error("t12_probe_clock: hipMalloc failed");
        return T12_ELAUNCH;
    }
    for (int rep = 0; rep < 2; rep++) {                                // the first launch warms the clocks up
        if (hipMemsetAsync(d, 0, sizeof(long long) * 4 * workgroups, st) != hipSuccess) break;
        if (mix) hipLaunchKernelGGL(probe_clock_kernel<1>, dim3(workgroups), dim3(512), 0, st, iters, d, sink);
        else hipLaunchKernelGGL(probe_clock_kernel<0>, dim3(workgroups), dim3(512), 0, st, iters, d, sink);
    }
    hipError_t e = hipGetLastError();
    std::vector<long long> h(4 * (size_t)workgroups);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e == hipSuccess) e = hipMemcpy(h.data(), d, sizeof(long long) * h.size(), hipMemcpyDeviceToHost);
    (void)hipFree(d);
    (void)hipFree(sink);
    if (e != hipSuccess) {
        t12_set_error("t12_probe_clock: %s", hipGetErrorString(e));
        return T12_ELAUNCH;
    }
    double sum_ghz = 0.0, max_ns = 0.0;
    for (int i = 0; i < workgroups; i++) {
        const double ns = (double)h[4 * i + 1] * 10.0;                  // 100 MHz counter
        sum_ghz += ns > 0.0 ? (double)h[4 * i] / ns : 0.0;
        const double dur = (double)(h[4 * i + 3] - h[4 * i + 2]) * 10.0;
        max_ns = dur > max_ns ? dur : max_ns;
    }
    *ghz = sum_ghz / workgroups;
    *tflops = max_ns > 0.0 ? 2.0 * 32 * 32 * 16 * 4.0 * 8 * (double)iters * workgroups / max_ns / 1e3 : 0.0;
    return T12_OK;
}

// Measurement aid (no counterpart in the reference): the interval between consecutive kernels of one stream, as
// the GPU's command processor paces them (the host's enqueue cost is kept out: a first kernel holds the stream
// for 4 us per launch while the host enqueues the whole chain behind it, and the clock runs from its end).
// Reports the time per launch of `launches` one-wave kernels that do nothing (us).  any_order = 0: the ordinary
// stream order, every kernel waits for the one before it -- the floor under any chain of dependent launches such
// as the B = 1 decode step.  any_order = 1: the launches carry hipExtAnyOrderLaunch, which lifts that ordering
// (such kernels overlap and may start before their predecessor has ended, so no launch whose input another launch
// of the chain writes may carry it): what the ordering itself costs.  Synchronous; allocates two events.
int t12_probe_launch_gap(int launches, int any_order, double* us_per_launch, void* stream)
{
    T12_REQUIRE(launches >= 1 && launches <= 20000 && us_per_launch, "t12_probe_launch_gap: launches must be 1..20000");
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        t12_set_error("t12_probe_launch_gap: hipEventCreate failed");
        return T12_ELAUNCH;
    }
    const int flags = any_order ? hipExtAnyOrderLaunch : 0;
    hipError_t e = hipSuccess;
    for (int rep = 0; rep < 2 && e == hipSuccess; rep++) {            // the first chain warms the queue up
        hipLaunchKernelGGL(idle_kernel, dim3(1), dim3(64), 0, st, launches * 400, (int*)nullptr);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipEventRecord(e0, st);
        for (int i = 0; i < launches && e == hipSuccess; i++) {
            hipExtLaunchKernelGGL(idle_kernel, dim3(1), dim3(64), 0, st, nullptr, nullptr, flags, 0, (int*)nullptr);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
    }
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess) {
        t12_set_error("t12_probe_launch_gap: %s", hipGetErrorString(e));
        return T12_ELAUNCH;
    }
    *us_per_launch = (double)ms * 1e3 / launches;
    return T12_OK;
}

// dst[0..n) = src[0..n) by a kernel (dst may be pinned host memory: a handful of ids reach the host
// without a DMA engine hand-over in the middle of the stream).
int t12_util_copy_i32(void* dst, const void* src, int n, void* stream)
{
    T12_REQUIRE(dst && src && n >= 1, "t12_util_copy_i32: bad operands");
    hipLaunchKernelGGL(copy_i32_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, (int*)dst,
                       (const int*)src, n);
    T12_CHECK_LAUNCH("t12_util_copy_i32");
    return T12_OK;
}

}  // extern "C"
