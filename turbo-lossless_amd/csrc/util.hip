// Plain streaming kernels of known traffic: the yardsticks the benchmark and the
// profiler counters are calibrated against (what a pure HBM read / copy reaches
// on this chip with the same load instructions the split-12 kernels use).

#include "t12_device.h"
#include "t12_host.h"

namespace {

// Reads n16 16-byte pieces; folds them so the loads cannot be dropped; one
// 4-byte store per workgroup.
__global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ src, size_t n16,
                                                   uint32_t* __restrict__ sink)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
    size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; q + 3 * stride < n16; q += 4 * stride) {
        const uint4 a = t12_ldg_stream16(src + q);
        const uint4 b = t12_ldg_stream16(src + q + stride);
        const uint4 c = t12_ldg_stream16(src + q + 2 * stride);
        const uint4 d = t12_ldg_stream16(src + q + 3 * stride);
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; q < n16; q += stride) {
        const uint4 a = t12_ldg_stream16(src + q);
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    acc ^= __shfl_xor(acc, 32, 64);
    if (acc == 0x9E3779B9u || threadIdx.x == 0) sink[blockIdx.x] = acc;   // data dependent: loads stay
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                   size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < n16; q += stride)
        t12_stg_stream16(dst + q, t12_ldg_stream16(src + q));
}

__global__ void copy_i32_kernel(int* __restrict__ dst, const int* __restrict__ src, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

}  // namespace

extern "C" {

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

// Streams `bytes` (a multiple of 16) from src; sink must hold `blocks` uint32.
int t12_util_read(const void* src, size_t bytes, void* sink, int blocks, void* stream)
{
    T12_REQUIRE(src && sink && bytes % 16 == 0 && blocks >= 1, "t12_util_read: bad operands");
    hipLaunchKernelGGL(read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src, bytes / 16,
                       (uint32_t*)sink);
    T12_CHECK_LAUNCH("t12_util_read");
    return T12_OK;
}

// dst[0..bytes) = src[0..bytes), bytes a multiple of 16.
int t12_util_copy(void* dst, const void* src, size_t bytes, int blocks, void* stream)
{
    T12_REQUIRE(src && dst && bytes % 16 == 0 && blocks >= 1, "t12_util_copy: bad operands");
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src, (uint4*)dst,
                       bytes / 16);
    T12_CHECK_LAUNCH("t12_util_copy");
    return T12_OK;
}

}  // extern "C"
