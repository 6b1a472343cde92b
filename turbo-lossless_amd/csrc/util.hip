// Small utility kernels of the engine.

#include "t12_device.h"
#include "t12_host.h"

namespace {

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

}  // extern "C"
