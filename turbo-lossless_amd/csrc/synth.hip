// Seeded synthetic tensors generated on the GPU (counter based, so the value of
// element i depends only on (seed, i) and not on the launch shape).

#include "t12_device.h"
#include "t12_host.h"

namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;                 // splitmix64 finaliser
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ float normal_from(uint64_t r)
{
    const float u1 = ((float)(uint32_t)(r >> 40) + 0.5f) * (1.0f / 16777216.0f);   // (0, 1)
    const float u2 = ((float)(uint32_t)((r >> 16) & 0xFFFFFFu)) * (1.0f / 16777216.0f);
    return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);                    // Box-Muller
}

// out[i] = bf16( N(0, sigma) ), or with probability p_out bf16( N(0, sigma_out) ).
__global__ __launch_bounds__(256) void normal_bf16_kernel(uint16_t* __restrict__ out, size_t n, uint64_t seed,
                                                          float sigma, float p_out, float sigma_out)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t a = mix64(seed * 0xD1342543DE82EF95ull + i);
        const uint64_t b = mix64(a);
        const float pick = (float)(uint32_t)(b >> 40) * (1.0f / 16777216.0f);
        const float s = pick < p_out ? sigma_out : sigma;
        out[i] = t12_f32_to_bf16(normal_from(a) * s);
    }
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ out, size_t n, float v)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = v;
}

}  // namespace

extern "C" {

int t12_synth_normal_bf16(void* out_bf16, size_t n, uint64_t seed, float sigma, float p_outlier, float sigma_outlier,
                          void* stream)
{
    T12_REQUIRE(out_bf16 || n == 0, "t12_synth_normal_bf16: null output");
    if (n == 0) return T12_OK;
    const size_t want = (n + 255) / 256;
    const int blocks = (int)(want < 256 * 32 ? want : 256 * 32);
    hipLaunchKernelGGL(normal_bf16_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out_bf16, n,
                       seed, sigma, p_outlier, sigma_outlier);
    T12_CHECK_LAUNCH("t12_synth_normal_bf16");
    return T12_OK;
}

int t12_fill_f32(void* out, size_t n, float value, void* stream)
{
    T12_REQUIRE(out || n == 0, "t12_fill_f32: null output");
    if (n == 0) return T12_OK;
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (float*)out, n, value);
    T12_CHECK_LAUNCH("t12_fill_f32");
    return T12_OK;
}

}  // extern "C"
