// Standalone split-12 decompress: planes -> bf16 matrix, bit-exact (gfx950).
//
// out[i] = sign<<15 | (base_exp + group)<<7 | mantissa  for every flat element i,
// the function of the reference's nv_decode_split12_to_bf16
// (nvidia_kernels.cu:533-548); in patched mode the escapes (group 0) are then
// overwritten with their exact bf16 from the CSR list, which makes the result
// equal to the tensor that was packed (inverse of pack_split12,
// split12_pack.c:47-128).
// The decode is elementwise on the flat index, so the kernel ignores the row
// structure: a lane turns 16 B of sm + 8 B of gr into 32 B of bf16.
// HBM bound: 1.5 B read + 2 B written per weight.

#include "t12_device.h"
#include "t12_host.h"

namespace {

// 16 elements per lane per step; n16 = number of whole 16-element pieces.
__global__ __launch_bounds__(256) void decompress_vec_kernel(const uint8_t* __restrict__ sm,
                                                             const uint8_t* __restrict__ gr,
                                                             uint32_t be2, uint16_t* __restrict__ out,
                                                             size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    be2 = t12_opaque(be2);
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < n16; q += stride) {
        const uint4 S = t12_ldg_stream16(sm + q * 16);
        const uint2 G = t12_ldg_stream8(gr + q * 8);
        uint32_t a[4], b[4];
        t12_decode8(S.x, S.y, G.x, be2, a);     // a[i] = {w[i+4], w[i]}
        t12_decode8(S.z, S.w, G.y, be2, b);
        uint4 o0, o1;
        o0.x = __builtin_amdgcn_perm(a[1], a[0], 0x05040100u);   // {w1, w0}
        o0.y = __builtin_amdgcn_perm(a[3], a[2], 0x05040100u);   // {w3, w2}
        o0.z = __builtin_amdgcn_perm(a[1], a[0], 0x07060302u);   // {w5, w4}
        o0.w = __builtin_amdgcn_perm(a[3], a[2], 0x07060302u);   // {w7, w6}
        o1.x = __builtin_amdgcn_perm(b[1], b[0], 0x05040100u);
        o1.y = __builtin_amdgcn_perm(b[3], b[2], 0x05040100u);
        o1.z = __builtin_amdgcn_perm(b[1], b[0], 0x07060302u);
        o1.w = __builtin_amdgcn_perm(b[3], b[2], 0x07060302u);
        uint4* dst = (uint4*)(out + q * 16);
        t12_stg_stream16(dst, o0);
        t12_stg_stream16(dst + 1, o1);
    }
}

// The same with the escapes written in the same launch (patched mode, n % 16 == 0): a workgroup owns PIECES x 4096
// consecutive elements; the rows it touches are consecutive, so their CSR entries are one slice [e0, e1) of the list, and the
// workgroup overwrites those of them that fall into its own elements once its decoded values are stored (a barrier and
// a workgroup-scope fence in between; no other workgroup writes these addresses).
template <int PIECES>
__global__ __launch_bounds__(256) void decompress_patched_kernel(const uint8_t* __restrict__ sm,
                                                                 const uint8_t* __restrict__ gr, uint32_t be2,
                                                                 const int32_t* __restrict__ row_off,
                                                                 const int32_t* __restrict__ cols,
                                                                 const int16_t* __restrict__ correct,
                                                                 uint16_t* __restrict__ out, size_t n16, int M, int K)
{
    constexpr size_t CHUNK = (size_t)PIECES * 4096;
    const size_t c0 = (size_t)blockIdx.x * CHUNK;
    const size_t c1 = min(c0 + CHUNK, n16 * 16);
    const int r_lo = (int)(c0 / (size_t)K), r_hi = (int)((c1 - 1) / (size_t)K);
    // the slice of the list is requested before the planes: it is used last
    const int e0 = row_off[r_lo], e1 = row_off[r_hi + 1];
    be2 = t12_opaque(be2);
    uint4 S[PIECES];
    uint2 G[PIECES];
#pragma unroll
    for (int u = 0; u < PIECES; u++) {
        const size_t q = (size_t)blockIdx.x * (256 * PIECES) + u * 256 + threadIdx.x;
        if (q < n16) {
            S[u] = t12_ldg_stream16(sm + q * 16);
            G[u] = t12_ldg_stream8(gr + q * 8);
        }
    }
#pragma unroll
    for (int u = 0; u < PIECES; u++) {
        const size_t q = (size_t)blockIdx.x * (256 * PIECES) + u * 256 + threadIdx.x;
        if (q < n16) {
            uint32_t a[4], b[4];
            t12_decode8(S[u].x, S[u].y, G[u].x, be2, a);
            t12_decode8(S[u].z, S[u].w, G[u].y, be2, b);
            uint4 o0, o1;
            o0.x = __builtin_amdgcn_perm(a[1], a[0], 0x05040100u);
            o0.y = __builtin_amdgcn_perm(a[3], a[2], 0x05040100u);
            o0.z = __builtin_amdgcn_perm(a[1], a[0], 0x07060302u);
            o0.w = __builtin_amdgcn_perm(a[3], a[2], 0x07060302u);
            o1.x = __builtin_amdgcn_perm(b[1], b[0], 0x05040100u);
            o1.y = __builtin_amdgcn_perm(b[3], b[2], 0x05040100u);
            o1.z = __builtin_amdgcn_perm(b[1], b[0], 0x07060302u);
            o1.w = __builtin_amdgcn_perm(b[3], b[2], 0x07060302u);
            uint4* dst = (uint4*)(out + q * 16);
            t12_stg_stream16(dst, o0);
            t12_stg_stream16(dst + 1, o1);
        }
    }
    if (e0 == e1) return;                                // (workgroup-uniform)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    int r = r_lo;
    for (int p = e0 + (int)threadIdx.x; p < e1; p += 256) {
        while (r < r_hi && row_off[r + 1] <= p) r++;     // entries ascend with the rows: the cursor only moves forward
        const size_t flat = (size_t)r * K + cols[p];
        if (flat >= c0 && flat < c1) out[flat] = (uint16_t)correct[p];
    }
}

// Scalar rule for what the vector kernel cannot take: the tail (n % 16), a
// base_exp outside 0..240, unaligned outputs.  Elements [first, n).
__global__ __launch_bounds__(256) void decompress_scalar_kernel(const uint8_t* __restrict__ sm,
                                                                const uint8_t* __restrict__ gr,
                                                                int base_exp, uint16_t* __restrict__ out,
                                                                size_t first, size_t n)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = first + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t g = (gr[i >> 1] >> (4 * (i & 1))) & 0xFu;
        out[i] = t12_decode_scalar(sm[i], g, base_exp);
    }
}

// One wave per row writes that row's exact values.
__global__ __launch_bounds__(256) void scatter_escapes_kernel(const int32_t* __restrict__ row_off,
                                                              const int32_t* __restrict__ cols,
                                                              const int16_t* __restrict__ correct,
                                                              uint16_t* __restrict__ out, int M, int K)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int beg = row_off[row], end = row_off[row + 1];
    for (int p = beg + (threadIdx.x & 63); p < end; p += T12_WAVE)
        out[(size_t)row * K + cols[p]] = (uint16_t)correct[p];
}

}  // namespace

extern "C" int t12_decompress(const void* sm, const void* gr, int base_exp, const void* row_off,
                              const void* cols, const void* correct, void* out_bf16,
                              int M, int K, int patched, void* stream)
{
    T12_REQUIRE(M >= 0 && K >= 0, "t12_decompress: negative shape %d x %d", M, K);
    if (M == 0 || K == 0) return T12_OK;
    T12_REQUIRE(sm && gr && out_bf16, "t12_decompress: null plane or output");
    T12_REQUIRE(base_exp >= -1 && base_exp <= 254, "t12_decompress: base_exp %d out of range", base_exp);
    T12_REQUIRE(!patched || !row_off || (cols && correct), "t12_decompress: row_off given without cols/correct");
    hipStream_t st = (hipStream_t)stream;
    const size_t n = (size_t)M * K;
    const bool vec_ok = base_exp >= 0 && base_exp <= 240 && ((uintptr_t)sm % 16 == 0) &&
                        ((uintptr_t)gr % 8 == 0) && ((uintptr_t)out_bf16 % 16 == 0);
    const size_t n16 = vec_ok ? n / 16 : 0;
    if (n16 && n16 * 16 == n && patched && row_off && (n + 4095) / 4096 <= 0x7FFFFFFFull) {
        const uint32_t be2 = ((uint32_t)base_exp << 7) | ((uint32_t)base_exp << 23);
        // one 16-element piece per lane: two and four pieces in flight per lane measured 5-8 % slower (42.6 / 43.3 us
        // against 40.5 on 14336 x 4096)
        hipLaunchKernelGGL(decompress_patched_kernel<1>, dim3((unsigned)((n + 4095) / 4096)), dim3(256), 0, st, (const uint8_t*)sm,
                           (const uint8_t*)gr, be2, (const int32_t*)row_off, (const int32_t*)cols, (const int16_t*)correct,
                           (uint16_t*)out_bf16, n16, M, K);
        T12_CHECK_LAUNCH("t12_decompress(patched)");
        return T12_OK;
    }
    if (n16) {
        const uint32_t be2 = ((uint32_t)base_exp << 7) | ((uint32_t)base_exp << 23);
        const size_t want = (n16 + 255) / 256;
        const int blocks = (int)(want < 256 * 64 ? want : 256 * 64);
        hipLaunchKernelGGL(decompress_vec_kernel, dim3(blocks), dim3(256), 0, st, (const uint8_t*)sm,
                           (const uint8_t*)gr, be2, (uint16_t*)out_bf16, n16);
        T12_CHECK_LAUNCH("t12_decompress(vec)");
    }
    if (n16 * 16 < n) {
        const size_t rest = n - n16 * 16;
        const size_t want = (rest + 255) / 256;
        const int blocks = (int)(want < 256 * 64 ? want : 256 * 64);
        hipLaunchKernelGGL(decompress_scalar_kernel, dim3(blocks), dim3(256), 0, st, (const uint8_t*)sm,
                           (const uint8_t*)gr, base_exp, (uint16_t*)out_bf16, n16 * 16, n);
        T12_CHECK_LAUNCH("t12_decompress(scalar)");
    }
    if (patched && row_off) {
        hipLaunchKernelGGL(scatter_escapes_kernel, dim3((M + 3) / 4), dim3(256), 0, st, (const int32_t*)row_off,
                           (const int32_t*)cols, (const int16_t*)correct, (uint16_t*)out_bf16, M, K);
        T12_CHECK_LAUNCH("t12_decompress(escapes)");
    }
    return T12_OK;
}
