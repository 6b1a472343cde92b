// Device-side helpers shared by the split-12 kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(2))) __bf16 t12_bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 t12_bf16x8;
typedef __attribute__((ext_vector_type(4))) float t12_f32x4;
typedef __attribute__((ext_vector_type(16))) float t12_f32x16;

#define T12_WAVE 64

__device__ __forceinline__ float t12_bf16_to_f32(uint16_t b)
{
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// float -> bf16 bits, round to nearest even, no NaN special case: the rounding
// rule of the reference's float_to_bf16 (engine/kernels.hip:21-27).
__device__ __forceinline__ uint16_t t12_f32_to_bf16(float v)
{
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// The scalar decode rule (decompress_v2.hip:192): works for every base_exp,
// including -1, because the sum is truncated to 16 bits exactly as there.
__device__ __forceinline__ uint16_t t12_decode_scalar(uint32_t sm, uint32_t g, int base_exp)
{
    return (uint16_t)(((sm >> 7) << 15) | ((uint32_t)(base_exp + (int)g) << 7) | (sm & 0x7Fu));
}

// ---------------------------------------------------------------------------
// Packed decode of 8 consecutive weights.
//   s0 = sm bytes 0..3, s1 = sm bytes 4..7, g = their eight nibbles (nibble i in
//   bits 4i+3..4i), be2 = (base_exp << 7) | (base_exp << 23) with 0 <= base_exp <= 240,
//   passed through t12_opaque() once by the caller.
// Result w[i] = bf16x2 { weight i (low half), weight i+4 (high half) }, i = 0..3.
// Pairing i with i+4 puts both nibbles of a pair exactly 16 bits apart, so one
// AND isolates both exponents offsets of a pair and one shift-add rebases them:
// the "1-ADD" exponent rebase, done for two weights at once.  base_exp + group
// <= 255, so the add never carries out of the exponent field.
// Cost: per pair 1 v_perm_b32 + 1 v_and_or_b32 + 1 v_and_b32 (+1 shift for the
// two right-shifted pairs) + 1 v_lshl_add_u32/v_add_u32.
// ---------------------------------------------------------------------------
// An empty asm that makes a value opaque to the optimiser without emitting an
// instruction.  Used to keep (g & mask) in the form that selects to
// v_and_b32 + v_lshl_add_u32, and to keep the rebased-exponent constant in a
// VGPR so that (m & keep) | be2 selects to one v_and_or_b32.  No real
// instruction hides in inline asm: every VALU result that feeds an MFMA is
// written by an instruction the compiler's hazard recogniser can see (a VALU
// write inside an asm block followed directly by an MFMA reading it is a
// hardware hazard the compiler does not pad).
__device__ __forceinline__ uint32_t t12_opaque(uint32_t v)
{
    asm("" : "+v"(v));
    return v;
}

// be2v must come from t12_opaque(be2) (a VGPR).
__device__ __forceinline__ void t12_decode8(uint32_t s0, uint32_t s1, uint32_t g, uint32_t be2v,
                                            uint32_t w[4])
{
    // v_perm_b32: selector bytes 0-3 pick from the 2nd operand, 4-7 from the 1st.
    const uint32_t m0 = __builtin_amdgcn_perm(s1, s0, 0x04040000u);
    const uint32_t m1 = __builtin_amdgcn_perm(s1, s0, 0x05050101u);
    const uint32_t m2 = __builtin_amdgcn_perm(s1, s0, 0x06060202u);
    const uint32_t m3 = __builtin_amdgcn_perm(s1, s0, 0x07070303u);
    // byte duplicated in both bytes of its half: keep sign (bit 15) + mantissa (bits 6..0)
    const uint32_t keep = 0x807F807Fu;
    const uint32_t t0 = (m0 & keep) | be2v;
    const uint32_t t1 = (m1 & keep) | be2v;
    const uint32_t t2 = (m2 & keep) | be2v;
    const uint32_t t3 = (m3 & keep) | be2v;
    w[0] = (t12_opaque(g & 0x000F000Fu) << 7) + t0;
    w[1] = (t12_opaque(g & 0x00F000F0u) << 3) + t1;
    w[2] = ((g >> 1) & 0x07800780u) + t2;
    w[3] = ((g >> 5) & 0x07800780u) + t3;
}

// Activations that pair with t12_decode8: from 8 consecutive bf16 (x0..x7 in four
// dwords) build a[i] = { x_i (low), x_{i+4} (high) }.
__device__ __forceinline__ uint4 t12_pair_acts(uint4 v)
{
    uint4 r;
    r.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);   // {x4, x0}
    r.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);   // {x5, x1}
    r.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);   // {x6, x2}
    r.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);   // {x7, x3}
    return r;
}

__device__ __forceinline__ float t12_dot2(uint32_t w, uint32_t a, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(t12_bf16x2, w),
                                           __builtin_bit_cast(t12_bf16x2, a), acc, false);
}

// 8 weights x 8 paired activations -> accumulate.
__device__ __forceinline__ float t12_decode_dot8(uint32_t s0, uint32_t s1, uint32_t g, uint32_t be2,
                                                 uint4 a, float acc)
{
    uint32_t w[4];
    t12_decode8(s0, s1, g, be2, w);
    acc = t12_dot2(w[0], a.x, acc);
    acc = t12_dot2(w[1], a.y, acc);
    acc = t12_dot2(w[2], a.z, acc);
    acc = t12_dot2(w[3], a.w, acc);
    return acc;
}

// Wave-wide sum, result valid in every lane (xor butterfly through ds_bpermute).
__device__ __forceinline__ float t12_wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, T12_WAVE);
    return v;
}

// Wave-wide sum by DPP row operations; the total is valid in lane 63 only.
__device__ __forceinline__ float t12_wave_sum_lane63(float v)
{
#define T12_DPP_ADD(ctrl, rmask)                                                               \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), \
                                                               (ctrl), (rmask), 0xF, true))
    T12_DPP_ADD(0xB1, 0xF);    // quad_perm [1,0,3,2]
    T12_DPP_ADD(0x4E, 0xF);    // quad_perm [2,3,0,1]
    T12_DPP_ADD(0x141, 0xF);   // row_half_mirror
    T12_DPP_ADD(0x140, 0xF);   // row_mirror: every lane of a 16-lane row holds the row sum
    T12_DPP_ADD(0x142, 0xA);   // row_bcast15 into rows 1 and 3
    T12_DPP_ADD(0x143, 0xC);   // row_bcast31 into rows 2 and 3
#undef T12_DPP_ADD
    return v;
}

// streaming (read-once) loads: keep the weight planes from displacing the
// activations in L2
typedef __attribute__((ext_vector_type(4))) uint32_t t12_u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t t12_u32x2;

__device__ __forceinline__ uint4 t12_ldg_stream16(const void* p)
{
    const t12_u32x4 v = __builtin_nontemporal_load((const t12_u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 t12_ldg_stream8(const void* p)
{
    const t12_u32x2 v = __builtin_nontemporal_load((const t12_u32x2*)p);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ void t12_stg_stream16(void* p, uint4 v)
{
    t12_u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, (t12_u32x4*)p);
}
