// The one definition of "dequantize" used on the device (by woq_dequantize and by the GEMM main
// loop), matching the CPU oracle bit for bit:
//   fp16 : w = fma_f16(q, s, z)                    one rounding (a half-precision FMA, as the
//                                                  reference's `fma2` in the activation type,
//                                                  weightOnlyBatchedGemv/utility.h:157-162)
//   bf16 : w = bf16_rn(fma_f32(q, s, z))           float32 FMA, then round to nearest even
//   fp8  : w = e4m3_rn_sat(fma_f32(q, s_h, z_h))   W4A8: scales/zeros are fp16 values
// q is the exact signed integer.
#pragma once

#include "device_common.h"

namespace woq
{

// signed values of the 8 elements of int4 dword `w` (biased storage, element e at nibble
// (e even ? e/2 : 4 + e/2)), natural element order
__device__ __forceinline__ void unpack_int4_signed(uint32_t w, int (&q)[8])
{
    uint32_t const t = w ^ 0x88888888u; // biased -> two's complement nibbles
#pragma unroll
    for (int e = 0; e < 8; ++e)
    {
        int const slot = (e & 1) ? 4 + (e >> 1) : (e >> 1);
        q[e] = (int) (t << (28 - 4 * slot)) >> 28; // v_bfe_i32
    }
}

__device__ __forceinline__ void unpack_int8_signed(uint32_t w0, uint32_t w1, int (&q)[8])
{
#pragma unroll
    for (int e = 0; e < 4; ++e)
    {
        q[e] = (int) ((w0 >> (8 * e)) & 0xFF) - 128;
        q[4 + e] = (int) ((w1 >> (8 * e)) & 0xFF) - 128;
    }
}

__device__ __forceinline__ float clamp_e4m3(float v)
{
    return __builtin_fminf(__builtin_fmaxf(v, -448.f), 448.f);
}

// 8 dequantized values -> packed operand: 4 dwords of 16-bit pairs (fp16 / bf16)
template <int DT>
__device__ __forceinline__ u32x4 dequant8(int const (&q)[8], float s, float z);

template <>
__device__ __forceinline__ u32x4 dequant8<WOQ_BF16>(int const (&q)[8], float s, float z)
{
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        r[i] = Elem<WOQ_BF16>::pack(
            __builtin_fmaf((float) q[2 * i], s, z), __builtin_fmaf((float) q[2 * i + 1], s, z));
    return r;
}

template <>
__device__ __forceinline__ u32x4 dequant8<WOQ_FP16>(int const (&q)[8], float s, float z)
{
    // s and z are fp16 values carried in float; the FMA itself is done in half precision
    f16x2 const s2 = {(_Float16) s, (_Float16) s};
    f16x2 const z2 = {(_Float16) z, (_Float16) z};
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        f16x2 const q2 = {(_Float16) q[2 * i], (_Float16) q[2 * i + 1]};
        r[i] = bit_cast<uint32_t>(__builtin_elementwise_fma(q2, s2, z2));
    }
    return r;
}

// one int4 dword (8 elements of one MFMA slab) -> the slab's B operand
template <int DT>
__device__ __forceinline__ u32x4 dequant_int4_dword(uint32_t w, float s, float z)
{
    int q[8];
    unpack_int4_signed(w, q);
    return dequant8<DT>(q, s, z);
}

// two int8 dwords (8 elements of one MFMA slab) -> the slab's B operand
template <int DT>
__device__ __forceinline__ u32x4 dequant_int8_dwords(uint32_t w0, uint32_t w1, float s, float z)
{
    int q[8];
    unpack_int8_signed(w0, w1, q);
    return dequant8<DT>(q, s, z);
}

// 8 dequantized values -> 8 e4m3 bytes (2 dwords), element order preserved
__device__ __forceinline__ u32x2 dequant8_fp8(int const (&q)[8], float s, float z)
{
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
        v[e] = clamp_e4m3(__builtin_fmaf((float) q[e], s, z));
    u32x2 r = {0, 0};
    r[0] = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], (int) r[0], false);
    r[0] = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], (int) r[0], true);
    r[1] = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], (int) r[1], false);
    r[1] = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], (int) r[1], true);
    return r;
}

} // namespace woq
