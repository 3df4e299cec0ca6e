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

// ---- pair-granular form used by the GEMM main loop --------------------------------------------
// An MFMA B operand is 4 registers, register p holding elements (2p, 2p+1) of the slab.  The GEMM
// produces one such register at a time so the conversion work can be spread evenly between the
// matrix instructions.

// signed values of elements 2p and 2p+1 of an int4 dword; `t` is the dword XOR 0x88888888
// (biased nibbles -> two's complement); element 2p sits at nibble p, element 2p+1 at nibble p+4
__device__ __forceinline__ void int4_pair(uint32_t t, int p, int& q0, int& q1)
{
    q0 = (int) (t << (28 - 4 * p)) >> 28;
    q1 = (int) (t << (12 - 4 * p)) >> 28;
}

// signed values of elements 2p and 2p+1 of an int8 slab held in two dwords (bytes, biased by 128)
__device__ __forceinline__ void int8_pair(uint32_t w0, uint32_t w1, int p, int& q0, int& q1)
{
    uint32_t const w = p < 2 ? w0 : w1;
    int const sh = (p & 1) * 16;
    q0 = (int) ((w >> sh) & 0xFF) - 128;
    q1 = (int) ((w >> (sh + 8)) & 0xFF) - 128;
}

// The same two values divided by 16, as floats: v_cvt_off_f32_i4 converts the signed nibble in
// bits [3:0] of its operand to q/16, and a byte select on the source reaches the low nibble of any
// byte without a shift; the odd nibbles are the low nibbles of the bytes of t >> 4.  The caller
// multiplies by 16*s, so fma(q/16, 16*s, z) rounds the same real number as fma(q, s, z).
// (The byte select is written out: left to the compiler, a third of these conversions end up
// behind a separate bit-field extract.)
__device__ __forceinline__ float cvt_off_f32_i4_byte(uint32_t t, int byte)
{
    float x;
    switch (byte)
    {
    case 0: x = __builtin_amdgcn_cvt_off_f32_i4((int) t); break; // the instruction reads bits [3:0] only
    case 1: asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(x) : "v"(t)); break;
    case 2: asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(x) : "v"(t)); break;
    default: asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(x) : "v"(t)); break;
    }
    return x;
}

__device__ __forceinline__ void int4_pair_sixteenths(uint32_t t, int p, float& x0, float& x1)
{
    uint32_t const src = (p & 1) ? t >> 4 : t;
    x0 = cvt_off_f32_i4_byte(src, p >> 1);
    x1 = cvt_off_f32_i4_byte(src, 2 + (p >> 1));
}

// signed values of bytes 2h and 2h+1 of an int8 dword `t` (the stored dword XOR 0x80808080), as
// floats: sign-extending byte converts
__device__ __forceinline__ void int8_pair_float(uint32_t t, int h, float& x0, float& x1)
{
    x0 = (float) (int) (signed char) (t >> (16 * h));
    x1 = (float) (int) (signed char) (t >> (16 * h + 8));
}

// packed half-precision helpers on raw 32-bit pairs
__device__ __forceinline__ uint32_t half2_add(uint32_t a, float b)
{
    f16x2 const b2 = {(_Float16) b, (_Float16) b};
    return bit_cast<uint32_t>(bit_cast<f16x2>(a) + b2);
}

__device__ __forceinline__ uint32_t half2_fma(uint32_t a, uint32_t b, uint32_t c)
{
    return bit_cast<uint32_t>(__builtin_elementwise_fma(bit_cast<f16x2>(a), bit_cast<f16x2>(b), bit_cast<f16x2>(c)));
}

template <int DT>
__device__ __forceinline__ uint32_t dequant_pair(int q0, int q1, float s, float z);

template <>
__device__ __forceinline__ uint32_t dequant_pair<WOQ_BF16>(int q0, int q1, float s, float z)
{
    return Elem<WOQ_BF16>::pack(__builtin_fmaf((float) q0, s, z), __builtin_fmaf((float) q1, s, z));
}

template <>
__device__ __forceinline__ uint32_t dequant_pair<WOQ_FP16>(int q0, int q1, float s, float z)
{
    f16x2 const q2 = {(_Float16) q0, (_Float16) q1};
    f16x2 const s2 = {(_Float16) s, (_Float16) s};
    f16x2 const z2 = {(_Float16) z, (_Float16) z};
    return bit_cast<uint32_t>(__builtin_elementwise_fma(q2, s2, z2));
}

// register p (elements 2p, 2p+1) of the B operand of slab j of a lane's 16 packed bytes `w`
template <int DT, int BITS>
__device__ __forceinline__ uint32_t dequant_operand_reg(u32x4 const& w, int j, int p, float s, float z)
{
    int q0, q1;
    if constexpr (BITS == 4)
        int4_pair(w[j] ^ 0x88888888u, p, q0, q1);
    else
        int8_pair(w[2 * j], w[2 * j + 1], p, q0, q1);
    return dequant_pair<DT>(q0, q1, s, z);
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
