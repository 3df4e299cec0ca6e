// Pieces shared by the W4A8 kernels: the exact int4 -> e4m3 dequantize and the fp8 matrix instruction.
#pragma once

#include "dequant_math.h"
#include "device_common.h"

namespace woq
{

// elements 4h+2p, 4h+2p+1 of slab dword `w` -> 2 e4m3 bytes in 16-bit word p of `old` (a dword of
// the B operand holds elements 4h .. 4h+3 in order; the other word is kept).
// CLAMP = false is for kernels that run with fp8_saturation_on(): the conversion instruction then
// saturates by itself and the clamp (a quarter of the instructions) is not needed.
// With zero-points the weight is fma(q, s, z) on the two's-complement nibble.  Without them
// q * s = fma(u, s, -8 s) on the stored nibble u = q + 8: -8 s is exact, so this is the same
// single rounding, and u comes out of a byte-to-float conversion with no sign extension.
template <bool ZERO, bool CLAMP = true>
__device__ __forceinline__ uint32_t dequant2_fp8(uint32_t old, uint32_t w, int h, int p, float s, float z)
{
    float v0, v1;
    // elements e0 = 4h + 2p and e0 + 1 sit in nibble slots e0/2 and 4 + e0/2
    if constexpr (ZERO)
    {
        // q/16 straight from the nibble (see int4_pair_sixteenths), times 16 s: the same rounding.
        // Slots e0/2 and 4 + e0/2 are the low nibbles of bytes h and h+2 of t (p = 0) or t >> 4 (p = 1).
        uint32_t const t = w ^ 0x88888888u; // biased -> two's complement nibbles
        uint32_t const src = p == 0 ? t : t >> 4;
        float const s16 = 16.f * s;
        v0 = __builtin_fmaf(cvt_off_f32_i4_byte(src, h), s16, z);
        v1 = __builtin_fmaf(cvt_off_f32_i4_byte(src, h + 2), s16, z);
    }
    else
    {
        // slots e0/2 and 4 + e0/2 are bytes h and h+2 of the even-nibble word (p = 0) or of the
        // odd-nibble word (p = 1).  The masked word is made opaque so that the byte-to-float
        // conversions read it (the compiler would otherwise extract each 4-bit field from w).
        uint32_t m = (p == 0 ? w : (w >> 4)) & 0x0F0F0F0Fu;
        asm volatile("" : "+v"(m));
        float const m8s = -8.f * s;
        v0 = __builtin_fmaf((float) ((m >> (8 * h)) & 0xFF), s, m8s);
        v1 = __builtin_fmaf((float) ((m >> (8 * h + 16)) & 0xFF), s, m8s);
    }
    if constexpr (CLAMP) // saturation to +-448 in software; off when the conversion itself saturates
    {
        v0 = clamp_e4m3(v0);
        v1 = clamp_e4m3(v1);
    }
    return p == 0 ? (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, (int) old, false)
                  : (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, (int) old, true);
}

// One dword of the B operand (elements 4h .. 4h+3 of slab dword `w`), same arithmetic
// (`nib`: nibble_consts<WOQ_FP16>(), the mask 0x000F000F and 1024 as a pair of halves in registers).  CLAMP =
// false leaves the saturation to +-448 out: for callers that know 8|s| + |z| stays below it.
template <bool ZERO, bool CLAMP>
__device__ __forceinline__ uint32_t dequant4_fp8(uint32_t w, int h, float s, float z, NibbleConsts const& nib)
{
    float v[4]; // elements 4h, 4h+1, 4h+2, 4h+3: nibble slots 2h, 4+2h, 2h+1, 5+2h
    if constexpr (ZERO)
    {
        uint32_t const t = w ^ 0x88888888u, t4 = t >> 4; // biased -> two's complement nibbles
        float const s16 = 16.f * s;
        v[0] = __builtin_fmaf(cvt_off_f32_i4_byte(t, h), s16, z);
        v[1] = __builtin_fmaf(cvt_off_f32_i4_byte(t, h + 2), s16, z);
        v[2] = __builtin_fmaf(cvt_off_f32_i4_byte(t4, h), s16, z);
        v[3] = __builtin_fmaf(cvt_off_f32_i4_byte(t4, h + 2), s16, z);
    }
    else
    {
        // slots 2h and 4+2h (elements 4h, 4h+1) are 16 bits apart, and so are slots 2h+1 and 5+2h
        // (elements 4h+2, 4h+3).  One and-or turns the first pair into two halves 0x6400 | u = 1024 + u,
        // which the FMA reads directly: q s = fma(1024 + u, s, -1032 s) with u = q + 8.  The second
        // pair is taken where it sits, four bits up, still inside the half's ten fraction bits:
        // 0x6400 | 16 u = 1024 + 16 u, and q s = fma(1024 + 16 u, s / 16, -72 s) - no shift.  The
        // constants (s / 16, 1032 s, 72 s) and the result are exact in float32, so either form is
        // fma(q, s, 0) bit for bit.
        uint32_t const wh = w >> (8 * h);
        f16x2 const p0 = bit_cast<f16x2>((wh & nib.mask) | nib.magic);
        f16x2 const p1 = bit_cast<f16x2>((wh & (nib.mask << 4)) | nib.magic);
        float const c = -1032.f * s, s16 = 0.0625f * s, c16 = -72.f * s;
        v[0] = __builtin_fmaf((float) p0[0], s, c);
        v[1] = __builtin_fmaf((float) p0[1], s, c);
        v[2] = __builtin_fmaf((float) p1[0], s16, c16);
        v[3] = __builtin_fmaf((float) p1[1], s16, c16);
    }
    if constexpr (CLAMP)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            v[i] = clamp_e4m3(v[i]);
    }
    // the first conversion overwrites a register that is dead anyway (v[0]'s), the second fills
    // the other half of it
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], bit_cast<int>(v[0]), false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], r, true);
    return (uint32_t) r;
}

// ---- table form of the same dequantize (the decode kernels) ----------------------------------------
// A (group, column) has only sixteen possible results e4m3(fma(u - 8, s, z)), u = 0 .. 15 the stored
// nibble.  The four lanes (kg = 0 .. 3) that hold one column of a tile each convert four of them - the
// same FMA and the same saturating conversion instruction as dequant4_fp8, so the bytes are identical -
// and exchange their quarters; every weight is then a byte looked up with v_perm_b32: 13 instructions
// per eight weights instead of 17-22, plus 12 per tile for the table.  Requires fp8_saturation_on().
struct Fp8Table
{
    uint32_t t[4]; // entries 4 i .. 4 i + 3 in dword i, entry u in byte u % 4
};

// qf[i] = float(4 kg + i - 8): the signed values of the lane's four table entries
__device__ __forceinline__ void fp8_table_lane_values(int kg, float (&qf)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i)
        qf[i] = (float) (4 * kg + i - 8);
}

__device__ __forceinline__ Fp8Table build_fp8_table(float s, float z, float const (&qf)[4])
{
    float const v0 = __builtin_fmaf(qf[0], s, z), v1 = __builtin_fmaf(qf[1], s, z);
    float const v2 = __builtin_fmaf(qf[2], s, z), v3 = __builtin_fmaf(qf[3], s, z);
    int d = __builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, 0, false);
    d = __builtin_amdgcn_cvt_pk_fp8_f32(v2, v3, d, true);
    // all-gather over the four rows of sixteen lanes: D = the lane's own quarter, D_r that of row r
    auto const r = __builtin_amdgcn_permlane16_swap((uint32_t) d, (uint32_t) d, false, false); // [D0 D0 D2 D2], [D1 D1 D3 D3]
    auto const e = __builtin_amdgcn_permlane32_swap(r[0], r[0], false, false);                   // D0 everywhere, D2 everywhere
    auto const o = __builtin_amdgcn_permlane32_swap(r[1], r[1], false, false);                   // D1 everywhere, D3 everywhere
    return Fp8Table{{e[0], o[0], e[1], o[1]}};
}

// Constants of the look-up as values the compiler cannot see through: with literals it emits v_and + v_or
// (a VOP3 encoding carries no 32-bit literal on gfx9); with the mask in an SGPR and the byte numbers in a
// VGPR it selects the fused v_and_or_b32 (as NibbleConsts does for the 16-bit kernels).
struct Fp8LookupConsts
{
    uint32_t low3;  // 0x07070707, SGPR
    uint32_t bit2;  // 0x04040404, SGPR
    uint32_t bytes; // 0x03020100, VGPR
};

__device__ __forceinline__ Fp8LookupConsts fp8_lookup_consts()
{
    Fp8LookupConsts k{0x07070707u, 0x04040404u, 0x03020100u};
    asm volatile("" : "+s"(k.low3));
    asm volatile("" : "+s"(k.bit2));
    asm volatile("" : "+v"(k.bytes));
    return k;
}

// The eight weights of slab dword `w` (element e in nibble e even ? e / 2 : 4 + e / 2) -> two operand
// dwords in the order the nibbles sit in: bytes [e0, e4, e1, e5] and [e2, e6, e3, e7].  The A operand
// has to present its eight k-values in the same order (fp8_a_order).
__device__ __forceinline__ void fp8_lookup8(uint32_t w, Fp8Table const& T, Fp8LookupConsts const& k, uint32_t& b0, uint32_t& b1)
{
    uint32_t const sel_e = w & k.low3, sel_o = (w >> 4) & k.low3; // entry % 8 of the low / high nibbles
    uint32_t const lo_e = __builtin_amdgcn_perm(T.t[1], T.t[0], sel_e), hi_e = __builtin_amdgcn_perm(T.t[3], T.t[2], sel_e);
    uint32_t const lo_o = __builtin_amdgcn_perm(T.t[1], T.t[0], sel_o), hi_o = __builtin_amdgcn_perm(T.t[3], T.t[2], sel_o);
    // bit 3 of each nibble picks the upper half of the table: byte j from lo (selector j) or hi (4 + j)
    uint32_t const pick_e = ((w >> 1) & k.bit2) | k.bytes;
    uint32_t const pick_o = ((w >> 5) & k.bit2) | k.bytes;
    b0 = __builtin_amdgcn_perm(hi_e, lo_e, pick_e);
    b1 = __builtin_amdgcn_perm(hi_o, lo_o, pick_o);
}

// eight consecutive k-values (bytes a0 .. a7 in v0, v1) in the order fp8_lookup8 delivers the weights
__device__ __forceinline__ void fp8_a_order(uint32_t v0, uint32_t v1, uint32_t& a0, uint32_t& a1)
{
    a0 = __builtin_amdgcn_perm(v1, v0, 0x05010400u); // [a0, a4, a1, a5]
    a1 = __builtin_amdgcn_perm(v1, v0, 0x07030602u); // [a2, a6, a3, a7]
}

// MODE.FP16_OVFL (bit 23 of the wavefront's MODE register) makes v_cvt_pk_fp8_f32 saturate finite
// overflow to +-448 instead of producing NaN - the rounding the W4A8 dequantize is defined with.
// The bit also makes fp16 results clamp instead of overflowing to infinity, so it is switched off
// again before an epilogue converts outputs: pass every value that a later conversion reads
// through after_mode_change() so that the conversion cannot be scheduled before the switch
// (volatile asm statements keep their order).  MODE is per wavefront and set from the kernel
// descriptor at launch: nothing leaks into other kernels.
__device__ __forceinline__ void fp8_saturation_on()
{
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1\n\ts_nop 3" ::: "memory");
}

__device__ __forceinline__ void fp8_saturation_off()
{
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 0\n\ts_nop 3" ::: "memory");
}

template <typename T>
__device__ __forceinline__ T after_mode_change(T v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// The other side of the switch: pass every sum that the conversions feed through before_mode_change()
// in front of fp8_saturation_off().  The statement needs the finished sum, so everything the sum depends on
// - the matrix instructions and, through them, the conversions - stays in front of it, and volatile asm
// statements keep their order: no conversion can be scheduled behind the switch.  (In straight-line code
// nothing else holds them there: the one-pass row kernel with seven tiles per wavefront had its last
// conversions moved behind the switch and returned NaN for saturating scales.)
__device__ __forceinline__ void before_mode_change(float& v)
{
    asm volatile("" : "+v"(v));
}
__device__ __forceinline__ void before_mode_change(f32x4& v)
{
    asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
}

// Row of the [ceil(k / group_size), n] scale / zero tables that the 128-row tile row kt reads.  Groups
// are multiples of 128 (the reference's Hopper kernels take any multiple of their K tile for e4m3
// activations, launchers/fpA_intB_launcher_sm90.inl:190-198; the last group may be shorter): `magic` is 0
// for groups of 128 (row = tile row) and ceil(2^32 / (group_size / 128)) otherwise, an exact division by
// multiplication for every tile row that can occur.
__device__ __forceinline__ uint32_t w4a8_scale_row(uint32_t kt, uint32_t magic)
{
    return magic ? __umulhi(kt, magic) : kt;
}

inline uint32_t w4a8_scale_row_magic(int group_size)
{
    uint64_t const d = (uint64_t) group_size / 128;
    return d <= 1 ? 0u : (uint32_t) ((((uint64_t) 1 << 32) + d - 1) / d);
}

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

// c += a x b (32 e4m3 values per lane each), accumulator tied to one AGPR quad (see Elem::mma_acc)
__device__ __forceinline__ void mma_fp8_acc(u32x8 a, u32x8 b, f32x4& c)
{
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// c = a x b: the first product of a new sum (the old value of c is dead: no input operand for it)
__device__ __forceinline__ void mma_fp8_first(u32x8 a, u32x8 b, f32x4& c)
{
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
}

} // namespace woq
