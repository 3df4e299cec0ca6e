// Device-side building blocks shared by the gfx950 kernels of libwoq: vector types, 16-bit float
// helpers, the int4/int8 -> MFMA-operand extractors and the 16x16x32 matrix-core wrappers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../woq_internal.h"

namespace woq
{

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <typename To, typename From>
__device__ __forceinline__ To bit_cast(From const& v)
{
    static_assert(sizeof(To) == sizeof(From), "size mismatch");
    return __builtin_bit_cast(To, v);
}

// ---- per-dtype traits ----------------------------------------------------------------------
// MAGIC4: OR-ed onto an isolated nibble pair it yields two 16-bit floats of value BASE4 + u
//         (bf16: 0x4300 = 128.0 with ulp 1; fp16: 0x6400 = 1024.0 with ulp 1).
template <int DT>
struct Elem;

template <>
struct Elem<WOQ_BF16>
{
    static constexpr uint32_t kMagic4 = 0x43004300u;
    static constexpr float kBase4 = 128.f;
    static constexpr uint32_t kOnes = 0x3F803F80u;
    static constexpr float kBase8 = 0.f; // int8 goes through an exact float conversion: value u

    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bit_cast<bf16x8>(a), bit_cast<bf16x8>(b), c, 0, 0, 0);
    }

    // c += a x b with the accumulator tied to ONE AGPR quad.  The builtin leaves destination and
    // addend independent; with 256 live accumulator registers the allocator then renames them
    // along the K loop and pays for it with hundreds of AGPR<->VGPR copies per step.  (A and B
    // operands written by ordinary VALU instructions need no software wait states before an
    // MFMA; the result must not be read by VALU code until the MFMA has drained - see
    // mma_drain().)
    static __device__ __forceinline__ void mma_acc(u32x4 a, u32x4 b, f32x4& c)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }

    // c = a x b: the first product of a new sum (the old value of c is dead: no input operand for it)
    static __device__ __forceinline__ void mma_first(u32x4 a, u32x4 b, f32x4& c)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }

    static __device__ __forceinline__ float lo(uint32_t pair)
    {
        return bit_cast<float>(pair << 16);
    }

    static __device__ __forceinline__ float hi(uint32_t pair)
    {
        return bit_cast<float>(pair & 0xFFFF0000u);
    }

    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        bf16x2 r;
        r[0] = (__bf16) a; // round to nearest even (v_cvt_pk_bf16_f32)
        r[1] = (__bf16) b;
        return bit_cast<uint32_t>(r);
    }

    static __device__ __forceinline__ float load(void const* p, size_t i)
    {
        return bit_cast<float>((uint32_t) static_cast<uint16_t const*>(p)[i] << 16);
    }

    static __device__ __forceinline__ uint16_t store(float v)
    {
        return bit_cast<uint16_t>((__bf16) v);
    }

    static __device__ __forceinline__ float from_bits(uint16_t b)
    {
        return bit_cast<float>((uint32_t) b << 16);
    }

    // elementwise product of two packed pairs, rounded once to the type
    static __device__ __forceinline__ uint32_t mul2(uint32_t a, uint32_t b)
    {
        return pack(lo(a) * lo(b), hi(a) * hi(b));
    }
};

template <>
struct Elem<WOQ_FP16>
{
    static constexpr uint32_t kMagic4 = 0x64006400u;
    static constexpr float kBase4 = 1024.f;
    static constexpr uint32_t kOnes = 0x3C003C00u;
    static constexpr float kBase8 = 1024.f; // int8 uses the byte-permute form 0x6400 | u

    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<f16x8>(a), bit_cast<f16x8>(b), c, 0, 0, 0);
    }

    static __device__ __forceinline__ void mma_acc(u32x4 a, u32x4 b, f32x4& c)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }

    static __device__ __forceinline__ void mma_first(u32x4 a, u32x4 b, f32x4& c)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }

    static __device__ __forceinline__ float lo(uint32_t pair)
    {
        return (float) bit_cast<f16x2>(pair)[0];
    }

    static __device__ __forceinline__ float hi(uint32_t pair)
    {
        return (float) bit_cast<f16x2>(pair)[1];
    }

    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        f16x2 r;
        r[0] = (_Float16) a;
        r[1] = (_Float16) b;
        return bit_cast<uint32_t>(r);
    }

    static __device__ __forceinline__ float load(void const* p, size_t i)
    {
        return (float) static_cast<_Float16 const*>(p)[i];
    }

    static __device__ __forceinline__ uint16_t store(float v)
    {
        return bit_cast<uint16_t>((_Float16) v);
    }

    static __device__ __forceinline__ float from_bits(uint16_t b)
    {
        return (float) bit_cast<_Float16>(b);
    }

    static __device__ __forceinline__ uint32_t mul2(uint32_t a, uint32_t b)
    {
        return bit_cast<uint32_t>(bit_cast<f16x2>(a) * bit_cast<f16x2>(b));
    }
};

// Wait until every MFMA issued through mma_acc() has written its result: the compiler cannot
// see that those asm statements are matrix instructions, so the wait states it would insert
// before the first VALU read of an accumulator are inserted here (16 passes at most).
__device__ __forceinline__ void mma_drain()
{
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
}

// ---- packed weights -> MFMA B operand holding (BASE + u) exactly ---------------------------
// int4: dword `w` holds elements e at nibble (e even ? e/2 : 4 + e/2); operand register i is
// the pair (element 2i, element 2i+1).
// The nibble mask and the exponent pattern as values the compiler cannot see through.  With
// literal constants it emits v_and + v_or (a VOP3 encoding cannot carry 32-bit literals on gfx9);
// with the mask in an SGPR and the pattern in a VGPR it selects the fused v_and_or_b32 itself,
// and - unlike hand-written asm in the data path - still sees every VALU->MFMA dependency it has
// to schedule around.
struct NibbleConsts
{
    uint32_t mask;  // 0x000F000F, in an SGPR
    uint32_t magic; // Elem<DT>::kMagic4, in a VGPR
};

template <int DT>
__device__ __forceinline__ NibbleConsts nibble_consts()
{
    NibbleConsts c;
    c.mask = 0x000F000Fu;
    c.magic = Elem<DT>::kMagic4;
    asm volatile("" : "+s"(c.mask));
    asm volatile("" : "+v"(c.magic));
    return c;
}

template <int DT>
__device__ __forceinline__ u32x4 expand_int4(uint32_t w, NibbleConsts const& c)
{
    u32x4 r;
    r[0] = (w & c.mask) | c.magic;
    r[1] = ((w >> 4) & c.mask) | c.magic;
    r[2] = ((w >> 8) & c.mask) | c.magic;
    r[3] = ((w >> 12) & c.mask) | c.magic;
    return r;
}

// int8: two dwords hold elements 0..3 and 4..7 as bytes.
template <int DT>
__device__ __forceinline__ u32x4 expand_int8(uint32_t w0, uint32_t w1);

template <>
__device__ __forceinline__ u32x4 expand_int8<WOQ_BF16>(uint32_t w0, uint32_t w1)
{
    // 0..255 is exact in bf16 (8 significant bits); v_cvt_f32_ubyteN then a packed bf16 convert
    u32x4 r;
    r[0] = Elem<WOQ_BF16>::pack((float) (w0 & 0xFF), (float) ((w0 >> 8) & 0xFF));
    r[1] = Elem<WOQ_BF16>::pack((float) ((w0 >> 16) & 0xFF), (float) (w0 >> 24));
    r[2] = Elem<WOQ_BF16>::pack((float) (w1 & 0xFF), (float) ((w1 >> 8) & 0xFF));
    r[3] = Elem<WOQ_BF16>::pack((float) ((w1 >> 16) & 0xFF), (float) (w1 >> 24));
    return r;
}

template <>
__device__ __forceinline__ u32x4 expand_int8<WOQ_FP16>(uint32_t w0, uint32_t w1)
{
    // byte permute builds [u, 0x64] pairs: fp16 1024 + u, exact for u <= 1023
    constexpr uint32_t K = 0x64646464u;
    u32x4 r;
    r[0] = __builtin_amdgcn_perm(K, w0, 0x04010400u);
    r[1] = __builtin_amdgcn_perm(K, w0, 0x04030402u);
    r[2] = __builtin_amdgcn_perm(K, w1, 0x04010400u);
    r[3] = __builtin_amdgcn_perm(K, w1, 0x04030402u);
    return r;
}

// one register of the above: `half` 0 -> bytes 0,1 of w, 1 -> bytes 2,3
template <int DT>
__device__ __forceinline__ uint32_t expand_int8_reg(uint32_t w, int half)
{
    if constexpr (DT == WOQ_BF16)
        return half == 0 ? Elem<WOQ_BF16>::pack((float) (w & 0xFF), (float) ((w >> 8) & 0xFF))
                         : Elem<WOQ_BF16>::pack((float) ((w >> 16) & 0xFF), (float) (w >> 24));
    else
        return __builtin_amdgcn_perm(0x64646464u, w, half == 0 ? 0x04010400u : 0x04030402u);
}

// additive constant carried by the expanded operand: expanded value = q + kOffset
template <int DT, int BITS>
struct Offset
{
    static constexpr float value = BITS == 4 ? Elem<DT>::kBase4 + 8.f : Elem<DT>::kBase8 + 128.f;
};

// ---- buffer (descriptor-based) loads: out-of-range accesses return 0 ---------------------------
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(void const* base, uint32_t bytes)
{
    // raw buffer (stride 0): num_records counts bytes; 0x00020000 = 32-bit untyped data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int) bytes, 0x00020000);
}

__device__ __forceinline__ u32x4 buffer_load_x4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset)
{
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int) byte_offset, 0, 0);
}

// The same load with the non-temporal hint, for data a launch reads exactly once - the packed weights of the
// streaming kernels.  Lines fetched this way are not kept in the caches at the expense of what is reused
// (activations, scales) and the fetch itself is cheaper: measured on MI355X, one row, 8192 x 57344 42.9 ->
// 39.0 us (0.80 of 8 TB/s, above what a plain read with ordinary loads reaches), 4096 x 28672 12.5 -> 12.0.
__device__ __forceinline__ u32x4 buffer_load_x4_once(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset)
{
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int) byte_offset, 0, 2 /* nt */);
}

__device__ __forceinline__ u32x2 buffer_load_x2(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset)
{
    return __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int) byte_offset, 0, 0);
}

__device__ __forceinline__ uint16_t buffer_load_u16(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset)
{
    return __builtin_amdgcn_raw_buffer_load_b16(rsrc, (int) byte_offset, 0, 0);
}

// ---- row of the scale / zero tables -----------------------------------------------------------------
// Group sizes that are multiples of 64 above 128 ("flexible" group sizes, what the reference's Hopper
// kernels accept) have kernel instantiations of their own, GROUP = kFlexGroup: scales are applied per
// 64 rows of K as for groups of 64, and only the row of the [ceil(k / group), n] tables follows the
// real group size: `magic` = ceil(2^32 / (group / 64)), an exact division by multiplication for every
// row index that can occur.  (Serving them from the GROUP = 64 instantiations through a run-time test
// cost those 10-30 %: their table addresses no longer folded into immediate offsets.)
constexpr int kFlexGroup = 1;

// rows of K that share one scale inside a tile of TK rows
template <int GROUP, int TK>
constexpr int segment_rows()
{
    return GROUP == 0 ? TK : GROUP == kFlexGroup ? 64 : (GROUP > TK ? TK : GROUP);
}

// rows per group as far as sizes computed on the host go (the segment length for flexible groups)
constexpr int host_group_rows(int group)
{
    return group == kFlexGroup ? 64 : group;
}

template <int GROUP>
__device__ __forceinline__ uint32_t scale_row(uint32_t k_row, uint32_t magic)
{
    if constexpr (GROUP == kFlexGroup)
        return __umulhi(k_row >> 6, magic);
    else
        return k_row / (uint32_t) (GROUP != 0 ? GROUP : 1);
}

// host side: the magic of a group size (0 unless it is a multiple of 64 above 128)
inline uint32_t scale_row_magic(int group_size)
{
    if (group_size <= 128 || group_size % 64)
        return 0;
    uint64_t const d = (uint64_t) group_size / 64;
    return (uint32_t) ((((uint64_t) 1 << 32) + d - 1) / d);
}

// the kernel instantiation that serves a group size: 0 / 64 / 128 themselves, kFlexGroup for larger multiples of 64
inline int template_group(int group_size)
{
    return group_size <= 128 ? group_size : kFlexGroup;
}

// ---- epilogue activations (values of the reference's ActivationType,
// kernels/internal_cutlass_kernels/include/moe_gemm_kernels.h:197-206) -------------------------
constexpr int kActGelu = 0, kActRelu = 1, kActSilu = 2, kActSwiglu = 3, kActGeglu = 4, kActIdentity = 5;

__host__ __device__ __forceinline__ bool act_is_gated(int act)
{
    return act == kActSwiglu || act == kActGeglu;
}

// erf by Abramowitz & Stegun 7.1.26 (|error| < 1.5e-7, far below the 16-bit output rounding)
__device__ __forceinline__ float erf_approx(float x)
{
    float const ax = __builtin_fabsf(x);
    float const t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, ax, 1.f));
    float poly = __builtin_fmaf(1.061405429f, t, -1.453152027f);
    poly = __builtin_fmaf(poly, t, 1.421413741f);
    poly = __builtin_fmaf(poly, t, -0.284496736f);
    poly = __builtin_fmaf(poly, t, 0.254829592f);
    float const r = 1.f - poly * t * __expf(-ax * ax);
    return __builtin_copysignf(r, x);
}

// the non-gated function of an activation (Swiglu -> silu, Geglu -> gelu), in float32 as the
// reference's epilogues compute it (fused_moe_kernel_routine.cuh:393-400)
__device__ __forceinline__ float apply_act(int act, float v)
{
    if (act == kActGelu || act == kActGeglu)
        return 0.5f * v * (1.f + erf_approx(v * 0.70710678118654752f));
    if (act == kActRelu)
        return __builtin_fmaxf(v, 0.f);
    if (act == kActSilu || act == kActSwiglu)
        return v * __builtin_amdgcn_rcpf(1.f + __expf(-v));
    return v;
}

// A pointer (or count) that is the same in every lane but was computed from loaded values: moved
// into scalar registers, so that buffer descriptors built from it stay scalar too.
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* ptr)
{
    uint64_t const v = reinterpret_cast<uint64_t>(ptr);
    uint32_t const lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) v);
    uint32_t const hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (v >> 32));
    return reinterpret_cast<T*>(((uint64_t) hi << 32) | lo);
}

// Workgroups are handed to the 8 XCDs round-robin.  Mapping block b to
// strip (b % 8) * strips_per_xcd + b / 8 keeps neighbouring 16-column strips (which share
// 128-byte lines of the scale / zero rows) on one XCD, hence in one L2.
// v + (v of the lane a DPP control selects); every lane of the 16-lane row must be active
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    int const x = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return v + __builtin_bit_cast(float, x);
}

__device__ __forceinline__ int xcd_strip(int block, int strips_per_xcd)
{
    return (block & 7) * strips_per_xcd + (block >> 3);
}

} // namespace woq
