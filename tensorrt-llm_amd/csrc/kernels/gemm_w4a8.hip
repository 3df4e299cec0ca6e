// W4A8: fp8 (e4m3) activations x int4 weights on the CDNA4 fp8 matrix core.
//
// Semantics of the reference's W4A8 path (fpA_intB runner instantiated for __nv_fp8_e4m3 x uint4
// with half scales, cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h,
// selected by weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): the int4 weight is dequantized
// with fp16 scales/zeros and rounded to e4m3, the MMA accumulates fp8 x fp8 products in float32,
// and the epilogue applies alpha and the bias: out = T(alpha * acc + bias).  Group size 128 only.
//
// First version of this kernel: 4 wavefronts per workgroup in a 2 x 2 arrangement, 128 x 128
// output tile, each wavefront 64 rows x 64 columns.  Packed weights go straight from global
// memory into the registers of the lane that feeds them to the matrix core (same tile layout
// as the 16-bit kernels: 8 k-values per lane per MFMA); activation fragments are read directly
// from global memory / L2 (8 bytes per lane per MFMA), no LDS staging yet.
#include "dequant_math.h"

namespace woq
{

struct W4A8Params
{
    void const* act; // [m, k] e4m3
    void const* weight;
    void const* scales; // [k/128, n] fp16
    void const* zeros;  // [k/128, n] fp16 or null
    void const* bias;   // [n] out dtype or null
    void* out;          // [m, n] out dtype
    float alpha;
    int m, n, k, k_tiles, strips, tiles_m, tiles_n;
};

template <int ODT, bool ZERO>
__global__ void __launch_bounds__(256) gemm_w4a8_kernel(W4A8Params p)
{
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    constexpr int TK = 128, SLABS = 4, RT = 4, NS = 4;
    int const tile = blockIdx.x;
    int const tm = tile % p.tiles_m, tn = tile / p.tiles_m;
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const m0 = tm * 128 + (wave & 1) * 64;
    int const strip0 = tn * 8 + (wave >> 1) * NS;
    int const K = p.k, KT = p.k_tiles;

    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K);
    uint32_t const sz_bytes = (uint32_t) (K / 128) * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) KT * 1024u);

    int strip_of[NS];
    uint32_t wlane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        strip_of[s] = strip0 + s < p.strips ? strip0 + s : p.strips - 1;
        wlane[s] = ((uint32_t) strip_of[s] * (uint32_t) KT * 64u + (uint32_t) lane) * 16u;
    }

    f32x4 acc[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc[rt][s] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int kt = 0; kt < KT; ++kt)
    {
        u32x4 w[NS];
        float sc[NS], zr[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            w[s] = buffer_load_x4(w_rsrc, wlane[s] + (uint32_t) kt * 1024u);
            uint32_t const off = ((uint32_t) kt * (uint32_t) p.n + (uint32_t) (strip_of[s] * 16 + c)) * 2u;
            sc[s] = EH::from_bits(buffer_load_u16(sc_rsrc, off));
            zr[s] = ZERO ? EH::from_bits(buffer_load_u16(zr_rsrc, off)) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
        {
            // rows >= m and k >= K read as zero through the descriptor
            int const kk = kt * TK + j * 32 + kg * 8;
            u32x2 a[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                uint32_t const row = (uint32_t) (m0 + rt * 16 + c);
                uint32_t const off = kk < K ? row * (uint32_t) K + (uint32_t) kk : 0x80000000u;
                a[rt] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(act_rsrc, (int) off, 0, 0));
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                int q[8];
                unpack_int4_signed(w[s][j], q);
                u32x2 const b = dequant8_fp8(q, sc[s], zr[s]);
                long const bl = __builtin_bit_cast(long, b);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    acc[rt][s] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(
                        __builtin_bit_cast(long, a[rt]), bl, acc[rt][s], 0, 0, 0);
            }
        }
    }

    uint16_t* out16 = static_cast<uint16_t*>(p.out);
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        if (strip0 + s >= p.strips)
            continue;
        int const col = (strip0 + s) * 16 + c;
        float const bias = p.bias ? EO::load(p.bias, col) : 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                int const row = m0 + rt * 16 + kg * 4 + r;
                if (row < p.m)
                    out16[(size_t) row * p.n + col] = EO::store(__builtin_fmaf(p.alpha, acc[rt][s][r], bias));
            }
    }
}

int launch_gemm_w4a8(MatmulProblem const& p, void* stream)
{
    W4A8Params gp;
    gp.act = p.act;
    gp.weight = p.weight;
    gp.scales = p.scales;
    gp.zeros = p.zeros;
    gp.bias = p.bias;
    gp.out = p.out;
    gp.alpha = p.alpha;
    gp.m = p.m;
    gp.n = p.n;
    gp.k = p.k;
    gp.k_tiles = (p.k + 127) / 128;
    gp.strips = p.n / kTileN;
    gp.tiles_m = (p.m + 127) / 128;
    gp.tiles_n = (p.n + 127) / 128;
    dim3 grid(gp.tiles_m * gp.tiles_n), block(256);
    auto s = static_cast<hipStream_t>(stream);
    bool const zero = p.zeros != nullptr;
    if (p.out_dtype == WOQ_BF16)
    {
        if (zero)
            hipLaunchKernelGGL((gemm_w4a8_kernel<WOQ_BF16, true>), grid, block, 0, s, gp);
        else
            hipLaunchKernelGGL((gemm_w4a8_kernel<WOQ_BF16, false>), grid, block, 0, s, gp);
    }
    else
    {
        if (zero)
            hipLaunchKernelGGL((gemm_w4a8_kernel<WOQ_FP16, true>), grid, block, 0, s, gp);
        else
            hipLaunchKernelGGL((gemm_w4a8_kernel<WOQ_FP16, false>), grid, block, 0, s, gp);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "W4A8 gemm kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

} // namespace woq
