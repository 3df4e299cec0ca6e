// woq_dequantize: preprocessed weights -> row-major W[k, n] in fp16 / bf16 / fp8 e4m3, using the
// same device dequantize the GEMM main loop uses.  One wavefront per 1 KiB tile.
#include "dequant_math.h"

namespace woq
{

template <int DT, int BITS> // DT: WOQ_FP16 / WOQ_BF16 / WOQ_FP8_E4M3
__global__ void __launch_bounds__(256) dequant_kernel(void* out, void const* weight, void const* scales,
    void const* zeros, int k, int n, int group_size, int k_tiles, long total_tiles)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    constexpr int SLABS = TK / 32;
    constexpr int SDT = DT == WOQ_FP8_E4M3 ? WOQ_FP16 : DT; // type of scales / zeros
    long const tile = (long) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= total_tiles)
        return;
    int const lane = threadIdx.x & 63, c = lane & 15, kg = lane >> 4;
    int const strip = (int) (tile / k_tiles), kt = (int) (tile % k_tiles);
    int const col = strip * 16 + c;
    u32x4 const w = static_cast<u32x4 const*>(weight)[tile * 64 + lane];
#pragma unroll
    for (int j = 0; j < SLABS; ++j)
    {
        int const k0 = kt * TK + j * 32 + kg * 8;
        if (k0 >= k)
            continue;
        size_t const gi = group_size ? (size_t) (k0 / group_size) * n + col : (size_t) col;
        float const s = Elem<SDT>::load(scales, gi);
        float const z = zeros ? Elem<SDT>::load(zeros, gi) : 0.f;
        if constexpr (DT == WOQ_FP8_E4M3)
        {
            int q[8];
            if constexpr (BITS == 4)
                unpack_int4_signed(w[j], q);
            else
                unpack_int8_signed(w[2 * j], w[2 * j + 1], q);
            u32x2 const r = dequant8_fp8(q, s, z);
            uint8_t* o = static_cast<uint8_t*>(out);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                o[(size_t) (k0 + e) * n + col] = (uint8_t) (r[e >> 2] >> (8 * (e & 3)));
        }
        else
        {
            // the very function the GEMM main loop calls
            u32x4 r;
#pragma unroll
            for (int pr = 0; pr < 4; ++pr)
                r[pr] = dequant_operand_reg<DT, BITS>(w, j, pr, s, z);
            uint16_t* o = static_cast<uint16_t*>(out);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                o[(size_t) (k0 + e) * n + col] = (uint16_t) (r[e >> 1] >> (16 * (e & 1)));
        }
    }
}

template <int DT, int BITS>
static int run(void* out, void const* weight, void const* scales, void const* zeros, int k, int n, int group_size,
    hipStream_t s)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    int const k_tiles = (k + TK - 1) / TK;
    long const tiles = (long) k_tiles * (n / kTileN);
    dim3 grid((unsigned) ((tiles + 3) / 4)), block(256);
    hipLaunchKernelGGL((dequant_kernel<DT, BITS>), grid, block, 0, s, out, weight, scales, zeros, k, n, group_size,
        k_tiles, tiles);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "dequant kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

int launch_dequant(void* out, void const* weight, void const* scales, void const* zeros, int k, int n, int group_size,
    int bits, int dtype, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
#define WOQ_DQ(DT)                                                                                                     \
    return bits == 4 ? run<DT, 4>(out, weight, scales, zeros, k, n, group_size, s)                                     \
                     : run<DT, 8>(out, weight, scales, zeros, k, n, group_size, s);
    switch (dtype)
    {
    case WOQ_FP16: WOQ_DQ(WOQ_FP16)
    case WOQ_BF16: WOQ_DQ(WOQ_BF16)
    case WOQ_FP8_E4M3: WOQ_DQ(WOQ_FP8_E4M3)
    default: return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_dequantize: dtype %d", dtype);
    }
#undef WOQ_DQ
}

} // namespace woq
