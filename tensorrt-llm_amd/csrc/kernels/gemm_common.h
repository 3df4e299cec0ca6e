// Pieces shared by the two MFMA GEMM kernels (exact-dequantize prefill kernel, deferred-scale
// skinny kernel): the parameter block, the workgroup -> tile order and the split-K helpers.
#pragma once

#include "device_common.h"

namespace woq
{

struct GemmParams
{
    void const* act;
    void const* weight;
    void const* scales;
    void const* zeros;
    void const* bias;
    void* out;
    float alpha;
    int m, n, k;
    int k_tiles; // ceil(k / TILE_K)
    int strips;  // n / 16
    int tiles_m, tiles_n;
    int k_splits;        // workgroups along K per output tile (blockIdx.y)
    int tiles_per_split; // tile rows of K each of them covers
    float* partial;      // [m, n] float32, zeroed, when k_splits > 1
};

constexpr int kGemmBN = 256; // columns of an output tile (4 wavefronts x 64)

// Output tiles are numbered m-fastest inside a column panel; the 8 XCDs each take one contiguous
// chunk of that order (workgroup i runs on XCD i % 8), so the workgroups that share weight
// columns or activation rows also share an L2.
__device__ __forceinline__ bool xcd_tile(int total, int& t)
{
    int const per_xcd = (total + 7) / 8;
    t = (int) (blockIdx.x & 7) * per_xcd + (int) (blockIdx.x >> 3);
    return (int) (blockIdx.x >> 3) < per_xcd && t < total;
}

// split-K helpers: clear the float32 partial buffer, then out = T(alpha * partial + bias)
template <int DT>
__global__ void __launch_bounds__(256) gemm_zero_partial(float* partial, size_t count)
{
    size_t const i = ((size_t) blockIdx.x * 256 + threadIdx.x) * 4;
    if (i < count)
        *reinterpret_cast<f32x4*>(partial + i) = f32x4{0.f, 0.f, 0.f, 0.f}; // count is a multiple of 16
}

template <int DT>
__global__ void __launch_bounds__(256) gemm_finish_partial(
    void* out, float const* partial, void const* bias, float alpha, int m, int n)
{
    using E = Elem<DT>;
    size_t const i = (size_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t) m * n)
        return;
    int const col = (int) (i % n);
    float const b = bias ? E::load(bias, col) : 0.f;
    static_cast<uint16_t*>(out)[i] = E::store(__builtin_fmaf(alpha, partial[i], b));
}

} // namespace woq
