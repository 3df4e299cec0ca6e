// Activation pass behind the tiled kernels of the grouped matmul: out = f(in) elementwise, or for a
// gated activation out[m, n/2] = in[:, :n/2] * f(in[:, n/2:]).  The reference also has both forms:
// a fused gated kernel where one applies (MoeGemmRunner::isFusedGatedActivation,
// kernels/internal_cutlass_kernels/include/moe_gemm_kernels.h:255-257) and a separate pass
// otherwise.  Here the streaming kernel applies the activation in its own epilogue, the tiled
// kernels use this pass.  Computed in float32, one rounding to the output type.
#include "device_common.h"

namespace woq
{

template <int DT>
__global__ void __launch_bounds__(256) activation_kernel(
    void* out, void const* in, void const* residual, long m, int n_in, int act)
{
    using E = Elem<DT>;
    bool const gated = act_is_gated(act);
    int const n_out = gated ? n_in / 2 : n_in;
    // each thread owns 8 consecutive output columns (n_out % 8 == 0) and walks rows with a grid stride
    int const col8 = blockIdx.x * blockDim.x + threadIdx.x;
    if (col8 * 8 >= n_out)
        return;
    for (long row = blockIdx.y; row < m; row += gridDim.y)
    {
        uint16_t const* src = static_cast<uint16_t const*>(in) + row * n_in + (long) col8 * 8;
        long const o = row * n_out + (long) col8 * 8;
        u32x4 const x = *reinterpret_cast<u32x4 const*>(src);
        u32x4 const g = gated ? *reinterpret_cast<u32x4 const*>(src + n_out) : x;
        u32x4 const res = residual ? *reinterpret_cast<u32x4 const*>(static_cast<uint16_t const*>(residual) + o)
                                   : u32x4{0u, 0u, 0u, 0u}; // +0.0 in both 16-bit formats
        u32x4 y;
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float const lo = gated ? E::lo(x[r]) * apply_act(act, E::lo(g[r])) : apply_act(act, E::lo(x[r]));
            float const hi = gated ? E::hi(x[r]) * apply_act(act, E::hi(g[r])) : apply_act(act, E::hi(x[r]));
            y[r] = E::pack(lo + E::lo(res[r]), hi + E::hi(res[r]));
        }
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + o) = y;
    }
}

int launch_activation(void* out, void const* in, void const* residual, long m, int n_in, int act, int dtype,
    void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    int const n_out = act_is_gated(act) ? n_in / 2 : n_in;
    dim3 block(256), grid((n_out / 8 + 255) / 256, (unsigned) (m < 4096 ? m : 4096));
    if (dtype == WOQ_BF16)
        hipLaunchKernelGGL((activation_kernel<WOQ_BF16>), grid, block, 0, s, out, in, residual, m, n_in, act);
    else
        hipLaunchKernelGGL((activation_kernel<WOQ_FP16>), grid, block, 0, s, out, in, residual, m, n_in, act);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "activation kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

} // namespace woq
