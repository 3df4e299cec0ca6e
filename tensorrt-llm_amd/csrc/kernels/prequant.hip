// out[m, k] = T_out(T_in(act[m, k] * scale[k])): the AWQ smoothing pass in front of the GEMM
// regime (the streaming kernel fuses it instead).  Behaviour of
// apply_per_channel_scale_kernel_launcher<T_in, T_out> (kernels/preQuantScaleKernel.cu:42-149):
// one multiply rounded to the input type, then an optional saturating cast to fp8 e4m3.
#include "dequant_math.h"

namespace woq
{

template <int DT, bool TO_FP8>
__global__ void __launch_bounds__(256) prequant_kernel(void* out, void const* act, void const* scale, long m, int k)
{
    using E = Elem<DT>;
    // each thread owns 8 consecutive columns (k % 8 == 0) and walks rows with a grid stride
    int const col8 = blockIdx.x * blockDim.x + threadIdx.x;
    if (col8 * 8 >= k)
        return;
    u32x4 const sc = static_cast<u32x4 const*>(scale)[col8];
    for (long row = blockIdx.y; row < m; row += gridDim.y)
    {
        u32x4 a = *reinterpret_cast<u32x4 const*>(static_cast<uint16_t const*>(act) + row * k + (long) col8 * 8);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            a[r] = E::mul2(a[r], sc[r]);
        if constexpr (TO_FP8)
        {
            int lo = 0, hi = 0;
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(a[0])), clamp_e4m3(E::hi(a[0])), lo, false);
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(a[1])), clamp_e4m3(E::hi(a[1])), lo, true);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(a[2])), clamp_e4m3(E::hi(a[2])), hi, false);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(a[3])), clamp_e4m3(E::hi(a[3])), hi, true);
            u32x2 const o = {(uint32_t) lo, (uint32_t) hi};
            *reinterpret_cast<u32x2*>(static_cast<uint8_t*>(out) + row * k + (long) col8 * 8) = o;
        }
        else
            *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + row * k + (long) col8 * 8) = a;
    }
}

int launch_prequant(void* out, void const* act, void const* scale, int m, int k, int in_dtype, int out_dtype,
    void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    dim3 block(256), grid((k / 8 + 255) / 256, (unsigned) (m < 4096 ? m : 4096));
    bool const fp8 = out_dtype == WOQ_FP8_E4M3;
    if (in_dtype == WOQ_BF16 && fp8)
        hipLaunchKernelGGL((prequant_kernel<WOQ_BF16, true>), grid, block, 0, s, out, act, scale, (long) m, k);
    else if (in_dtype == WOQ_BF16)
        hipLaunchKernelGGL((prequant_kernel<WOQ_BF16, false>), grid, block, 0, s, out, act, scale, (long) m, k);
    else if (fp8)
        hipLaunchKernelGGL((prequant_kernel<WOQ_FP16, true>), grid, block, 0, s, out, act, scale, (long) m, k);
    else
        hipLaunchKernelGGL((prequant_kernel<WOQ_FP16, false>), grid, block, 0, s, out, act, scale, (long) m, k);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "pre-quant scale kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

} // namespace woq
