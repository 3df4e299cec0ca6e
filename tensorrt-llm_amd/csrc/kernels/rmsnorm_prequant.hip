// RMSNorm fused with the smoothing pass in front of the matmul:
//     normed = T(x * rsqrt(mean(x^2) + eps) * gamma [+ beta])              (one rounding to T)
//     out    = T_out(T(normed * pre_quant_scale))                          (T_out = T or fp8 e4m3)
// i.e. invokeGeneralRmsNorm (kernels/rmsnormKernels.cu:29-38, 83-124, 230-262: float32 sum of
// squares, rsqrtf, float32 products, cast to T) followed by apply_per_channel_scale
// (kernels/preQuantScaleKernel.cu:42-149: one multiply rounded to T, optional saturating cast to
// e4m3) in ONE pass over the activations: the normalised tensor never goes to memory, and with fp8
// output only half as many bytes are written.  pre_quant_scale may be NULL (plain RMSNorm, or
// RMSNorm + cast).
// One workgroup of 256 threads per row; a row of up to 16384 elements stays in registers between
// the two phases (longer rows are read again, from L2); 16-byte loads and stores; sum of squares by
// wavefront butterfly + one LDS step.
#include "dequant_math.h"

namespace woq
{

template <int DT, bool TO_FP8, int CHUNKS>
__global__ void __launch_bounds__(256) rmsnorm_prequant_kernel(void* out, void const* x, void const* gamma,
    void const* beta, void const* scale, float eps, int k)
{
    using E = Elem<DT>;
    long const row = blockIdx.x;
    uint16_t const* src = static_cast<uint16_t const*>(x) + row * k;
    int const n8 = k / 8; // 16-byte pieces of a row; thread t owns pieces t, t + 256, ...

    u32x4 v[CHUNKS];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i)
    {
        int const piece = threadIdx.x + i * 256;
        v[i] = piece < n8 ? *reinterpret_cast<u32x4 const*>(src + (long) piece * 8) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float const a = E::lo(v[i][r]), b = E::hi(v[i][r]);
            ss = __builtin_fmaf(a, a, ss);
            ss = __builtin_fmaf(b, b, ss);
        }
    }
    for (int piece = threadIdx.x + CHUNKS * 256; piece < n8; piece += 256) // rows longer than CHUNKS * 2048
    {
        u32x4 const w = *reinterpret_cast<u32x4 const*>(src + (long) piece * 8);
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float const a = E::lo(w[r]), b = E::hi(w[r]);
            ss = __builtin_fmaf(a, a, ss);
            ss = __builtin_fmaf(b, b, ss);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        ss += __shfl_xor(ss, off, 64);
    __shared__ float part[4];
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float const inv = __frsqrt_rn((part[0] + part[1] + part[2] + part[3]) / (float) k + eps);

    auto finish = [&](u32x4 w, int piece)
    {
        u32x4 const g = static_cast<u32x4 const*>(gamma)[piece];
        u32x4 const b = beta ? static_cast<u32x4 const*>(beta)[piece] : u32x4{0u, 0u, 0u, 0u};
        u32x4 y;
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float lo = E::lo(w[r]) * inv * E::lo(g[r]), hi = E::hi(w[r]) * inv * E::hi(g[r]);
            if (beta)
            {
                lo += E::lo(b[r]);
                hi += E::hi(b[r]);
            }
            y[r] = E::pack(lo, hi);
        }
        if (scale)
        {
            u32x4 const sc = static_cast<u32x4 const*>(scale)[piece];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                y[r] = E::mul2(y[r], sc[r]);
        }
        if constexpr (TO_FP8)
        {
            int lo = 0, hi = 0;
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(y[0])), clamp_e4m3(E::hi(y[0])), lo, false);
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(y[1])), clamp_e4m3(E::hi(y[1])), lo, true);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(y[2])), clamp_e4m3(E::hi(y[2])), hi, false);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(E::lo(y[3])), clamp_e4m3(E::hi(y[3])), hi, true);
            u32x2 const o = {(uint32_t) lo, (uint32_t) hi};
            *reinterpret_cast<u32x2*>(static_cast<uint8_t*>(out) + row * k + (long) piece * 8) = o;
        }
        else
            *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + row * k + (long) piece * 8) = y;
    };
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i)
    {
        int const piece = threadIdx.x + i * 256;
        if (piece < n8)
            finish(v[i], piece);
    }
    for (int piece = threadIdx.x + CHUNKS * 256; piece < n8; piece += 256)
        finish(*reinterpret_cast<u32x4 const*>(src + (long) piece * 8), piece);
}

template <int DT, bool TO_FP8>
static void launch_chunks(void* out, void const* x, void const* gamma, void const* beta, void const* scale, float eps,
    int m, int k, hipStream_t s)
{
    dim3 grid((unsigned) m), block(256);
    int const pieces_per_thread = (k / 8 + 255) / 256;
    if (pieces_per_thread <= 2)
        hipLaunchKernelGGL((rmsnorm_prequant_kernel<DT, TO_FP8, 2>), grid, block, 0, s, out, x, gamma, beta, scale, eps, k);
    else if (pieces_per_thread <= 4)
        hipLaunchKernelGGL((rmsnorm_prequant_kernel<DT, TO_FP8, 4>), grid, block, 0, s, out, x, gamma, beta, scale, eps, k);
    else
        hipLaunchKernelGGL((rmsnorm_prequant_kernel<DT, TO_FP8, 8>), grid, block, 0, s, out, x, gamma, beta, scale, eps, k);
}

int launch_rmsnorm_prequant(void* out, void const* x, void const* gamma, void const* beta, void const* scale, float eps,
    int m, int k, int dtype, int out_dtype, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    bool const fp8 = out_dtype == WOQ_FP8_E4M3;
    if (dtype == WOQ_BF16)
        fp8 ? launch_chunks<WOQ_BF16, true>(out, x, gamma, beta, scale, eps, m, k, s)
            : launch_chunks<WOQ_BF16, false>(out, x, gamma, beta, scale, eps, m, k, s);
    else
        fp8 ? launch_chunks<WOQ_FP16, true>(out, x, gamma, beta, scale, eps, m, k, s)
            : launch_chunks<WOQ_FP16, false>(out, x, gamma, beta, scale, eps, m, k, s);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "rmsnorm kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

} // namespace woq
