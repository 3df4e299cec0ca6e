// Measurement probes: what the hardware allows, measured with the same harness as the kernels
// (bench.py --mode ceilings).  No counterpart in the reference.
//   woq_probe_read   plain streaming read of a buffer: every lane one 16-byte load per KiB, a wavefront
//                    reads `kib_per_wave` contiguous KiB with `U` loads in flight, ordinary loads or loads
//                    with the non-temporal hint (what the streaming kernels read their weights with) - the
//                    HBM ceiling the weight-streaming kernels are measured against
//   woq_probe_empty  a kernel that does nothing: the cost of a launch
//   woq_probe_mfma   nothing but matrix instructions on every SIMD: the matrix-core ceiling, with
//                    constant or with pseudo-random operands
#include <hip/hip_runtime.h>

#include "../woq_probes.h"
#include "device_common.h"

namespace woq
{
namespace
{
template <int U, bool NT>
__global__ void __launch_bounds__(256) probe_read_kernel(u32x4 const* __restrict__ src, size_t kib_per_wave, size_t waves,
    unsigned* sink)
{
    size_t const wave = (size_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= waves)
        return;
    u32x4 const* q = src + wave * kib_per_wave * 64 + (threadIdx.x & 63);
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = 0; i < kib_per_wave; i += U)
    {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            v[u] = NT ? __builtin_nontemporal_load(q + (i + u) * 64) : q[(i + u) * 64];
#pragma unroll
        for (int u = 0; u < U; ++u)
            acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) // never true for the benchmark's data: keeps the loads
        sink[wave & 1023] = 1;
}

__global__ void probe_empty_kernel(unsigned* sink)
{
    if (sink == nullptr)
        sink[0] = 1;
}

// 16 independent accumulators per wavefront, ITERS rounds: the matrix core never waits for a result.
// RANDOM = false: every instruction multiplies the same two operand registers (the least switching
// activity the matrix core can see); true: four operand pairs of pseudo-random finite values per
// lane, taken in turn, so that consecutive instructions toggle the operand buses as real data does -
// the rate then shows what the power management sustains under a realistic load.
template <int KIND, bool RANDOM>
__global__ void __launch_bounds__(256) probe_mfma_kernel(float* sink, int iters)
{
    typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
    if constexpr (KIND == 2)
    {
        // the 32x32x16 shape: 8 independent accumulators of 16 registers, the same flops per round
        typedef float f32x16 __attribute__((ext_vector_type(16)));
        f32x16 acc32[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc32[i][r] = 0.f;
        u32x4 a4[4], b4[4];
        uint32_t h = 0x9E3779B9u * (blockIdx.x * 256 + threadIdx.x + 1);
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                h = h * 1664525u + 1013904223u;
                a4[v][r] = ((RANDOM ? h : 0u) & 0x81FF81FFu) | 0x3C003C00u;
                h = h * 1664525u + 1013904223u;
                b4[v][r] = ((RANDOM ? h : 0u) & 0x81FF81FFu) | 0x3C003C00u;
            }
        for (int it = 0; it < iters; ++it)
        {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc32[i]) : "v"(a4[i & 3]), "v"(b4[i & 3]));
        }
        mma_drain();
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            s += acc32[i][0];
        sink[(blockIdx.x * 256 + threadIdx.x) & 511] = s;
        return;
    }
    f32x4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x8 a[4], b[4];
    uint32_t h = 0x9E3779B9u * (blockIdx.x * 256 + threadIdx.x + 1);
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int r = 0; r < 8; ++r)
        {
            h = h * 1664525u + 1013904223u;
            uint32_t const bits = RANDOM ? h : 0u;
            // finite small values in either format: bf16 pairs with exponent 0x3C..0x3F, e4m3 bytes below 0x78
            a[v][r] = KIND == 0 ? ((bits & 0x81FF81FFu) | 0x3C003C00u) : (bits & 0xB7B7B7B7u);
            h = h * 1664525u + 1013904223u;
            uint32_t const bits2 = RANDOM ? h : 0u;
            b[v][r] = KIND == 0 ? ((bits2 & 0x81FF81FFu) | 0x3C003C00u) : (bits2 & 0xB7B7B7B7u);
        }
    // shader-clock and constant-rate (100 MHz) counters around the loop: their ratio is the clock the
    // power management ran this wavefront at
    uint64_t const clk0 = __builtin_readcyclecounter(), ref0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it)
    {
#pragma unroll
        for (int i = 0; i < 16; ++i)
        {
            if constexpr (KIND == 0)
            {
                u32x4 const a4 = {a[i & 3][0], a[i & 3][1], a[i & 3][2], a[i & 3][3]};
                u32x4 const b4 = {b[i & 3][0], b[i & 3][1], b[i & 3][2], b[i & 3][3]};
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a4), "v"(b4));
            }
            else
                asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a[i & 3]), "v"(b[i & 3]));
        }
    }
    mma_drain();
    uint64_t const clk1 = __builtin_readcyclecounter(), ref1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        s += acc[i][0];
    sink[(blockIdx.x * 256 + threadIdx.x) & 511] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0)
    {
        reinterpret_cast<uint32_t*>(sink)[1020] = (uint32_t) (clk1 - clk0);
        reinterpret_cast<uint32_t*>(sink)[1021] = (uint32_t) (ref1 - ref0);
    }
}
} // namespace
} // namespace woq

using namespace woq;

extern "C" int woq_probe_read(const void* src, size_t bytes, int kib_per_wave, int loads_in_flight, int nontemporal, void* sink,
    void* stream)
{
    if (!src || !sink || kib_per_wave <= 0 || bytes < (size_t) kib_per_wave * 1024)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_read: src, sink and a buffer of at least one wavefront's share");
    if (loads_in_flight != 1 && loads_in_flight != 2 && loads_in_flight != 4 && loads_in_flight != 8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_read: loads_in_flight must be 1, 2, 4 or 8");
    if (kib_per_wave % loads_in_flight)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_read: kib_per_wave must be a multiple of loads_in_flight");
    size_t const waves = bytes / ((size_t) kib_per_wave * 1024);
    dim3 const grid((unsigned) ((waves + 3) / 4)), block(256);
    auto s = static_cast<hipStream_t>(stream);
    auto const* p = static_cast<u32x4 const*>(src);
    auto* k = static_cast<unsigned*>(sink);
#define WOQ_PROBE(U_)                                                                                                  \
    case U_:                                                                                                           \
        if (nontemporal)                                                                                               \
            hipLaunchKernelGGL((probe_read_kernel<U_, true>), grid, block, 0, s, p, (size_t) kib_per_wave, waves, k);   \
        else                                                                                                           \
            hipLaunchKernelGGL((probe_read_kernel<U_, false>), grid, block, 0, s, p, (size_t) kib_per_wave, waves, k);  \
        break;
    switch (loads_in_flight)
    {
        WOQ_PROBE(1)
        WOQ_PROBE(2)
        WOQ_PROBE(4)
        WOQ_PROBE(8)
    default: return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_read: loads_in_flight must be 1, 2, 4 or 8");
    }
#undef WOQ_PROBE
    hipError_t const err = hipGetLastError();
    return err == hipSuccess ? WOQ_OK : fail(WOQ_ERR_RUNTIME, "probe launch failed: %s", hipGetErrorString(err));
}

extern "C" int woq_probe_empty(void* sink, void* stream)
{
    if (!sink)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_empty: sink is NULL");
    hipLaunchKernelGGL(probe_empty_kernel, dim3(256), dim3(64), 0, static_cast<hipStream_t>(stream),
        static_cast<unsigned*>(sink));
    hipError_t const err = hipGetLastError();
    return err == hipSuccess ? WOQ_OK : fail(WOQ_ERR_RUNTIME, "probe launch failed: %s", hipGetErrorString(err));
}

extern "C" double woq_probe_mfma(int kind, int random_operands, int iters, int workgroups, void* sink, void* stream)
{
    if (!sink || iters <= 0 || workgroups <= 0 || kind < 0 || kind > 2)
    {
        fail(WOQ_ERR_INVALID_ARGUMENT, "woq_probe_mfma: kind 0 (bf16 16x16x32), 1 (fp8 16x16x128) or 2 (bf16 32x32x16), iters, workgroups > 0");
        return -1.0;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto* out = static_cast<float*>(sink);
    dim3 const grid(workgroups), block(256);
    if (kind == 0 && !random_operands)
        hipLaunchKernelGGL((probe_mfma_kernel<0, false>), grid, block, 0, s, out, iters);
    else if (kind == 0)
        hipLaunchKernelGGL((probe_mfma_kernel<0, true>), grid, block, 0, s, out, iters);
    else if (kind == 1 && !random_operands)
        hipLaunchKernelGGL((probe_mfma_kernel<1, false>), grid, block, 0, s, out, iters);
    else if (kind == 1)
        hipLaunchKernelGGL((probe_mfma_kernel<1, true>), grid, block, 0, s, out, iters);
    else if (!random_operands)
        hipLaunchKernelGGL((probe_mfma_kernel<2, false>), grid, block, 0, s, out, iters);
    else
        hipLaunchKernelGGL((probe_mfma_kernel<2, true>), grid, block, 0, s, out, iters);
    if (hipGetLastError() != hipSuccess)
    {
        fail(WOQ_ERR_RUNTIME, "probe launch failed");
        return -1.0;
    }
    // per round and wavefront: 16 instructions of the 16x16 shapes, 8 of the 32x32 one
    double const per_round = kind == 1 ? 16 * 2.0 * 16 * 16 * 128 : 16 * 2.0 * 16 * 16 * 32;
    return per_round * iters * 4.0 * workgroups; // floating-point operations of the launch
}
