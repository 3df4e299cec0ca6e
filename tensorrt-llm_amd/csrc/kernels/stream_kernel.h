// Weight-streaming kernel for small M (decode GEMV up to skinny GEMM, M <= 128).
//
// Counterpart of the reference's small-M kernel
// (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernel.h:29-146) in purpose only.  The design
// is for CDNA4:
//   * every lane streams its slice of the packed weights with one 128-bit load per 1 KiB tile
//     (a wavefront reads the tile contiguously), several tiles in flight per wavefront;
//   * int4/int8 values are widened in registers to 16-bit floats holding (BASE + u) exactly and
//     fed to the 16x16x32 matrix core as the B operand; the activations (up to 16 rows per
//     M-tile, rows >= M are zero) are the A operand, so M = 1..16 cost the same;
//   * scales are applied to the per-group partial products in float32, together with the
//     row sums of the activations (a second MFMA against an all-ones operand) that remove the
//     BASE + 2^(bits-1) offset and carry the additive zeros:
//         out += s * P + (z - OFFSET * s) * S,   P = sum a * (q + OFFSET),   S = sum a;
//   * the wavefronts of a workgroup split K and are reduced through LDS in a fixed order
//     (results are bit-reproducible from run to run).
#pragma once

#include "device_common.h"

namespace woq
{

struct StreamParams
{
    void const* act;
    void const* pqs;
    void const* weight;
    void const* scales;
    void const* zeros;
    void const* bias;
    void* out;
    float alpha;
    int m, n, k;
    int k_tiles;        // ceil(k / TILE_K)
    int strips;         // n / 16
    int strips_per_xcd; // ceil(strips / 8)
};

template <int DT, int BITS, int GROUP, bool PQS, int MT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) stream_kernel(StreamParams p)
{
    using E = Elem<DT>;
    constexpr int TK = BITS == 4 ? 128 : 64;
    constexpr int SEG = (GROUP == 0 || GROUP > TK) ? TK : GROUP; // rows that share one scale inside a tile
    constexpr int SEG_SLABS = SEG / 32;
    constexpr int SEGS = TK / SEG;
    constexpr int PF = 4; // weight tiles in flight per wavefront
    constexpr float OFF = Offset<DT, BITS>::value;

    int const strip = xcd_strip(blockIdx.x, p.strips_per_xcd);
    if (strip >= p.strips)
        return; // whole workgroup leaves together

    int const lane = threadIdx.x & 63;
    int const wave = threadIdx.x >> 6;
    int const c = lane & 15;  // column inside the strip (B operand) / row inside the M-tile (A operand)
    int const kg = lane >> 4; // which 8 of a slab's 32 rows this lane holds
    int const col = strip * 16 + c;
    int const K = p.k;
    int const KT = p.k_tiles;

    u32x4 const ones = {E::kOnes, E::kOnes, E::kOnes, E::kOnes};
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};

    f32x4 acc_out[MT], acc_p[MT], acc_s[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        acc_out[mt] = acc_p[mt] = acc_s[mt] = zero4;

    u32x4 const* wbase = static_cast<u32x4 const*>(p.weight) + (size_t) strip * KT * 64 + lane;
    uint16_t const* act16 = static_cast<uint16_t const*>(p.act);

    u32x4 buf[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i)
    {
        int kt = wave + i * WAVES;
        buf[i] = kt < KT ? wbase[(size_t) kt * 64] : u32x4{0, 0, 0, 0};
    }

    for (int kt0 = wave; kt0 < KT; kt0 += WAVES * PF)
    {
#pragma unroll
        for (int i = 0; i < PF; ++i)
        {
            int const kt = kt0 + i * WAVES;
            if (kt >= KT)
                break; // wave-uniform
            u32x4 const w = buf[i];
            int const ktn = kt + PF * WAVES;
            if (ktn < KT)
                buf[i] = wbase[(size_t) ktn * 64];

#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                int const krow0 = kt * TK + seg * SEG; // first row of this segment
                if (krow0 >= K)
                    break; // padded tail of K: wave-uniform
#pragma unroll
                for (int js = 0; js < SEG_SLABS; ++js)
                {
                    int const j = seg * SEG_SLABS + js;
                    u32x4 b;
                    if constexpr (BITS == 4)
                        b = expand_int4<DT>(w[j]);
                    else
                        b = expand_int8<DT>(w[2 * j], w[2 * j + 1]);
                    int const kk = kt * TK + j * 32 + kg * 8; // this lane's 8 rows of the slab
                    bool const k_ok = kk < K;
                    u32x4 sm = {0, 0, 0, 0};
                    if constexpr (PQS)
                        if (k_ok)
                            sm = *reinterpret_cast<u32x4 const*>(static_cast<uint16_t const*>(p.pqs) + kk);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                    {
                        int const row = mt * 16 + c;
                        u32x4 a = {0, 0, 0, 0};
                        if (k_ok && row < p.m)
                            a = *reinterpret_cast<u32x4 const*>(act16 + (size_t) row * K + kk);
                        if constexpr (PQS)
                        {
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                a[r] = E::mul2(a[r], sm[r]);
                        }
                        acc_p[mt] = E::mma(a, b, acc_p[mt]);
                        acc_s[mt] = E::mma(a, ones, acc_s[mt]);
                    }
                }
                if constexpr (GROUP != 0)
                {
                    size_t const gi = (size_t) (krow0 / GROUP) * p.n + col;
                    float const s = E::load(p.scales, gi);
                    float const z = p.zeros ? E::load(p.zeros, gi) : 0.f;
                    float const cc = z - OFF * s;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                    {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            acc_out[mt][r] += s * acc_p[mt][r] + cc * acc_s[mt][r];
                        acc_p[mt] = zero4;
                        acc_s[mt] = zero4;
                    }
                }
            }
        }
    }

    if constexpr (GROUP == 0)
    {
        float const s = E::load(p.scales, col);
        float const z = p.zeros ? E::load(p.zeros, col) : 0.f;
        float const cc = z - OFF * s;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                acc_out[mt][r] = s * acc_p[mt][r] + cc * acc_s[mt][r];
    }

    // ---- cross-wavefront reduction (fixed order) and epilogue -------------------------------
    __shared__ float red[WAVES][MT * 4][64];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            red[wave][mt * 4 + r][lane] = acc_out[mt][r];
    __syncthreads();

    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    for (int e = threadIdx.x; e < MT * 4 * 64; e += WAVES * 64)
    {
        int const slot = e >> 6, ln = e & 63;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][slot][ln];
        int const row = (slot >> 2) * 16 + (ln >> 4) * 4 + (slot & 3);
        int const ocol = strip * 16 + (ln & 15);
        if (row < p.m)
        {
            float v = p.alpha * sum;
            if (p.bias)
                v += E::load(p.bias, ocol);
            out16[(size_t) row * p.n + ocol] = E::store(v);
        }
    }
}

template <int DT, int BITS, int GROUP, bool PQS, int MT>
int launch_stream_variant(StreamParams const& sp, hipStream_t stream)
{
    constexpr int WAVES = MT >= 8 ? 4 : 8;
    dim3 grid(sp.strips_per_xcd * 8), block(WAVES * 64);
    hipLaunchKernelGGL((stream_kernel<DT, BITS, GROUP, PQS, MT, WAVES>), grid, block, 0, stream, sp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int DT, int BITS>
int launch_stream_typed(MatmulProblem const& p, void* stream)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    StreamParams sp;
    sp.act = p.act;
    sp.pqs = p.pre_quant_scale;
    sp.weight = p.weight;
    sp.scales = p.scales;
    sp.zeros = p.zeros;
    sp.bias = p.bias;
    sp.out = p.out;
    sp.alpha = p.alpha;
    sp.m = p.m;
    sp.n = p.n;
    sp.k = p.k;
    sp.k_tiles = (p.k + TK - 1) / TK;
    sp.strips = p.n / kTileN;
    sp.strips_per_xcd = (sp.strips + 7) / 8;
    auto s = static_cast<hipStream_t>(stream);
    int const mt = p.m <= 16 ? 1 : (p.m <= 32 ? 2 : (p.m <= 64 ? 4 : 8));
    bool const pqs = p.pre_quant_scale != nullptr;

#define WOQ_STREAM_MT(G, Q)                                                                                            \
    switch (mt)                                                                                                        \
    {                                                                                                                  \
    case 1: return launch_stream_variant<DT, BITS, G, Q, 1>(sp, s);                                                    \
    case 2: return launch_stream_variant<DT, BITS, G, Q, 2>(sp, s);                                                    \
    case 4: return launch_stream_variant<DT, BITS, G, Q, 4>(sp, s);                                                    \
    default: return launch_stream_variant<DT, BITS, G, Q, 8>(sp, s);                                                   \
    }
#define WOQ_STREAM_PQS(G)                                                                                              \
    if (pqs)                                                                                                           \
    {                                                                                                                  \
        WOQ_STREAM_MT(G, true)                                                                                         \
    }                                                                                                                  \
    else                                                                                                               \
    {                                                                                                                  \
        WOQ_STREAM_MT(G, false)                                                                                        \
    }
    switch (p.group_size)
    {
    case 0: WOQ_STREAM_PQS(0)
    case 64: WOQ_STREAM_PQS(64)
    case 128: WOQ_STREAM_PQS(128)
    default: return fail(WOQ_ERR_UNSUPPORTED, "group_size %d", p.group_size);
    }
#undef WOQ_STREAM_PQS
#undef WOQ_STREAM_MT
}

} // namespace woq
