// Decode of up to sixteen rows without a staging pass (int4 or int8 weights; group scales of 64 or 128 rows, or
// per-channel scales).
//
// Counterpart of the reference's small-M kernel at batch 2 ... 16
// (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernel.h:57-146) in purpose only.  The row kernel
// (stream_row.hip) showed what a decode launch is made of on this part: a stream at the rate of a plain read
// with fixed pieces around it, the largest of which - scalar loads of the arguments, a staging pass, a
// barrier - a kernel can avoid.  This is the same skeleton for more rows than fit its (group, row) packing:
//   * plain scalar arguments, the ones the requests need among the first fourteen dwords (preloaded into
//     SGPRs when the wavefront starts);
//   * a workgroup owns NS neighbouring strips of 16 columns, its wavefronts split K: wavefront w takes the TPW
//     consecutive tile rows (pass * WAVES + w) * TPW .. of it and requests everything those need at once -
//     the activation fragments (row c of the 16x16x32 instruction's A operand is row c of the problem; rows
//     past m lie outside the descriptor, read zeros and cost no traffic), NS x TPW weight tiles, and the
//     scales and zeros: lane (kg, c) fetches those of tile row kg for its column c, one two-byte load per strip
//     and table for the whole pass, and hands them to the lanes that need them with a lane permute; a
//     smoothing vector, if any, comes as the same 8 k-values per lane for every row and is multiplied in;
//   * an activation fragment is read once per wavefront and used for all NS strips, which is what bounds the
//     traffic from the L2 (per workgroup m rows of activations against NS x 8 bytes per k of weights);
//   * P = A x (q + OFFSET) per group and strip, S = A x ones per group, out += s * P + (z - OFFSET * s) * S in
//     float32, as in the other streaming kernels; the wavefronts are added through LDS in wavefront order:
//     results are bit-reproducible.  With per-channel scales P and S run over all of K and the scale is applied
//     once, after the wavefronts are added.
// Instantiated per weight width in stream_rows_int4.hip / stream_rows_int8.hip.
#pragma once

#include "stream_kernel.h"

namespace woq
{

struct RowsTail
{
    void const* pqs; // smoothing vector [k] in the activation type, or NULL (PQS variants only)
    void const* bias;
    float alpha;
    int m;
};

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int WAVES, int NS, int TPW>
__global__ void __launch_bounds__(WAVES * 64) stream_rows_kernel(void const* weight, void const* act, void const* scales,
    void const* zeros, int k_tiles, int strips, int groups_per_xcd, int n, int k, int act_bytes, void* out, RowsTail tail)
{
    using E = Elem<DT>;
    constexpr int TK = BITS == 4 ? 128 : 64; // rows of K in a 1 KiB tile
    constexpr int SLABS = TK / 32;
    constexpr bool PER_CHANNEL = GROUP == 0;
    constexpr int SEGS = (!PER_CHANNEL && GROUP < TK) ? TK / GROUP : 1; // scale groups inside a tile row
    constexpr int SEG_SLABS = SLABS / SEGS;
    static_assert(GROUP == 0 || GROUP == 64 || GROUP == 128, "per-channel scales or group scales of 64 or 128 rows");
    static_assert(!(PER_CHANNEL && ZERO), "per-channel scales come without zeros");
    static_assert(TPW >= 1 && TPW <= 4, "tile row kg of a pass has its scales fetched by the lanes kg");
    constexpr float OFF = Offset<DT, BITS>::value;
    constexpr uint32_t kOob = 0x80000000u;

    int const groups = (strips + NS - 1) / NS;
    int const group = xcd_strip(blockIdx.x, groups_per_xcd);
    if (group >= groups)
        return; // whole workgroup leaves together
    int const strip0 = group * NS;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const KT = k_tiles;
    auto const w_rsrc = make_rsrc(weight, (uint32_t) strips * (uint32_t) KT * 1024u);
    auto const act_rsrc = make_rsrc(act, (uint32_t) act_bytes);
    int const groups_k = PER_CHANNEL ? 1 : k / (PER_CHANNEL ? 1 : GROUP);
    uint32_t const sz_bytes = (uint32_t) groups_k * (uint32_t) n * 2u;
    auto const sc_rsrc = make_rsrc(scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? zeros : scales, sz_bytes);
    // (with a smoothing vector the first request waits for one more scalar load: its pointer lies past the
    // preloaded arguments)
    auto const pq_rsrc = make_rsrc(PQS ? tail.pqs : act, (uint32_t) k * 2u);
    // lane (kg, c): A operand row c, k offset kg * 8 inside a slab; B operand column c
    uint32_t const a_lane = ((uint32_t) c * (uint32_t) k + (uint32_t) (kg * 8)) * 2u;
    uint32_t wlane[NS], sc_lane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        bool const ok = strip0 + s < strips;
        wlane[s] = ok ? ((uint32_t) (strip0 + s) * (uint32_t) KT * 64u + (uint32_t) lane) * 16u : kOob;
        sc_lane[s] = ok ? (uint32_t) ((strip0 + s) * 16 + c) * 2u : kOob;
    }

    u32x4 const ones = {E::kOnes, E::kOnes, E::kOnes, E::kOnes};
    NibbleConsts const nib = nibble_consts<DT>();
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 total[NS];     // finished sums (group scales) / running P (per-channel)
    f32x4 s_all = zero4; // running S of the per-channel mode
#pragma unroll
    for (int s = 0; s < NS; ++s)
        total[s] = zero4;
    // one slab's B operand from a lane's 16 packed bytes
    auto expand = [&](u32x4 const& wv, int j) -> u32x4
    {
        if constexpr (BITS == 4)
            return expand_int4<DT>(wv[j], nib);
        else
            return expand_int8<DT>(wv[2 * j], wv[2 * j + 1]);
    };

    int const passes = (KT + WAVES * TPW - 1) / (WAVES * TPW);
    for (int pass = 0; pass < passes; ++pass)
    {
        int const kt0 = (pass * WAVES + wave) * TPW;
        // ---- every request of the pass ----
        u32x4 a[TPW][SLABS], w[TPW][NS], pq[PQS ? TPW : 1][SLABS];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int j = 0; j < SLABS; ++j)
            {
                bool const in_k = (kt0 + i) * TK + j * 32 < k;
                a[i][j] = buffer_load_x4(act_rsrc, in_k ? a_lane + (uint32_t) ((kt0 + i) * TK + j * 32) * 2u : kOob);
                if constexpr (PQS) // the same 8 k-values for every row
                    pq[i][j] = buffer_load_x4(pq_rsrc, in_k ? (uint32_t) ((kt0 + i) * TK + j * 32 + kg * 8) * 2u : kOob);
            }
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int s = 0; s < NS; ++s)
                w[i][s] = buffer_load_x4_once(w_rsrc, kt0 + i < KT ? wlane[s] + (uint32_t) (kt0 + i) * 1024u : (uint32_t) kOob);
        // scale (low half) and zero (high half) of tile row kt0 + kg, segment seg, strip s, column c
        uint32_t sz[NS][SEGS];
        if constexpr (!PER_CHANNEL)
        {
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int seg = 0; seg < SEGS; ++seg)
                {
                    int const g = ((kt0 + kg) * TK + seg * (TK / SEGS)) / (PER_CHANNEL ? 1 : GROUP);
                    uint32_t const off
                        = kg < TPW && g < groups_k ? (uint32_t) g * (uint32_t) n * 2u + sc_lane[s] : (uint32_t) kOob;
                    uint32_t const sv = buffer_load_u16(sc_rsrc, off);
                    uint32_t const zv = ZERO ? (uint32_t) buffer_load_u16(zr_rsrc, off) : 0u;
                    sz[s][seg] = sv | (zv << 16);
                }
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- products and scale application, tile row by tile row ----
#pragma unroll
        for (int i = 0; i < TPW; ++i)
        {
            if constexpr (PQS) // T(a * s), one rounding, as the separate smoothing pass does
            {
#pragma unroll
                for (int j = 0; j < SLABS; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        a[i][j][r] = E::mul2(a[i][j][r], pq[i][j][r]);
            }
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                if constexpr (PER_CHANNEL)
                {
#pragma unroll
                    for (int js = 0; js < SLABS; ++js)
                    {
                        s_all = E::mma(a[i][js], ones, s_all);
#pragma unroll
                        for (int s = 0; s < NS; ++s)
                            total[s] = E::mma(a[i][js], expand(w[i][s], js), total[s]);
                    }
                    continue;
                }
                f32x4 S = zero4;
#pragma unroll
                for (int js = 0; js < SEG_SLABS; ++js)
                    S = E::mma(a[i][seg * SEG_SLABS + js], ones, S);
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    f32x4 P = zero4;
#pragma unroll
                    for (int js = 0; js < SEG_SLABS; ++js)
                        P = E::mma(a[i][seg * SEG_SLABS + js], expand(w[i][s], seg * SEG_SLABS + js), P);
                    // the lanes (i, c) hold this tile row's scale and zero for column c
                    uint32_t const got = (uint32_t) __shfl((int) sz[s][seg], i * 16 + c);
                    float const sc = E::from_bits((uint16_t) (got & 0xFFFFu));
                    float const cc = __builtin_fmaf(-OFF, sc, ZERO ? E::from_bits((uint16_t) (got >> 16)) : 0.f);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        total[s][r] = __builtin_fmaf(sc, P[r], __builtin_fmaf(cc, S[r], total[s][r]));
                }
            }
        }
    }

    // ---- the wavefronts' sums, in wavefront order ----
    __shared__ float red[WAVES][NS][16][16];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int r = 0; r < 4; ++r) // per-channel: sum a * q = P - OFFSET * S; the column's scale follows below
            red[wave][s][kg * 4 + r][c] = PER_CHANNEL ? __builtin_fmaf(-OFF, s_all[r], total[s][r]) : total[s][r];
    __syncthreads();
    for (int e = threadIdx.x; e < NS * 256; e += WAVES * 64)
    {
        int const s = e >> 8, row = (e >> 4) & 15, col = e & 15;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][s][row][col];
        if (row < tail.m && strip0 + s < strips)
        {
            int const ocol = (strip0 + s) * 16 + col;
            if constexpr (PER_CHANNEL)
                sum *= E::load(scales, ocol);
            float v = tail.alpha * sum;
            if (tail.bias)
                v += E::load(tail.bias, ocol);
            static_cast<uint16_t*>(out)[(size_t) row * n + ocol] = E::store(v);
        }
    }
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int WAVES, int NS, int TPW>
int launch_rows_variant(StreamParams sp, hipStream_t stream)
{
    sp.groups = (sp.strips + NS - 1) / NS;
    sp.groups_per_xcd = (sp.groups + 7) / 8;
    dim3 grid(sp.groups_per_xcd * 8), block(WAVES * 64);
    note_launch("stream multirow waves=%d ns=%d tpw=%d passes=%d", WAVES, NS, TPW, (sp.k_tiles + WAVES * TPW - 1) / (WAVES * TPW));
    RowsTail tail{sp.pqs, sp.bias, sp.alpha, sp.m};
    int const act_bytes = sp.m * sp.k * 2;
    hipLaunchKernelGGL((stream_rows_kernel<DT, BITS, GROUP, PQS, ZERO, WAVES, NS, TPW>), grid, block, 0, stream, sp.weight,
        sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, sp.groups_per_xcd, sp.n, sp.k, act_bytes, sp.out, tail);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "rows stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO>
int launch_rows_shaped(StreamParams const& sp, int waves, int ns, int tpw, hipStream_t s)
{
#define WOQ_ROWS(WAVES_, NS_, TPW_)                                                                                    \
    if (waves == WAVES_ && ns == NS_ && tpw == TPW_)                                                                   \
        return launch_rows_variant<DT, BITS, GROUP, PQS, ZERO, WAVES_, NS_, TPW_>(sp, s);
    WOQ_ROWS(8, 1, 2)
    WOQ_ROWS(8, 2, 2)
    WOQ_ROWS(8, 4, 2)
    WOQ_ROWS(16, 2, 2)
    WOQ_ROWS(4, 1, 4)
#undef WOQ_ROWS
    return fail(WOQ_ERR_UNSUPPORTED, "rows stream shape waves=%d ns=%d tpw=%d is not instantiated", waves, ns, tpw);
}

template <int DT, int BITS, int GROUP>
int launch_rows_flags(StreamParams const& sp, bool zero, int waves, int ns, int tpw, hipStream_t s)
{
    if constexpr (GROUP == 0)
    {
        if (zero)
            return fail(WOQ_ERR_UNSUPPORTED, "rows stream kernel: per-channel scales come without zeros");
        return sp.pqs ? launch_rows_shaped<DT, BITS, 0, true, false>(sp, waves, ns, tpw, s)
                      : launch_rows_shaped<DT, BITS, 0, false, false>(sp, waves, ns, tpw, s);
    }
    else
    {
        if (sp.pqs)
            return zero ? launch_rows_shaped<DT, BITS, GROUP, true, true>(sp, waves, ns, tpw, s)
                        : launch_rows_shaped<DT, BITS, GROUP, true, false>(sp, waves, ns, tpw, s);
        return zero ? launch_rows_shaped<DT, BITS, GROUP, false, true>(sp, waves, ns, tpw, s)
                    : launch_rows_shaped<DT, BITS, GROUP, false, false>(sp, waves, ns, tpw, s);
    }
}

// the launcher of one weight width (its translation unit instantiates every kernel of that width)
template <int BITS>
int launch_stream_rows_bits(StreamParams const& sp, int dtype, int group, bool zero, int waves, int ns, int tpw, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    if (sp.m < 1 || sp.m > 16 || (group != 0 && group != 64 && group != 128) || (group && sp.k % group) || sp.num_experts
        || sp.activation != kActIdentity || sp.residual)
        return fail(WOQ_ERR_UNSUPPORTED,
            "rows stream kernel: up to sixteen rows, per-channel scales or group size 64 or 128, plain epilogue");
    if ((uint64_t) sp.m * (uint64_t) sp.n * 2 >= ((uint64_t) 1 << 31) || (uint64_t) sp.m * (uint64_t) sp.k * 2 >= ((uint64_t) 1 << 31))
        return fail(WOQ_ERR_UNSUPPORTED, "rows stream kernel: operand beyond 2 GiB");
    if (dtype == WOQ_BF16)
        return group == 0 ? launch_rows_flags<WOQ_BF16, BITS, 0>(sp, zero, waves, ns, tpw, s)
                          : (group == 64 ? launch_rows_flags<WOQ_BF16, BITS, 64>(sp, zero, waves, ns, tpw, s)
                                         : launch_rows_flags<WOQ_BF16, BITS, 128>(sp, zero, waves, ns, tpw, s));
    return group == 0 ? launch_rows_flags<WOQ_FP16, BITS, 0>(sp, zero, waves, ns, tpw, s)
                      : (group == 64 ? launch_rows_flags<WOQ_FP16, BITS, 64>(sp, zero, waves, ns, tpw, s)
                                     : launch_rows_flags<WOQ_FP16, BITS, 128>(sp, zero, waves, ns, tpw, s));
}

} // namespace woq
