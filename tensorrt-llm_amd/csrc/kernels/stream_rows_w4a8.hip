// W4A8 decode of up to sixteen rows (e4m3 activations, int4 weights, fp16 group scales) without a staging pass:
// the multi-row kernel of stream_rows_kernel.h on the fp8 matrix core.
//
// Same semantics as the other W4A8 kernels (stream_w4a8.hip, gemm_w4a8.hip; the reference's fpA_intB runner
// for __nv_fp8_e4m3 x uint4, weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): every weight is dequantized
// with its fp16 group scale (and zero), rounded to e4m3, multiplied as fp8 x fp8 with float32 sums;
// out = T(alpha * sum + bias).  Division of work as in stream_rows_kernel.h: plain scalar arguments preloaded
// into SGPRs, a workgroup owns NS neighbouring strips of 16 columns, its wavefronts split K and request
// everything of their TPW tile rows at once (activations - row c of the A operand is row c of the problem, rows
// past m read zeros - NS x TPW weight tiles, and the scales / zeros, fetched by the lanes kg for tile row kg and
// handed on by lane permute), no staging, no barrier before the arithmetic.
//   * one v_mfma_f32_16x16x128_f8f6f4 covers a tile (128 rows of K) and accumulates straight into the strip's
//     sums: the scale is inside the converted weights;
//   * the weights of a tile are converted through the sixteen-entry table of their (group, column)
//     (w4a8_common.h: the same FMA and saturating conversion as the arithmetic form, so the bytes are
//     identical); a tile row's activations are reordered once to the order the look-up delivers and used for
//     all NS strips.
#include "stream_kernel.h"
#include "w4a8_common.h"

namespace woq
{

struct RowsW4a8Tail
{
    void const* bias;
    float alpha;
    int m;
    uint32_t group_magic; // see w4a8_scale_row
};

// (the first fourteen dwords of the arguments are preloaded into SGPRs: what the requests need, except the
// divisor of the scale row, which only the scale requests wait for)
template <int ODT, bool ZERO, int WAVES, int NS, int TPW>
__global__ void __launch_bounds__(WAVES * 64) stream_rows_w4a8_kernel(void const* weight, void const* act, void const* scales,
    void const* zeros, int k_tiles, int strips, int groups_per_xcd, int n, int scale_rows, int act_bytes, void* out,
    RowsW4a8Tail tail)
{
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    static_assert(TPW >= 1 && TPW <= 4, "tile row kg of a pass has its scales fetched by the lanes kg");
    constexpr uint32_t kOob = 0x80000000u;

    int const groups = (strips + NS - 1) / NS;
    int const group = xcd_strip(blockIdx.x, groups_per_xcd);
    if (group >= groups)
        return; // whole workgroup leaves together
    int const strip0 = group * NS;

    // The conversions rely on the saturating mode; it is switched on before the first request is issued:
    // every converted value depends on a load, and loads are not moved across the switch, whereas arithmetic
    // on values loaded before it could be.  Off again before the epilogue.
    fp8_saturation_on();
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const KT = k_tiles;
    int const K = KT * 128;
    auto const w_rsrc = make_rsrc(weight, (uint32_t) strips * (uint32_t) KT * 1024u);
    auto const act_rsrc = make_rsrc(act, (uint32_t) act_bytes);
    uint32_t const sz_bytes = (uint32_t) scale_rows * (uint32_t) n * 2u;
    auto const sc_rsrc = make_rsrc(scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? zeros : scales, sz_bytes);
    // lane (kg, c): A operand row c, bytes kg * 8 .. of every slab; B operand column c
    uint32_t const a_lane = (uint32_t) c * (uint32_t) K + (uint32_t) (kg * 8);
    uint32_t wlane[NS], sc_lane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        bool const ok = strip0 + s < strips;
        wlane[s] = ok ? ((uint32_t) (strip0 + s) * (uint32_t) KT * 64u + (uint32_t) lane) * 16u : kOob;
        sc_lane[s] = ok ? (uint32_t) ((strip0 + s) * 16 + c) * 2u : kOob;
    }

    float qf[4];
    fp8_table_lane_values(kg, qf);
    Fp8LookupConsts const lk = fp8_lookup_consts();
    f32x4 total[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        total[s] = f32x4{0.f, 0.f, 0.f, 0.f};

    int const passes = (KT + WAVES * TPW - 1) / (WAVES * TPW);
    for (int pass = 0; pass < passes; ++pass)
    {
        int const kt0 = (pass * WAVES + wave) * TPW;
        // ---- every request of the pass ----
        u32x2 a[TPW][4];
        u32x4 w[TPW][NS];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a[i][j] = buffer_load_x2(act_rsrc, kt0 + i < KT ? a_lane + (uint32_t) ((kt0 + i) * 128 + j * 32) : kOob);
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int s = 0; s < NS; ++s)
                w[i][s] = buffer_load_x4_once(w_rsrc, kt0 + i < KT ? wlane[s] + (uint32_t) (kt0 + i) * 1024u : (uint32_t) kOob);
        // scale (low half) and zero (high half) of tile row kt0 + kg, strip s, column c
        uint32_t sz[NS];
        uint32_t const magic = tail.group_magic;
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            uint32_t const off = kg < TPW && kt0 + kg < KT
                ? w4a8_scale_row((uint32_t) (kt0 + kg), magic) * (uint32_t) n * 2u + sc_lane[s]
                : (uint32_t) kOob;
            uint32_t const sv = buffer_load_u16(sc_rsrc, off);
            uint32_t const zv = ZERO ? (uint32_t) buffer_load_u16(zr_rsrc, off) : 0u;
            sz[s] = sv | (zv << 16);
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- tile row by tile row: activations in look-up order, then one table and one product per strip ----
#pragma unroll
        for (int i = 0; i < TPW; ++i)
        {
            i32x8 av;
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                uint32_t a0, a1;
                fp8_a_order(a[i][j][0], a[i][j][1], a0, a1);
                av[2 * j] = (int) a0;
                av[2 * j + 1] = (int) a1;
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                // the lanes (i, c) hold this tile row's scale and zero for column c
                uint32_t const got = (uint32_t) __shfl((int) sz[s], i * 16 + c);
                float const sc = EH::from_bits((uint16_t) (got & 0xFFFFu));
                float const zr = ZERO ? EH::from_bits((uint16_t) (got >> 16)) : 0.f;
                Fp8Table const table = build_fp8_table(sc, zr, qf);
                i32x8 b;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    uint32_t b0, b1;
                    fp8_lookup8(w[i][s][j], table, lk, b0, b1);
                    b[2 * j] = (int) b0;
                    b[2 * j + 1] = (int) b1;
                }
                total[s] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, b, total[s], 0, 0, 0, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int s = 0; s < NS; ++s)
        before_mode_change(total[s]);
    fp8_saturation_off();

    // ---- the wavefronts' sums, in wavefront order ----
    __shared__ float red[WAVES][NS][16][16];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            red[wave][s][kg * 4 + r][c] = after_mode_change(total[s][r]);
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
            float const bias = tail.bias ? EO::load(tail.bias, ocol) : 0.f;
            static_cast<uint16_t*>(out)[(size_t) row * n + ocol] = EO::store(__builtin_fmaf(tail.alpha, sum, bias));
        }
    }
}

namespace
{
template <int ODT, bool ZERO, int WAVES, int NS, int TPW>
int launch_rows_w4a8_variant(StreamParams const& sp, hipStream_t stream)
{
    int const groups_per_xcd = ((sp.strips + NS - 1) / NS + 7) / 8;
    dim3 grid(groups_per_xcd * 8), block(WAVES * 64);
    note_launch("stream multirow w4a8 waves=%d ns=%d tpw=%d passes=%d", WAVES, NS, TPW,
        (sp.k_tiles + WAVES * TPW - 1) / (WAVES * TPW));
    RowsW4a8Tail const tail{sp.bias, sp.alpha, sp.m, sp.group_magic};
    int const act_bytes = sp.m * sp.k;
    hipLaunchKernelGGL((stream_rows_w4a8_kernel<ODT, ZERO, WAVES, NS, TPW>), grid, block, 0, stream, sp.weight, sp.act,
        sp.scales, sp.zeros, sp.k_tiles, sp.strips, groups_per_xcd, sp.n, sp.scale_rows, act_bytes, sp.out, tail);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "W4A8 rows stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int ODT, bool ZERO>
int launch_rows_w4a8_shaped(StreamParams const& sp, int waves, int ns, int tpw, hipStream_t s)
{
#define WOQ_ROWS(WAVES_, NS_, TPW_)                                                                                    \
    if (waves == WAVES_ && ns == NS_ && tpw == TPW_)                                                                   \
        return launch_rows_w4a8_variant<ODT, ZERO, WAVES_, NS_, TPW_>(sp, s);
    WOQ_ROWS(8, 1, 2)
    WOQ_ROWS(8, 2, 2)
    WOQ_ROWS(8, 4, 2)
    WOQ_ROWS(16, 2, 2)
    WOQ_ROWS(4, 1, 4)
#undef WOQ_ROWS
    return fail(WOQ_ERR_UNSUPPORTED, "W4A8 rows stream shape waves=%d ns=%d tpw=%d is not instantiated", waves, ns, tpw);
}
} // namespace

// sp: act (e4m3), weight, scales, zeros (fp16), bias, out, alpha, m, n, k, k_tiles, strips, scale_rows, group_magic
int launch_stream_rows_w4a8(StreamParams const& sp, int out_dtype, int waves, int ns, int tpw, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    if (sp.m < 1 || sp.m > 16 || sp.k % 128)
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 rows stream kernel: up to sixteen rows, k %% 128 == 0");
    if ((uint64_t) sp.m * (uint64_t) sp.n * 2 >= ((uint64_t) 1 << 31) || (uint64_t) sp.m * (uint64_t) sp.k >= ((uint64_t) 1 << 31))
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 rows stream kernel: operand beyond 2 GiB");
    bool const zero = sp.zeros != nullptr;
    if (out_dtype == WOQ_BF16)
        return zero ? launch_rows_w4a8_shaped<WOQ_BF16, true>(sp, waves, ns, tpw, s)
                    : launch_rows_w4a8_shaped<WOQ_BF16, false>(sp, waves, ns, tpw, s);
    return zero ? launch_rows_w4a8_shaped<WOQ_FP16, true>(sp, waves, ns, tpw, s)
                : launch_rows_w4a8_shaped<WOQ_FP16, false>(sp, waves, ns, tpw, s);
}

} // namespace woq
