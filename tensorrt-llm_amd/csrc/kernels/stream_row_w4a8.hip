// W4A8 decode of one to four rows (e4m3 activations, int4 weights, fp16 group scales): the row kernel of
// stream_row.hip on the fp8 matrix core.
//
// Same semantics as the other W4A8 kernels (stream_w4a8.hip, gemm_w4a8.hip; the reference's fpA_intB runner
// for __nv_fp8_e4m3 x uint4, weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): every weight is dequantized
// with its fp16 group scale (and zero), rounded to e4m3, multiplied as fp8 x fp8 with float32 sums;
// out = T(alpha * sum + bias).  Same division of work as stream_row.hip: one workgroup per strip of 16
// columns, wavefront w multiplies the TPW consecutive tiles w * TPW .. of each pass, all requests of a
// pass issued at once, no staging pass, kernel arguments preloaded into SGPRs.
//   * one v_mfma_f32_16x16x128_f8f6f4 covers a whole tile (128 rows of K).  Row c of its A operand carries
//     activation row c % R of the wavefront's (c / R)-th tile and nothing else; D_t = A x W_t is kept per
//     tile t and only its rows t * R .. t * R + R - 1 are used;
//   * the weights of a tile are converted through the sixteen-entry table of their (group, column)
//     (w4a8_common.h: the same FMA and saturating conversion as the arithmetic form, so the bytes are
//     identical); the lane's activations are reordered once per pass to the order the look-up delivers.
#include "stream_kernel.h"
#include "w4a8_common.h"

namespace woq
{

struct RowW4a8Tail
{
    void const* bias;
    float alpha;
    int m;
    uint32_t group_magic; // see w4a8_scale_row
};

// (the first fourteen dwords of the arguments are preloaded into SGPRs: what the requests need)
template <int ODT, bool ZERO, int WAVES, int TPW, bool MULTI, int R>
__global__ void __launch_bounds__(WAVES * 64) stream_row_w4a8_kernel(void const* weight, void const* act, void const* scales,
    void const* zeros, int k_tiles, int strips, int groups_per_xcd, int n, int scale_rows, int act_bytes, void* out,
    RowW4a8Tail tail)
{
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    constexpr int ROWS = TPW * R; // rows of the M-tile in use
    static_assert(R == 1 || R == 2 || R == 4, "one, two or four activation rows");
    static_assert(ROWS <= 16, "the M-tile has 16 rows");
    constexpr uint32_t kOob = 0x80000000u;

    int const strip = xcd_strip(blockIdx.x, groups_per_xcd);
    if (strip >= strips)
        return; // whole workgroup leaves together

    // The conversions rely on the saturating mode; it is switched on before the first request is issued:
    // every converted value depends on a load, and loads are not moved across the switch, whereas arithmetic
    // on values loaded before it could be.  Off again before the epilogue.
    fp8_saturation_on();
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const KT = k_tiles;
    int const K = KT * 128;
    auto const w_rsrc = make_rsrc(weight, (uint32_t) strips * (uint32_t) KT * 1024u);
    uint32_t const wlane = ((uint32_t) strip * (uint32_t) KT * 64u + (uint32_t) lane) * 16u;
    int const c = lane & 15, kg = lane >> 4;
    auto const act_rsrc = make_rsrc(act, (uint32_t) act_bytes);
    // this lane's activations: row c % R of the problem, tile c / R of the pass; 8 bytes of each slab
    uint32_t const a_lane = (uint32_t) (c % R) * (uint32_t) K + (uint32_t) (kg * 8);

    struct Stage
    {
        u32x4 w[TPW];
        u32x2 a[4];
        uint16_t s[TPW], z[TPW];
    };
    auto fetch_operands = [&](Stage& st, int kt0)
    {
        int const kt_mine = kt0 + c / R; // the tile whose activations this lane holds
        bool const a_ok = c < ROWS && kt_mine < KT;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            st.a[j] = buffer_load_x2(act_rsrc, a_ok ? a_lane + (uint32_t) (kt_mine * 128 + j * 32) : kOob);
#pragma unroll
        for (int i = 0; i < TPW; ++i)
            st.w[i] = buffer_load_x4_once(w_rsrc, kt0 + i < KT ? wlane + (uint32_t) (kt0 + i) * 1024u : kOob);
    };
    auto kt_of = [&](int pass) { return (pass * WAVES + wave) * TPW; };
    Stage st[1];
    fetch_operands(st[0], kt_of(0));
    __builtin_amdgcn_sched_barrier(0);

    uint32_t const sz_bytes = (uint32_t) scale_rows * (uint32_t) n * 2u;
    auto const sc_rsrc = make_rsrc(scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? zeros : scales, sz_bytes);
    uint32_t const sc_lane = (uint32_t) (strip * 16 + c) * 2u;
    uint32_t const magic = tail.group_magic;
    // the scale (and zero) of every tile of the pass for this lane's column
    auto fetch_scales = [&](Stage& st, int kt0)
    {
#pragma unroll
        for (int i = 0; i < TPW; ++i)
        {
            uint32_t const off = kt0 + i < KT ? w4a8_scale_row((uint32_t) (kt0 + i), magic) * (uint32_t) n * 2u + sc_lane : kOob;
            st.s[i] = buffer_load_u16(sc_rsrc, off);
            st.z[i] = ZERO ? buffer_load_u16(zr_rsrc, off) : (uint16_t) 0;
        }
    };
    fetch_scales(st[0], kt_of(0));
    __builtin_amdgcn_sched_barrier(0);

    float qf[4];
    fp8_table_lane_values(kg, qf);
    [[maybe_unused]] Fp8LookupConsts const lk = fp8_lookup_consts();
    float total[R];
#pragma unroll
    for (int i = 0; i < R; ++i)
        total[i] = 0.f;
    auto compute = [&](Stage& st)
    {
        i32x8 a;
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            uint32_t a0, a1;
            fp8_a_order(st.a[j][0], st.a[j][1], a0, a1);
            a[2 * j] = (int) a0;
            a[2 * j + 1] = (int) a1;
        }
        f32x4 acc[TPW];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
        {
            float const sc = EH::from_bits(st.s[i]);
            float const zr = ZERO ? EH::from_bits(st.z[i]) : 0.f;
            Fp8Table const table = build_fp8_table(sc, zr, qf);
            i32x8 b;
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                uint32_t b0, b1;
                fp8_lookup8(st.w[i][j], table, lk, b0, b1);
                b[2 * j] = (int) b0;
                b[2 * j + 1] = (int) b1;
            }
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        }
        // register r of lane (kg, c) is row kg * 4 + r of the M-tile: tile (kg * 4 + r) / R of the pass
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float P = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                int const t = (q * 4 + r) / R;
                if (t < TPW)
                    P = kg == q ? acc[t][r] : P;
            }
            total[r % R] += P;
        }
    };
    compute(st[0]);
    if constexpr (MULTI)
    {
        int const passes = (KT + WAVES * TPW - 1) / (WAVES * TPW);
        for (int pass = 1; pass < passes; ++pass)
        {
            __builtin_amdgcn_sched_barrier(0);
            fetch_operands(st[0], kt_of(pass));
            fetch_scales(st[0], kt_of(pass));
            __builtin_amdgcn_sched_barrier(0);
            compute(st[0]);
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i)
        before_mode_change(total[i]);
    fp8_saturation_off();

    // ---- rows (lanes kg) of a wavefront, then the wavefronts, in fixed order ----
    __shared__ float red[WAVES][R][16];
#pragma unroll
    for (int i = 0; i < R; ++i)
    {
        total[i] += __shfl_xor(total[i], 16);
        total[i] += __shfl_xor(total[i], 32);
        if (kg == 0)
            red[wave][i][c] = total[i];
    }
    __syncthreads();
    if (threadIdx.x < 16 * R)
    {
        int const row = threadIdx.x >> 4;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][row][c];
        int const ocol = strip * 16 + c;
        float const bias = tail.bias ? EO::load(tail.bias, ocol) : 0.f;
        if (row < tail.m)
            static_cast<uint16_t*>(out)[(size_t) row * n + ocol]
                = EO::store(after_mode_change(__builtin_fmaf(tail.alpha, sum, bias)));
    }
}

namespace
{
template <int ODT, bool ZERO, int WAVES, int TPW, int R>
int launch_row_w4a8_variant(StreamParams const& sp, hipStream_t stream)
{
    if constexpr (TPW * R > 16)
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 row stream shape: %d tiles x %d rows do not fit the 16 MFMA rows", TPW, R);
    else
    {
        bool const multi = sp.k_tiles > WAVES * TPW; // K longer than one pass of the workgroup
        int const groups_per_xcd = (sp.strips + 7) / 8;
        dim3 grid(groups_per_xcd * 8), block(WAVES * 64);
        note_launch("stream row w4a8 waves=%d tpw=%d passes=%d rows=%d", WAVES, TPW,
            (sp.k_tiles + WAVES * TPW - 1) / (WAVES * TPW), R);
        RowW4a8Tail const tail{sp.bias, sp.alpha, sp.m, sp.group_magic};
        int const act_bytes = sp.m * sp.k;
        if (multi)
            hipLaunchKernelGGL((stream_row_w4a8_kernel<ODT, ZERO, WAVES, TPW, true, R>), grid, block, 0, stream, sp.weight,
                sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, groups_per_xcd, sp.n, sp.scale_rows, act_bytes, sp.out, tail);
        else
            hipLaunchKernelGGL((stream_row_w4a8_kernel<ODT, ZERO, WAVES, TPW, false, R>), grid, block, 0, stream, sp.weight,
                sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, groups_per_xcd, sp.n, sp.scale_rows, act_bytes, sp.out, tail);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess)
            return fail(WOQ_ERR_RUNTIME, "W4A8 row stream kernel launch failed: %s", hipGetErrorString(err));
        return WOQ_OK;
    }
}

template <int ODT, bool ZERO, int R>
int launch_row_w4a8_shaped(StreamParams const& sp, int waves, int tpw, hipStream_t s)
{
#define WOQ_ROW(WAVES_, TPW_)                                                                                          \
    if (waves == WAVES_ && tpw == TPW_)                                                                                \
        return launch_row_w4a8_variant<ODT, ZERO, WAVES_, TPW_, R>(sp, s);
    WOQ_ROW(4, 8)
    WOQ_ROW(8, 8)
    WOQ_ROW(16, 8)
    WOQ_ROW(4, 4)
    WOQ_ROW(8, 4)
    WOQ_ROW(16, 4)
    WOQ_ROW(14, 4) // K = 14336 is 112 tiles: shapes that divide it
    WOQ_ROW(16, 7)
#undef WOQ_ROW
    return fail(WOQ_ERR_UNSUPPORTED, "W4A8 row stream shape waves=%d tpw=%d is not instantiated", waves, tpw);
}

template <int ODT, bool ZERO>
int launch_row_w4a8_rows(StreamParams const& sp, int waves, int tpw, hipStream_t s)
{
    if (sp.m == 1)
        return launch_row_w4a8_shaped<ODT, ZERO, 1>(sp, waves, tpw, s);
    if (sp.m == 2)
        return launch_row_w4a8_shaped<ODT, ZERO, 2>(sp, waves, tpw, s);
    return launch_row_w4a8_shaped<ODT, ZERO, 4>(sp, waves, tpw, s);
}
} // namespace

// sp: act (e4m3), weight, scales, zeros (fp16), bias, out, alpha, m, n, k, k_tiles, strips, scale_rows, group_magic
int launch_stream_row_w4a8(StreamParams const& sp, int out_dtype, int waves, int tpw, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    if (sp.m < 1 || sp.m > 4 || sp.k % 128)
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 row stream kernel: one to four rows, k %% 128 == 0");
    bool const zero = sp.zeros != nullptr;
    if (out_dtype == WOQ_BF16)
        return zero ? launch_row_w4a8_rows<WOQ_BF16, true>(sp, waves, tpw, s) : launch_row_w4a8_rows<WOQ_BF16, false>(sp, waves, tpw, s);
    return zero ? launch_row_w4a8_rows<WOQ_FP16, true>(sp, waves, tpw, s) : launch_row_w4a8_rows<WOQ_FP16, false>(sp, waves, tpw, s);
}

} // namespace woq
