// W4A8 decode: weight-streaming kernel for fp8 (e4m3) activations and int4 weights, M <= 16.
//
// Same semantics as the W4A8 GEMM (gemm_w4a8.hip; the reference's fpA_intB runner instantiated
// for __nv_fp8_e4m3 x uint4, selected by weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): every
// weight is dequantized with its fp16 group scale (and zero) and rounded to e4m3, the matrix core
// accumulates fp8 x fp8 products in float32, the epilogue applies alpha and the bias.  Because the
// rounding to e4m3 is part of the result, the scale cannot be deferred to the group sums as in the
// 16-bit streaming kernel: each weight is converted exactly, in registers, by the lane that loaded
// it (about 3 VALU instructions per weight - still under what HBM delivers; the saturation to
// +-448 is done by the conversion instruction itself, see fp8_saturation_on()).
//
// Same skeleton as the 16-bit streaming kernel (stream_kernel.h): a workgroup owns NS strips of 16
// columns, its wavefronts split K (tile row kt goes to wave kt % WAVES, PF tile rows in flight
// each) and are reduced through LDS in a fixed order.  One v_mfma_f32_16x16x128_f8f6f4 covers a
// whole 128-deep tile row: lane (kg, c) supplies, for output column c (B) and activation row c (A),
// the 32 k-values 32 j + 8 kg + e (j = 0..3 slabs, e = 0..7) in that order - the tile layout's own
// order for the weights, four 8-byte loads of its activation row for A (rows >= M fall outside the
// buffer descriptor and read as zeros).
#include "stream_kernel.h"
#include "w4a8_common.h"

namespace woq
{

// LDSM 1: the workgroup stages the activation rows in LDS once (small M x K) and the lanes read
// their A pieces from there; a pipeline stage then holds packed weights and scales only.
// LDSM 2: the group scales and zeros of the workgroup's columns are staged as well.
// LDSM 3: only those (activations too large for the LDS come from registers).
// MT   16-row tiles of activations per wavefront (1; 2 for 17..32 rows, activations from registers: every
//      converted B operand then feeds two matrix instructions)
template <int ODT, bool ZERO, int NS, int WAVES, int PF, int LDSM, int MT = 1>
__global__ void __launch_bounds__(WAVES * 64) stream_w4a8_kernel(StreamParams p)
{
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    constexpr int TK = 128, SLABS = 4;
    constexpr bool ALDS = LDSM == 1 || LDSM == 2; // activation rows staged in LDS
    static_assert(MT == 1 || !ALDS, "staged activations are for at most 16 rows");
    constexpr bool SCLDS = LDSM >= 2;             // the group scales / zeros of the workgroup's columns staged
    extern __shared__ u32x4 act_lds[]; // ALDS: rows x (K + 16) bytes, then the staged scales, then zeros

    int const group = xcd_strip(blockIdx.x, p.groups_per_xcd);
    if (group >= p.groups)
        return; // whole workgroup leaves together

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const K = p.k;
    int const KT = p.k_tiles;
    int const strip0 = group * NS;

    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    constexpr uint32_t kPast = 0x80000000u;
    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K);
    uint32_t const sz_bytes = (uint32_t) p.scale_rows * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) KT * 1024u);
    uint32_t const magic = p.group_magic; // groups above 128: table row of a tile row (w4a8_scale_row)

    // strips past the end of N (last group only) are clamped for loads and skipped at the store
    uint32_t wlane[NS], sc_lane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        int const strip = strip0 + s < p.strips ? strip0 + s : p.strips - 1;
        wlane[s] = ((uint32_t) strip * (uint32_t) KT * 64u + (uint32_t) lane) * 16u;
        sc_lane[s] = (uint32_t) (strip * 16 + c) * 2u;
    }
    // activation row c (rows >= m start past the end of the buffer), this lane's 8 bytes of slab 0
    uint32_t const a_lane = (uint32_t) c * (uint32_t) K + (uint32_t) kg * 8u;

    // LDS copy: row r at byte r * lds_row (+16: the rows of a half-wavefront's 8-byte reads fall
    // into different banks); lanes of rows >= m read row m-1, their outputs are never stored
    uint32_t const lds_row = (uint32_t) K + 16u;
    int const a_row = c < p.m ? c : p.m - 1;
    char const* a_lds = reinterpret_cast<char const*>(act_lds) + (uint32_t) a_row * lds_row + (uint32_t) kg * 8u;
    // SCLDS variants stage the group scales (and zeros) of the workgroup's columns behind the
    // activations (it pays on long K, where the staging pass is a small part of the workgroup's time): one row of NS * 16 values per tile row of K (group 128 = one tile row), strip
    // slot s at columns s * 16 ..; a pipeline stage then holds packed weights only
    constexpr uint32_t SC_ROW = NS * 32u;
    char* const sc_lds = reinterpret_cast<char*>(act_lds) + (ALDS ? (uint32_t) (p.m < 16 ? p.m : 16) * lds_row : 0u);
    char* const zr_lds = sc_lds + (uint32_t) KT * SC_ROW;

    struct Stage
    {
        u32x4 w[NS];
        u32x2 a[ALDS ? 1 : SLABS][MT];
        uint16_t s[NS];
        uint16_t z[NS];
    };

    auto fetch = [&](Stage& st, int kt)
    {
        uint32_t const past = kt < KT ? 0u : kPast; // scalar select: a tile row past K reads zeros everywhere
#pragma unroll
        for (int s = 0; s < NS; ++s)
            st.w[s] = buffer_load_x4_once(w_rsrc, (wlane[s] + (uint32_t) kt * 1024u) | past);
        if constexpr (!ALDS)
        {
#pragma unroll
            for (int j = 0; j < SLABS; ++j)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    st.a[j][mt] = buffer_load_x2(
                        act_rsrc, (a_lane + (uint32_t) mt * 16u * (uint32_t) K + (uint32_t) (kt * TK + j * 32)) | past);
        }
        if constexpr (!SCLDS)
        {
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                uint32_t const off = (w4a8_scale_row((uint32_t) kt, magic) * (uint32_t) p.n * 2u + sc_lane[s]) | past;
                st.s[s] = buffer_load_u16(sc_rsrc, off);
                if constexpr (ZERO)
                    st.z[s] = buffer_load_u16(zr_rsrc, off);
            }
        }
    };
    // raw scale / zero of strip slot s for tile row kt: from the stage, or from the staged copy
    auto scale_bits = [&](Stage const& st, int kt, int s) -> uint16_t
    {
        if constexpr (SCLDS)
            return *reinterpret_cast<uint16_t const*>(sc_lds + (uint32_t) kt * SC_ROW + (uint32_t) (s * 16 + c) * 2u);
        else
            return st.s[s];
    };
    auto zero_bits = [&](Stage const& st, int kt, int s) -> uint16_t
    {
        if constexpr (SCLDS)
            return *reinterpret_cast<uint16_t const*>(zr_lds + (uint32_t) kt * SC_ROW + (uint32_t) (s * 16 + c) * 2u);
        else
            return st.z[s];
    };

    [[maybe_unused]] NibbleConsts const nib = nibble_consts<WOQ_FP16>();
    [[maybe_unused]] float qf[4];
    fp8_table_lane_values(kg, qf);
    [[maybe_unused]] Fp8LookupConsts const lk = fp8_lookup_consts();
    // Saturation to +-448 is part of the conversion: the wavefront runs with the conversion instruction's
    // own saturating mode switched on (fp8_saturation_on below), as the tiled kernel does, so no clamp and
    // no test for scales that could reach the limit is needed.
    auto convert_and_multiply = [&](Stage const& st, int kt, i32x8 const (&a)[MT])
    {
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            float const sc = EH::from_bits(scale_bits(st, kt, s));
            float const zr = ZERO ? EH::from_bits(zero_bits(st, kt, s)) : 0.f;
            i32x8 b;
            if constexpr (MT == 1)
            {
                // the sixteen possible results of this (group, column), then every weight a table look-up
                // (70B gate_up at M = 1: 54.3 -> 51.1 us, at M = 16 56.4 -> 52.6; with two row tiles the
                // reordering of twice the A operand makes it 4 % slower than the arithmetic form)
                Fp8Table const table = build_fp8_table(sc, zr, qf);
#pragma unroll
                for (int j = 0; j < SLABS; ++j)
                {
                    uint32_t b0, b1;
                    fp8_lookup8(st.w[s][j], table, lk, b0, b1);
                    b[2 * j] = (int) b0;
                    b[2 * j + 1] = (int) b1;
                }
            }
            else
            {
#pragma unroll
                for (int j = 0; j < SLABS; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        b[2 * j + h] = (int) dequant4_fp8<ZERO, false>(st.w[s][j], h, sc, zr, nib);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[s][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[mt], b, acc[s][mt], 0, 0, 0, 0, 0, 0);
        }
    };
    auto compute = [&](Stage const& st, int kt)
    {
        i32x8 a[MT];
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
            {
                u32x2 const v = ALDS ? *reinterpret_cast<u32x2 const*>(a_lds + (uint32_t) (kt * TK + j * 32))
                                     : st.a[ALDS ? 0 : j][mt];
                uint32_t a0 = v[0], a1 = v[1];
                if constexpr (MT == 1) // the lane's eight k-values in the order the weight look-up delivers them
                    fp8_a_order(v[0], v[1], a0, a1);
                a[mt][2 * j] = (int) a0;
                a[mt][2 * j + 1] = (int) a1;
            }
        convert_and_multiply(st, kt, a);
    };

    // tile rows of this wavefront: kt = wave + it * WAVES.  Every load tolerates kt >= KT, so
    // prologue and loop are unconditional and the compiler's wait counts stay exact.
    int const n_my = (KT - wave + WAVES - 1) / WAVES;
    Stage st[PF];
    fp8_saturation_on(); // the conversions below rely on it; off again before the epilogue
    if constexpr (ALDS || SCLDS)
    {
        // Staged operands (the activations, the group scales / zeros of this workgroup's columns) are
        // requested FIRST, two 16-byte chunks of each per thread, and the weight prefetch right behind
        // them: loads complete in order, so the LDS writes and the barrier wait for the small staged
        // loads (from L2) only, while the weights stay in flight.  Longer operands are finished by
        // plain loops after the prefetch.
        constexpr int THREADS = WAVES * 64;
        constexpr int UA = 2;
        int const rows = p.m < 16 ? p.m : 16;
        int const chunks_per_row = K / 16;
        int const act_chunks = ALDS ? rows * chunks_per_row : 0;
        int const sc_chunks = SCLDS ? KT * NS * 2 : 0; // NS * 2 chunks of 8 columns per tile row of K
        auto act_src = [&](int idx, uint32_t& at)
        {
            int const row = rows == 1 ? 0 : idx / chunks_per_row, ch = idx - row * chunks_per_row;
            at = (uint32_t) row * lds_row + (uint32_t) ch * 16u;
            return idx < act_chunks ? (uint32_t) row * (uint32_t) K + (uint32_t) ch * 16u : kPast;
        };
        // strips past the end of N are clamped as for the weights
        auto sc_src = [&](int idx, uint32_t& at)
        {
            int const kt = idx / (NS * 2), ch = idx - kt * (NS * 2);
            int const strip = strip0 + (ch >> 1) < p.strips ? strip0 + (ch >> 1) : p.strips - 1;
            at = (uint32_t) kt * SC_ROW + (uint32_t) ch * 16u;
            // (the staged copy keeps one row per tile row: tile rows of one group hold the same values)
            return idx < sc_chunks
                ? (w4a8_scale_row((uint32_t) kt, magic) * (uint32_t) p.n + (uint32_t) (strip * 16 + (ch & 1) * 8)) * 2u
                : kPast;
        };
        u32x4 av[UA], sv[UA], zv[UA];
        uint32_t a_at[UA], s_at[UA];
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            if (u * THREADS < act_chunks) // uniform
                av[u] = buffer_load_x4(act_rsrc, act_src(threadIdx.x + u * THREADS, a_at[u]));
            if (u * THREADS < sc_chunks) // uniform
            {
                uint32_t const off = sc_src(threadIdx.x + u * THREADS, s_at[u]);
                sv[u] = buffer_load_x4(sc_rsrc, off);
                if constexpr (ZERO)
                    zv[u] = buffer_load_x4(zr_rsrc, off);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // at most two pipeline stages and 32 KiB of weights per workgroup before the barrier (a CU keeps
        // only some tens of KiB of loads in flight; a wavefront whose requests do not fit waits at the
        // issue, in front of its LDS writes); the rest of the prefetch follows the barrier
        constexpr int P0_FIT = 32 / (NS * WAVES) < 1 ? 1 : 32 / (NS * WAVES);
        constexpr int P0 = P0_FIT < (PF < 2 ? PF : 2) ? P0_FIT : (PF < 2 ? PF : 2);
#pragma unroll
        for (int i = 0; i < P0; ++i)
            fetch(st[i], wave + i * WAVES);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            if (u * THREADS < act_chunks && (int) threadIdx.x + u * THREADS < act_chunks)
                *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(act_lds) + a_at[u]) = av[u];
            if (u * THREADS < sc_chunks && (int) threadIdx.x + u * THREADS < sc_chunks)
            {
                *reinterpret_cast<u32x4*>(sc_lds + s_at[u]) = sv[u];
                if constexpr (ZERO)
                    *reinterpret_cast<u32x4*>(zr_lds + s_at[u]) = zv[u];
            }
        }
        for (int idx = threadIdx.x + UA * THREADS; idx < act_chunks; idx += THREADS)
        {
            uint32_t at;
            uint32_t const off = act_src(idx, at);
            *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(act_lds) + at) = buffer_load_x4(act_rsrc, off);
        }
        for (int idx = threadIdx.x + UA * THREADS; idx < sc_chunks; idx += THREADS)
        {
            uint32_t at;
            uint32_t const off = sc_src(idx, at);
            *reinterpret_cast<u32x4*>(sc_lds + at) = buffer_load_x4(sc_rsrc, off);
            if constexpr (ZERO)
                *reinterpret_cast<u32x4*>(zr_lds + at) = buffer_load_x4(zr_rsrc, off);
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = P0; i < PF; ++i)
            fetch(st[i], wave + i * WAVES);
        __builtin_amdgcn_sched_barrier(0);
    }
    else
    {
#pragma unroll
        for (int i = 0; i < PF; ++i)
            fetch(st[i], wave + i * WAVES);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (int it = 0; it < n_my; it += PF)
    {
#pragma unroll
        for (int i = 0; i < PF; ++i)
        {
            if (it + i < n_my)
                compute(st[i], wave + (it + i) * WAVES);
            __builtin_amdgcn_sched_barrier(0);
            fetch(st[i], wave + (it + i + PF) * WAVES);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- cross-wavefront reduction (fixed order) and epilogue: out = T(alpha * sum + bias) ----
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            before_mode_change(acc[s][mt]);
    fp8_saturation_off();
    constexpr int SLOTS = NS * MT * 4;
    __shared__ float red[WAVES][SLOTS][64];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (mt * 16 + kg * 4 + r < p.m)
                    red[wave][(s * MT + mt) * 4 + r][lane] = acc[s][mt][r];
    __syncthreads();

    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    for (int e = threadIdx.x; e < SLOTS * 64; e += WAVES * 64)
    {
        int const slot = e >> 6, ln = e & 63;
        int const s = (slot >> 2) / MT, mt = (slot >> 2) % MT, r = slot & 3;
        int const row = mt * 16 + (ln >> 4) * 4 + r;
        if (row >= p.m || strip0 + s >= p.strips)
            continue;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][slot][ln];
        int const ocol = (strip0 + s) * 16 + (ln & 15);
        float const bias = p.bias ? EO::load(p.bias, ocol) : 0.f;
        out16[(size_t) row * p.n + ocol] = EO::store(after_mode_change(__builtin_fmaf(p.alpha, sum, bias)));
    }
}

namespace
{

struct W4a8Shape
{
    int ns, waves, pf, lds;
};

constexpr size_t kMaxActLds = 48 * 1024;
// most dynamic LDS of a staged variant: activations plus the group scales and zeros of its columns
// (k / 128 rows of ns * 32 bytes each); the static reduction buffer takes up to 32 KiB more
constexpr size_t kMaxStagedLds = 96 * 1024;

size_t scale_lds_bytes(int k_tiles, int ns, bool zeros)
{
    return (size_t) k_tiles * (size_t) ns * 32 * (zeros ? 2 : 1);
}

size_t act_lds_bytes(int m, int k)
{
    return (size_t) (m < 16 ? m : 16) * ((size_t) k + 16);
}

// WOQ_STREAM_SHAPE="ns,waves,pf,lds" overrides the heuristic (for tuning sweeps)
W4a8Shape pick_shape(int m, int k, int strips, int k_tiles)
{
    EnvOverrides const& env = env_overrides();
    if (env.has_stream_shape)
        return {env.stream_shape[0], env.stream_shape[1], env.stream_shape[2], env.stream_shape[3]};
    // measured on MI355X.  Activations that fit the LDS staging area: one strip per wavefront
    // and 8-way split K (two strips on very wide matrices, deeper prefetch on long K).
    if (m <= 16 && act_lds_bytes(m, k) <= kMaxActLds)
    {
        // the group scales join the activations in LDS from K = 8192 on (2-4 % there; on K = 4096 the
        // staging pass costs more than the loads it saves)
        int const lds = k_tiles >= 64 && act_lds_bytes(m, k) + scale_lds_bytes(k_tiles, 2, true) <= kMaxStagedLds ? 2 : 1;
        if (strips >= 2048)
            return {2, 8, 2, lds};
        return k_tiles >= 112 ? W4a8Shape{1, 8, 4, lds} : W4a8Shape{1, 8, 2, lds};
    }
    // otherwise (activations in registers) the group scales alone are staged, and two strips per
    // wavefront share the activation loads once there are enough column groups to fill the chip, four
    // on very wide matrices with more than 8 rows; narrow matrices keep one strip (swept over every
    // instantiated shape on the Llama-3-8B / 70B layer shapes, M = 8 and 16)
    int const lds = scale_lds_bytes(k_tiles, 4, true) <= kMaxStagedLds ? 3 : 0;
    // 17..32 rows (two 16-row tiles per wavefront): the activation loads weigh twice as much, so wider
    // workgroups earlier (70B qkv, 640 strips, M = 32: 48.9 / 35.7 / 23.3 us with 1 / 2 / 4 strips)
    if (m > 16)
        return strips > 512 ? W4a8Shape{4, 8, 2, lds} : (strips >= 256 ? W4a8Shape{2, 8, 2, lds} : W4a8Shape{1, 8, 2, lds});
    if (strips > 1024)
        return m > 8 ? W4a8Shape{4, 8, 2, lds} : W4a8Shape{2, 8, 2, lds};
    if (strips >= 512 || (strips >= 384 && m > 4))
        return {2, 8, 2, lds};
    return {1, 8, 2, lds};
}

template <int ODT, bool ZERO, int NS, int WAVES, int PF, int LDSM, int MT = 1>
int launch_variant(StreamParams sp, hipStream_t stream)
{
    auto kernel = stream_w4a8_kernel<ODT, ZERO, NS, WAVES, PF, LDSM, MT>;
    size_t lds = 0;
    if constexpr (LDSM != 0)
    {
        lds = LDSM == 3 ? 0 : act_lds_bytes(sp.m, sp.k);
        if (lds > kMaxActLds)
            return fail(WOQ_ERR_UNSUPPORTED, "activations of %zu bytes do not fit the LDS staging area", lds);
        lds += LDSM >= 2 ? scale_lds_bytes(sp.k_tiles, NS, ZERO) : 0;
        if (lds > kMaxStagedLds)
            return fail(WOQ_ERR_UNSUPPORTED, "staged operands of %zu bytes do not fit the LDS staging area", lds);
        static std::atomic<uint64_t> raised{0}; // one bit per device
        if (lds > 32 * 1024)
            if (int rc = raise_lds_once(raised, reinterpret_cast<void const*>(kernel), (int) kMaxStagedLds))
                return rc;
    }
    sp.groups = (sp.strips + NS - 1) / NS;
    sp.groups_per_xcd = (sp.groups + 7) / 8;
    dim3 grid(sp.groups_per_xcd * 8), block(WAVES * 64);
    note_launch("stream w4a8 mt=%d ns=%d waves=%d pf=%d lds=%d", MT, NS, WAVES, PF, LDSM);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, sp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "W4A8 stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int ODT, bool ZERO>
int launch_shaped(StreamParams const& sp, hipStream_t s)
{
    W4a8Shape const sh = pick_shape(sp.m, sp.k, sp.strips, sp.k_tiles);
    if (sp.m > 16)
    {
        // 17..32 rows: two 16-row tiles per wavefront, activations from registers
#define WOQ_SHAPE2(NS_, WAVES_, PF_, LDS_)                                                                             \
    if (sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_ && sh.lds == LDS_)                                   \
        return launch_variant<ODT, ZERO, NS_, WAVES_, PF_, LDS_, 2>(sp, s);
        WOQ_SHAPE2(1, 8, 2, 0)
        WOQ_SHAPE2(2, 8, 2, 0)
        WOQ_SHAPE2(1, 8, 2, 3)
        WOQ_SHAPE2(2, 8, 2, 3)
        WOQ_SHAPE2(4, 8, 2, 3)
#undef WOQ_SHAPE2
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 stream shape ns=%d waves=%d pf=%d lds=%d is not instantiated for 17..32 rows",
            sh.ns, sh.waves, sh.pf, sh.lds);
    }
#define WOQ_SHAPE(NS_, WAVES_, PF_, LDS_)                                                                              \
    if (sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_ && sh.lds == LDS_)                                   \
        return launch_variant<ODT, ZERO, NS_, WAVES_, PF_, LDS_>(sp, s);
    WOQ_SHAPE(1, 8, 2, 0)
    WOQ_SHAPE(1, 16, 2, 0)
    WOQ_SHAPE(2, 8, 2, 0)
    WOQ_SHAPE(2, 8, 3, 0)
    WOQ_SHAPE(2, 4, 4, 0)
    WOQ_SHAPE(4, 8, 2, 0)
    WOQ_SHAPE(1, 8, 2, 1)
    WOQ_SHAPE(1, 8, 4, 1)
    WOQ_SHAPE(2, 8, 2, 1)
    WOQ_SHAPE(2, 4, 4, 1)
    WOQ_SHAPE(4, 8, 2, 1)
    WOQ_SHAPE(1, 8, 2, 2)
    WOQ_SHAPE(1, 8, 4, 2)
    WOQ_SHAPE(2, 8, 2, 2)
    WOQ_SHAPE(1, 8, 2, 3)
    WOQ_SHAPE(2, 8, 2, 3)
    WOQ_SHAPE(2, 8, 3, 3)
    WOQ_SHAPE(2, 4, 4, 3)
    WOQ_SHAPE(4, 8, 2, 3)
#undef WOQ_SHAPE
    return fail(WOQ_ERR_UNSUPPORTED, "W4A8 stream shape ns=%d waves=%d pf=%d lds=%d is not instantiated", sh.ns,
        sh.waves, sh.pf, sh.lds);
}

} // namespace

int launch_stream_row_w4a8(StreamParams const& sp, int out_dtype, int waves, int tpw, void* stream);
bool pick_row_w4a8_shape(int m, int n, int k, int& waves, int& tiles);
int launch_stream_rows_w4a8(StreamParams const& sp, int out_dtype, int waves, int ns, int tpw, void* stream);
bool pick_rows_w4a8_shape(int m, int n, int k, int& waves, int& ns, int& tiles);

int launch_stream_w4a8(MatmulProblem const& p, void* stream)
{
    if (p.m > kStreamW4a8MaxM)
        return fail(WOQ_ERR_UNSUPPORTED, "unsupported m: the W4A8 streaming kernel covers m <= %d (got %d)",
            kStreamW4a8MaxM, p.m);
    if (p.act_dtype != WOQ_FP8_E4M3 || p.group_size < 128 || p.group_size % 128 || p.k % 128)
        return fail(WOQ_ERR_INVALID_ARGUMENT,
            "W4A8 streaming kernel: e4m3 activations, group size a multiple of 128, k %% 128 == 0");
    StreamParams sp;
    sp.act = p.act;
    sp.pqs = nullptr;
    sp.weight = p.weight;
    sp.scales = p.scales;
    sp.zeros = p.zeros;
    sp.bias = p.bias;
    sp.out = p.out;
    sp.alpha = p.alpha;
    sp.m = p.m;
    sp.n = p.n;
    sp.k = p.k;
    sp.k_tiles = p.k / 128;
    sp.strips = p.n / kTileN;
    sp.scale_rows = (p.k + p.group_size - 1) / p.group_size;
    sp.group_magic = w4a8_scale_row_magic(p.group_size);
    sp.groups = sp.groups_per_xcd = 0;
    auto s = static_cast<hipStream_t>(stream);
    bool const zero = p.zeros != nullptr;
    {
        // one to four rows: the row kernel (stream_row_w4a8.hip), where the rule (or WOQ_ROW_SHAPE) picks it
        int waves = 0, tiles = 0;
        if (pick_row_w4a8_shape(p.m, p.n, p.k, waves, tiles))
        {
            int const rc = launch_stream_row_w4a8(sp, p.out_dtype, waves, tiles, stream);
            if (rc != WOQ_ERR_UNSUPPORTED)
                return rc;
        }
        // up to sixteen rows: the multi-row kernel (stream_rows_w4a8.hip), where its rule (or WOQ_ROWS_SHAPE) picks it
        int ns = 0;
        if (pick_rows_w4a8_shape(p.m, p.n, p.k, waves, ns, tiles))
        {
            int const rc = launch_stream_rows_w4a8(sp, p.out_dtype, waves, ns, tiles, stream);
            if (rc != WOQ_ERR_UNSUPPORTED)
                return rc;
        }
    }
    if (p.out_dtype == WOQ_BF16)
        return zero ? launch_shaped<WOQ_BF16, true>(sp, s) : launch_shaped<WOQ_BF16, false>(sp, s);
    return zero ? launch_shaped<WOQ_FP16, true>(sp, s) : launch_shaped<WOQ_FP16, false>(sp, s);
}

} // namespace woq
