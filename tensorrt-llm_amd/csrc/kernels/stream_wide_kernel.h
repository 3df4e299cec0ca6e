// Weight-streaming kernel for decode on wide matrices (many output columns, one row, group scales).
//
// Same arithmetic as stream_kernel.h (packed weights straight into MFMA B operands, scales applied to
// float32 group sums together with the activation row sums), different division of work: a
// wavefront owns NS strips of 16 columns over ALL of K instead of sharing a strip group with the
// other wavefronts of its workgroup.  Wavefronts are then independent after the one barrier that
// follows the staging of the activations: no reduction through LDS, no barrier at the end, nobody
// waits for the slowest of eight wavefronts, and each wavefront runs one long, evenly pipelined
// loop with PF tile rows in flight.  It needs N / (16 * NS) wavefronts to fill the chip, so it is
// chosen for wide N only (the gate_up projections).
//
// The 16 MFMA rows hold SLOTS = 16 / R groups of K side by side (R = rows of the M-tile a slot takes):
// the g-th group of K puts its activations in MFMA rows (g % SLOTS) * R .. + R - 1 and zeros elsewhere,
// so one accumulator collects the partial sums of SLOTS consecutive groups, each in its own rows,
// and scales are applied once per SLOTS groups ("window").  The scales and zeros of a window (SLOTS
// rows of NS * 16 columns each) are fetched by the wavefront itself with 16-byte loads at the start of
// the window and redistributed through a wavefront-private piece of LDS when the window ends.
#pragma once

#include "stream_kernel.h"

namespace woq
{

// lanes l, l + 16, l + 32, l + 48 -> their sum, in every lane (fixed order)
__device__ __forceinline__ float sum_over_kg(float v)
{
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int NS, int WAVES, int PF, int SLOTS>
__global__ void __launch_bounds__(WAVES * 64) stream_wide_kernel(StreamParams p)
{
    using E = Elem<DT>;
    static_assert(GROUP != 0, "group scales only");
    static_assert(SLOTS == 16 || SLOTS == 4, "one row (16 slots) or up to four rows (4 slots)");
    constexpr int R = 16 / SLOTS;
    constexpr int TK = BITS == 4 ? 128 : 64;
    static_assert(GROUP <= TK, "a group does not span tile rows here");
    constexpr int SEG = GROUP;
    constexpr int SEG_SLABS = SEG / 32;
    constexpr int SEGS = TK / SEG;
    constexpr float OFF = Offset<DT, BITS>::value;
    constexpr int THREADS = WAVES * 64;
    // 16-byte chunks of one window's scales (and zeros): SLOTS rows x NS * 2 chunks, zeros behind them
    constexpr int WCHUNKS = SLOTS * NS * 2;
    constexpr int WLOADS = (WCHUNKS * (ZERO ? 2 : 1) + 63) / 64;
    constexpr uint32_t kOob = 0x7FFFFFF0u;
    extern __shared__ u32x4 wide_lds[]; // activation rows, row sums, 256 zero bytes, per-wavefront scale windows

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const K = p.k, KT = p.k_tiles;
    int const groups_k = KT * SEGS; // groups of K including the zero-padded tail
    int const wg = xcd_strip(blockIdx.x, p.groups_per_xcd);
    int const strip0 = (wg * WAVES + wave) * NS; // first strip of this wavefront
    if (wg >= p.groups)
        return; // whole workgroup leaves together
    bool const has_work = strip0 < p.strips;

    NibbleConsts const nib = nibble_consts<DT>();
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};
    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K * 2u);
    auto const pqs_rsrc = make_rsrc(PQS ? p.pqs : p.act, (uint32_t) K * 2u);
    uint32_t const sz_bytes = (uint32_t) (K / GROUP) * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) KT * 1024u);

    int strip_of[NS];
    uint32_t wlane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        strip_of[s] = strip0 + s < p.strips ? strip0 + s : p.strips - 1;
        wlane[s] = ((uint32_t) strip_of[s] * (uint32_t) KT * 64u + (uint32_t) lane) * 16u;
    }

    // LDS: rows of (smoothed) activations, the row sums of every group (16 floats per group), zeros,
    // then WAVES scale windows
    int const rows = p.m;
    uint32_t const lds_row = (uint32_t) KT * TK * 2u + 16u;
    char* const lds = reinterpret_cast<char*>(wide_lds);
    char* const sum_lds = lds + (uint32_t) rows * lds_row;
    char* const zero_lds = sum_lds + (uint32_t) groups_k * 64u;
    char* const win_lds = zero_lds + 256u + (uint32_t) wave * (uint32_t) (WLOADS * 1024);
    int const c_row = c & (R - 1);
    int const a_row = c_row < rows ? c_row : rows - 1;
    char const* const a_lds = lds + (uint32_t) a_row * lds_row + (uint32_t) kg * 16u;
    int const c_slot = c / R;

    struct Stage
    {
        u32x4 w[NS];
    };
    auto fetch = [&](Stage& st, int kt)
    {
        uint32_t const tile_off = (kt < KT && has_work) ? (uint32_t) kt * 1024u : 0x80000000u;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            st.w[s] = buffer_load_x4_once(w_rsrc, wlane[s] + tile_off);
    };
    // chunk `ch` of window `wnd`: row (slot) ch / (NS*2) of the scales, or of the zeros behind them
    auto window_fetch = [&](u32x4 (&wv)[WLOADS], int wnd)
    {
#pragma unroll
        for (int t = 0; t < WLOADS; ++t)
        {
            int const ch = t * 64 + lane;
            bool const is_zero = ZERO && ch >= WCHUNKS;
            int const cc = is_zero ? ch - WCHUNKS : ch;
            int const slot = cc / (NS * 2), piece = cc - slot * (NS * 2);
            int const g = wnd * SLOTS + slot;
            bool const ok = cc < WCHUNKS && g < K / GROUP && has_work && strip0 * 16 + piece * 8 < p.n;
            uint32_t const off = ((uint32_t) g * (uint32_t) p.n + (uint32_t) (strip0 * 16 + piece * 8)) * 2u;
            wv[t] = is_zero ? buffer_load_x4(zr_rsrc, ok ? off : kOob) : buffer_load_x4(sc_rsrc, ok ? off : kOob);
        }
    };

    f32x4 acc_out[NS], acc_p[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        acc_out[s] = acc_p[s] = zero4;

    // ---- prologue: staged loads first, weight prefetch right behind them, then the LDS writes ----
    constexpr int UA = 2;
    int const chunks_per_row = KT * TK / 8;
    int const act_chunks = rows * chunks_per_row;
    auto act_offset = [&](int idx, uint32_t& lds_at, uint32_t& ch, uint32_t& sum_at)
    {
        int const row = rows == 1 ? 0 : idx / chunks_per_row;
        ch = (uint32_t) (idx - row * chunks_per_row);
        lds_at = (uint32_t) row * lds_row + ch * 16u;
        sum_at = ch / (SEG / 8) * 64u + (uint32_t) row * 4u;
        bool const ok = idx < act_chunks && (int) ch * 8 < K;
        return ok ? ((uint32_t) row * (uint32_t) K + ch * 8u) * 2u : kOob;
    };
    auto smooth = [&](u32x4 v, u32x4 sm)
    {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            v[r] = E::mul2(v[r], sm[r]);
        return v;
    };
    // sum of the SEG activations of one group: the SEG/8 consecutive lanes holding its chunks
    auto stage_sum = [&](u32x4 v, int idx, uint32_t sum_at)
    {
        float t = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            t += E::from_bits((uint16_t) (v[r] & 0xFFFFu)) + E::from_bits((uint16_t) (v[r] >> 16));
        t = dpp_add<0xB1>(t);
        t = dpp_add<0x4E>(t);
        t = dpp_add<0x141>(t);
        if constexpr (SEG == 128)
            t = dpp_add<0x140>(t);
        if ((threadIdx.x & (SEG / 8 - 1)) == 0 && idx < act_chunks)
            *reinterpret_cast<float*>(sum_lds + sum_at) = t;
    };

    Stage st[PF];
    u32x4 wv[WLOADS];
    {
        u32x4 av[UA], pv[UA];
        uint32_t a_at[UA], s_at[UA];
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            uint32_t ch;
            av[u] = buffer_load_x4(act_rsrc, act_offset(threadIdx.x + u * THREADS, a_at[u], ch, s_at[u]));
            if constexpr (PQS)
                pv[u] = buffer_load_x4(pqs_rsrc, ch * 16u);
        }
        __builtin_amdgcn_sched_barrier(0);
        window_fetch(wv, 0);
#pragma unroll
        for (int i = 0; i < PF; ++i)
            fetch(st[i], i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            u32x4 const v = PQS ? smooth(av[u], pv[u]) : av[u];
            if ((int) threadIdx.x + u * THREADS < act_chunks)
                *reinterpret_cast<u32x4*>(lds + a_at[u]) = v;
            stage_sum(v, threadIdx.x + u * THREADS, s_at[u]);
        }
        for (int idx = threadIdx.x + UA * THREADS; idx < act_chunks; idx += THREADS)
        {
            uint32_t at, ch, sum_at;
            u32x4 v = buffer_load_x4(act_rsrc, act_offset(idx, at, ch, sum_at));
            if constexpr (PQS)
                v = smooth(v, buffer_load_x4(pqs_rsrc, ch * 16u));
            *reinterpret_cast<u32x4*>(lds + at) = v;
            stage_sum(v, idx, sum_at);
        }
        if (threadIdx.x < 16)
            *reinterpret_cast<u32x4*>(zero_lds + threadIdx.x * 16u) = u32x4{0u, 0u, 0u, 0u};
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    }
    if (!has_work)
        return; // a wavefront past the last strip has done its share of the staging

    // scales of window `wnd` (in wv) -> this wavefront's LDS window -> acc_out; then the next window's fetch
    auto flush = [&](int wnd)
    {
#pragma unroll
        for (int t = 0; t < WLOADS; ++t)
            *reinterpret_cast<u32x4*>(win_lds + (uint32_t) (t * 64 + lane) * 16u) = wv[t];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            int const i = kg * 4 + r;
            int const slot = i / R;
            int const g = wnd * SLOTS + slot;
            bool const ok = g < groups_k;
            float const S = *reinterpret_cast<float const*>(
                ok ? sum_lds + (uint32_t) g * 64u + (uint32_t) (i & (R - 1)) * 4u : zero_lds);
            char const* const sp = win_lds + (uint32_t) slot * (NS * 32u) + (uint32_t) c * 2u;
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                float const sc = E::from_bits(*reinterpret_cast<uint16_t const*>(sp + s * 32));
                float const zz
                    = ZERO ? E::from_bits(*reinterpret_cast<uint16_t const*>(sp + WCHUNKS * 16 + s * 32)) : 0.f;
                float const cc = __builtin_fmaf(-OFF, sc, zz);
                acc_out[s][r] = __builtin_fmaf(sc, acc_p[s][r], __builtin_fmaf(cc, S, acc_out[s][r]));
            }
        }
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc_p[s] = zero4;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        window_fetch(wv, wnd + 1);
    };

    auto compute = [&](Stage const& stg, int kt)
    {
#pragma unroll
        for (int seg = 0; seg < SEGS; ++seg)
        {
            int const gi = kt * SEGS + seg;
            int const slot = gi & (SLOTS - 1);
            char const* const a_seg
                = c_slot == slot ? a_lds + (uint32_t) (kt * TK + seg * SEG) * 2u : zero_lds + (uint32_t) kg * 16u;
#pragma unroll
            for (int js = 0; js < SEG_SLABS; ++js)
            {
                int const j = seg * SEG_SLABS + js;
                u32x4 const a = *reinterpret_cast<u32x4 const*>(a_seg + (uint32_t) (js * 32) * 2u);
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    u32x4 b;
                    if constexpr (BITS == 4)
                        b = expand_int4<DT>(stg.w[s][j], nib);
                    else
                        b = expand_int8<DT>(stg.w[s][2 * j], stg.w[s][2 * j + 1]);
                    acc_p[s] = E::mma(a, b, acc_p[s]);
                }
            }
            if (slot == SLOTS - 1)
                flush(gi / SLOTS);
        }
    };

    for (int kt0 = 0; kt0 < KT; kt0 += PF)
    {
#pragma unroll
        for (int i = 0; i < PF; ++i)
        {
            if (kt0 + i < KT)
                compute(st[i], kt0 + i);
            __builtin_amdgcn_sched_barrier(0);
            fetch(st[i], kt0 + i + PF);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (groups_k & (SLOTS - 1))
        flush(groups_k / SLOTS);

    // ---- epilogue: fold the slots (registers and lanes kg) of each row, store ----------------------
    uint16_t* const out16 = static_cast<uint16_t*>(p.out);
    constexpr int RL = R < 4 ? R : 4;
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        float v[RL];
        if constexpr (R == 1)
            v[0] = (acc_out[s][0] + acc_out[s][1]) + (acc_out[s][2] + acc_out[s][3]);
        else
        {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[r] = acc_out[s][r];
        }
#pragma unroll
        for (int r = 0; r < RL; ++r)
        {
            float const sum = sum_over_kg(v[r]);
            int const ocol = (strip0 + s) * 16 + c;
            if (kg == 0 && r < rows && strip0 + s < p.strips)
            {
                float o = p.alpha * sum;
                if (p.bias)
                    o += E::load(p.bias, ocol);
                out16[(size_t) r * p.n + ocol] = E::store(o);
            }
        }
    }
}

// bytes of dynamic LDS of one workgroup
template <int BITS, int GROUP, bool ZERO, int NS, int WAVES, int SLOTS>
inline size_t stream_wide_lds_bytes(int m, int k)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    size_t const kt = (size_t) ((k + TK - 1) / TK);
    constexpr size_t wloads = ((size_t) SLOTS * NS * 2 * (ZERO ? 2 : 1) + 63) / 64;
    return (size_t) m * (kt * TK * 2 + 16) + kt * (TK / GROUP) * 64 + 256 + (size_t) WAVES * wloads * 1024;
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int NS, int WAVES, int PF, int SLOTS>
int launch_stream_wide_variant(StreamParams sp, hipStream_t stream)
{
    auto kernel = stream_wide_kernel<DT, BITS, GROUP, PQS, ZERO, NS, WAVES, PF, SLOTS>;
    size_t const lds = stream_wide_lds_bytes<BITS, GROUP, ZERO, NS, WAVES, SLOTS>(sp.m, sp.k);
    if (lds > (size_t) 64 * 1024)
        return fail(WOQ_ERR_UNSUPPORTED, "staged activations of %zu bytes do not fit the wide streaming kernel", lds);
    static std::atomic<uint64_t> raised{0}; // one bit per device
    if (lds > (size_t) 32 * 1024)
        if (int rc = raise_lds_once(raised, reinterpret_cast<void const*>(kernel), 64 * 1024))
            return rc;
    sp.groups = (sp.strips + NS * WAVES - 1) / (NS * WAVES); // workgroups
    sp.groups_per_xcd = (sp.groups + 7) / 8;
    dim3 grid(sp.groups_per_xcd * 8), block(WAVES * 64);
    note_launch("stream wide ns=%d waves=%d pf=%d slots=%d", NS, WAVES, PF, SLOTS);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, sp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "wide stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

// Launch shape of the wide kernel: strips per wavefront, wavefronts per workgroup, tile rows in flight.
// WOQ_WIDE_SHAPE="ns,waves,pf" overrides the rule; "0" switches the kernel off.
struct WideShape
{
    int ns, waves, pf;
};
bool pick_wide_shape(int m, int n, int k, int group, int bits, WideShape& out);

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO>
int launch_stream_wide_shaped(StreamParams const& sp, WideShape sh, hipStream_t s)
{
#define WOQ_WIDE(NS_, WAVES_, PF_)                                                                                     \
    if (sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_)                                                            \
        return launch_stream_wide_variant<DT, BITS, GROUP, PQS, ZERO, NS_, WAVES_, PF_, 16>(sp, s);
    WOQ_WIDE(2, 4, 4)
    WOQ_WIDE(1, 4, 4)
#undef WOQ_WIDE
    return fail(WOQ_ERR_UNSUPPORTED, "wide stream shape ns=%d waves=%d pf=%d is not instantiated", sh.ns, sh.waves,
        sh.pf);
}

// the wide kernel for this problem if the rule (or the override) picks it: returns true and the status
template <int DT, int BITS>
bool try_launch_stream_wide(MatmulProblem const& p, StreamParams const& sp, hipStream_t s, int& rc)
{
    WideShape sh;
    if (p.num_experts || p.m != 1 || (p.group_size != 64 && p.group_size != 128) || p.group_size > (BITS == 4 ? 128 : 64)
        || !pick_wide_shape(p.m, p.n, p.k, p.group_size, BITS, sh))
        return false;
    bool const pqs = p.pre_quant_scale != nullptr, zero = p.zeros != nullptr;
#define WOQ_WIDE_G(G)                                                                                                  \
    rc = pqs ? (zero ? launch_stream_wide_shaped<DT, BITS, G, true, true>(sp, sh, s)                                   \
                     : launch_stream_wide_shaped<DT, BITS, G, true, false>(sp, sh, s))                                 \
             : (zero ? launch_stream_wide_shaped<DT, BITS, G, false, true>(sp, sh, s)                                  \
                     : launch_stream_wide_shaped<DT, BITS, G, false, false>(sp, sh, s));
    if (p.group_size == 64)
    {
        WOQ_WIDE_G(64)
    }
    else
    {
        if constexpr (BITS == 4)
        {
            WOQ_WIDE_G(128)
        }
        else
            return false;
    }
#undef WOQ_WIDE_G
    return true;
}

} // namespace woq
