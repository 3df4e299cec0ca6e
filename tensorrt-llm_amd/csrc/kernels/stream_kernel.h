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
//     (results are bit-reproducible from run to run);
//   * for decode-sized activations (M rows x K fit in LDS) the workgroup stages the - already
//     smoothed - activations in LDS once and reads A fragments from there, so a pipeline stage
//     holds nothing but packed weights and their scales: few registers per byte in flight,
//     hence many wavefronts and many bytes in flight per CU, which is what HBM needs.
#pragma once

#include <type_traits>

#include "device_common.h"
#include "gemm_common.h"

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
    int act_stride;     // elements between rows of act (k, unless the launch splits K)
    int w_strip_tiles;  // weight tiles between neighbouring strips (k_tiles, unless the launch splits K)
    // K split across workgroups (k_slices > 1): blockIdx.y is the slice, slice_tiles tile rows each.  The
    // launcher fills k / k_tiles with the LARGEST slice (what the LDS areas are sized for) and k_total
    // with all of K; the kernel narrows the operands to its slice and stores float32 partial sums into
    // slab blockIdx.y of `partial` ([k_slices][m][n]) for the finish pass to add up in slice order.
    int k_slices = 1, slice_tiles = 0, k_total = 0;
    float* partial = nullptr;
    int real_group = 0; // host side: the problem's group size
    int split_shape[4] = {0, 0, 0, 0}; // host side: the launch shape chosen with the K split (ns, waves, pf, lds)
    int strips;         // n / 16
    int scale_rows = 1;       // rows of the scale / zero tables: ceil(k / group_size)
    uint32_t group_magic = 0; // see scale_row()
    int groups;         // ceil(strips / NS): column groups, one workgroup each
    int groups_per_xcd; // ceil(groups / 8)
    // grouped problems (rows sorted by expert, expert_rows[e] = rows of experts 0..e, device
    // memory): blockIdx.y is the expert, strides are bytes per expert; m is the total row count
    // (and, without expert_rows, the row count of the only expert)
    int64_t const* expert_rows = nullptr;
    int num_experts = 0;
    size_t weight_stride = 0, scale_stride = 0;
    int activation = kActIdentity;  // epilogue activation (grouped kernel only)
    void const* residual = nullptr; // [rows, n_out], added after the activation (grouped kernel only)
};

// Everything one wavefront needs for one tile row (NS tiles side by side), fetched together so
// that no load sits in the dependent chain of the compute that follows.
template <int NS, int SLABS, int SEGS, int MT, bool PQS, bool ALDS>
struct StreamStage
{
    u32x4 w[NS];                          // packed weights: this lane's 16 bytes of each tile
    u32x4 a[ALDS ? 1 : SLABS][ALDS ? 1 : MT]; // activation fragments (unused when they live in LDS)
    u32x4 sm[(PQS && !ALDS) ? SLABS : 1]; // pre-quant scale fragments
    uint16_t s[NS][SEGS];                 // raw scale / zero of each segment of each tile (this lane's column)
    uint16_t z[NS][SEGS];
};

// NS    strips (16 columns each) one wavefront covers; they share the activation fragments and
//       the row-sum MFMA
// WAVES wavefronts per workgroup; they split K (tile row kt goes to wave kt % WAVES)
// PF    tile rows in flight per wavefront
// ALDS  activations (m <= 16 rows) are staged in LDS by the workgroup; requires MT == 1.  The group
//       scales and zeros of the workgroup's columns are staged with them (one 16-byte load per
//       eight columns instead of a 2-byte load per lane, tile and strip inside the K loop), and
//       the activation row sums S of every segment are formed once while staging, which takes
//       the all-ones MFMA out of the K loop
// ACT   the epilogue applies p.activation; a gated activation (value column j, gate column j + n/2) pairs
//       the strips of a wavefront (even slot: value half, odd slot: gate half), output [m, n/2]
// SLOTS group slots of the 16 MFMA rows (staged activations with group scales only).  With R = 16 / SLOTS
//       rows or fewer, the M-tile has room for SLOTS groups of K side by side: the wavefront's g-th
//       group puts its activations in MFMA rows (g % SLOTS) * R .. + R - 1 and zeros in the others, so
//       one accumulator collects the partial sums of SLOTS groups, each in its own rows, and the scales
//       are applied once per SLOTS groups instead of once per group (M = 1: every 16th group, i.e. once
//       at the end for K up to 16 * WAVES tile rows).  1 = every group is scaled on its own.
template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int MT, int NS, int WAVES, int PF, int LDS,
    bool ACT = false, int SLOTS = 1>
__device__ __forceinline__ void stream_body(StreamParams const& p)
{
    constexpr bool ALDS = LDS == 1;
    static_assert(LDS != 1 || MT == 1, "LDS-staged activations are for M <= 16");
    constexpr bool SL = SLOTS > 1;
    constexpr int R = 16 / SLOTS; // rows of the M-tile one group slot takes
    static_assert(!SL || (ALDS && GROUP != 0 && !ACT), "group slots need staged activations and group scales");
    static_assert(SLOTS == 1 || SLOTS == 2 || SLOTS == 4 || SLOTS == 8 || SLOTS == 16, "SLOTS");
    using E = Elem<DT>;
    constexpr int TK = BITS == 4 ? 128 : 64;
    constexpr int SLABS = TK / 32;
    constexpr int SEG = segment_rows<GROUP, TK>(); // rows that share one scale inside a tile
    constexpr int SEG_SLABS = SEG / 32;
    constexpr int SEGS = TK / SEG;
    constexpr float OFF = Offset<DT, BITS>::value;
    using Stage = StreamStage<NS, SLABS, SEGS, MT, PQS, ALDS>;
    constexpr bool SCLDS = LDS != 0 && GROUP != 0; // group scales / zeros live in LDS
    constexpr bool SUMLDS = ALDS && GROUP != 0;    // and so do the activation row sums
    constexpr int THREADS = WAVES * 64;
    // Pipeline stages (1 KiB of weights per strip each) a wavefront requests BEFORE the staging barrier:
    // a CU keeps only some tens of KiB of loads in flight, and a wavefront whose requests do not fit
    // waits at the issue - in front of its LDS writes, so the whole workgroup's barrier waits with it.
    // At most two stages and at most 32 KiB per workgroup go first (measured: 16 / 32 / 64 KiB and
    // one / two / all stages); the rest of the prefetch is requested right after the barrier.
    constexpr int P0_FIT = 32 / (NS * WAVES) < 1 ? 1 : 32 / (NS * WAVES);
    constexpr int P0 = P0_FIT < (PF < 2 ? PF : 2) ? P0_FIT : (PF < 2 ? PF : 2);
    extern __shared__ u32x4 act_lds[]; // ALDS: rows x (KT*TK*2 + 16) bytes, then scales, then zeros

    int const group = xcd_strip(blockIdx.x, p.groups_per_xcd);
    if (group >= p.groups)
        return; // whole workgroup leaves together

    int const lane = threadIdx.x & 63;
    // the wavefront index is wave-uniform: keep it (and everything derived from it) in SGPRs so
    // that the K loop is straight scalar control flow
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15;  // column inside the strip (B operand) / row inside the M-tile (A operand)
    int const kg = lane >> 4; // which 8 of a slab's 32 rows this lane holds
    int const K = p.k;               // the rows of K this workgroup covers
    int const KT = p.k_tiles;
    uint32_t const AS = (uint32_t) p.act_stride;    // elements between activation rows
    uint32_t const WS = (uint32_t) p.w_strip_tiles; // tiles between strips
    int const strip0 = group * NS;

    u32x4 const ones = {E::kOnes, E::kOnes, E::kOnes, E::kOnes};
    NibbleConsts const nib = nibble_consts<DT>();
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};

    f32x4 acc_out[NS][MT], acc_p[NS][MT], acc_s[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
    {
        acc_s[mt] = zero4;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc_out[s][mt] = acc_p[s][mt] = zero4;
    }

    // Buffer descriptors: an access past num_records returns 0, which is exactly what rows >= m,
    // the padded tail of K and the scale rows of that tail must contribute - no branches needed.
    constexpr uint32_t kOob = 0x7FFFFFF0u;
    auto const act_rsrc = make_rsrc(p.act, ((uint32_t) (p.m - 1) * AS + (uint32_t) K) * 2u);
    auto const pqs_rsrc = make_rsrc(PQS ? p.pqs : p.act, (uint32_t) K * 2u);
    uint32_t const sz_bytes = (uint32_t) p.scale_rows * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    // weights too go through a descriptor: a prefetch past the last tile row is given an
    // out-of-range offset and costs no memory traffic, so the K loop needs no conditional loads
    auto const w_rsrc = make_rsrc(p.weight, ((uint32_t) (p.strips - 1) * WS + (uint32_t) KT) * 1024u);

    // strips past the end of N (last group only) are clamped for loads and skipped at the store
    bool const gated = ACT && act_is_gated(p.activation);
    int const half_strips = p.strips / 2;
    int strip_of[NS];
    uint32_t wlane[NS]; // byte offset of this lane's 16 bytes in tile row 0 of each strip
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        if (gated)
        {
            int const pair = strip0 / 2 + s / 2; // NS is even: this group's pairs are strip0/2 ..
            strip_of[s] = (pair < half_strips ? pair : half_strips - 1) + (s & 1) * half_strips;
        }
        else
            strip_of[s] = strip0 + s < p.strips ? strip0 + s : p.strips - 1;
        wlane[s] = ((uint32_t) strip_of[s] * WS * 64u + (uint32_t) lane) * 16u;
    }

    // LDS-staged activations: row r of the M-tile at byte r * lds_row; rows >= m read row m-1
    // (their products land in output rows that are never stored)
    uint32_t const lds_row = (uint32_t) KT * TK * 2u + 16u; // +16: rows start in different banks
    int const c_row = SL ? (c & (R - 1)) : c; // row of the M-tile this lane's A fragment belongs to
    int const a_row = c_row < p.m ? c_row : p.m - 1;
    char const* a_lds = reinterpret_cast<char const*>(act_lds) + (uint32_t) a_row * lds_row + (uint32_t) kg * 16u;
    // staged scales: one row of NS*16 values per group of K (rows past the end of K hold zeros),
    // strip slot s at columns s*16 ..; the zeros follow in the same arrangement
    int const act_rows = ALDS ? (p.m < 16 ? p.m : 16) : 0;
    int const sc_rows = SCLDS ? (int) scale_row<GROUP>((uint32_t) (KT * TK - 1), p.group_magic) + 1 : 0;
    constexpr uint32_t SC_ROW = NS * 32u;
    char* const sc_lds = reinterpret_cast<char*>(act_lds) + (uint32_t) act_rows * lds_row;
    char* const zr_lds = sc_lds + (uint32_t) sc_rows * SC_ROW;
    // activation row sums of segment i (SEG rows of K): 16 floats (one per row of the M-tile) at i * 64
    char* const sum_lds = zr_lds + (ZERO ? (uint32_t) sc_rows * SC_ROW : 0u);
    // group slots: 256 bytes of zeros behind the sums - the A fragments of the lanes whose slot is not the
    // current group's, and the scale / zero / sum of slots past the end of K
    char* const zero_lds = sum_lds + (SUMLDS ? (uint32_t) KT * SEGS * 64u : 0u);
    int const n_my = (KT - wave + WAVES - 1) / WAVES; // tile rows of this wavefront: kt = wave + it * WAVES

    auto fetch = [&](Stage& st, int kt)
    {
        uint32_t const tile_off = kt < KT ? (uint32_t) kt * 1024u : 0x80000000u; // scalar select
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            // The non-temporal hint, except in the grouped kernel (ACT): a launch with few active experts on a
            // long K is bound by latency, not bandwidth (two experts' 14336 x 4096 at one token: 20.9 us with
            // ordinary loads, 24.4 with the hint), and an expert with more than sixteen rows reads its weights
            // again; with 1 ... 8 rows in every expert the hint would gain 5-7 % there.
            uint32_t const off = wlane[s] + tile_off;
            st.w[s] = ACT ? buffer_load_x4(w_rsrc, off) : buffer_load_x4_once(w_rsrc, off);
        }
        if constexpr (!ALDS)
        {
#pragma unroll
            for (int j = 0; j < SLABS; ++j)
            {
                int const kk = kt * TK + j * 32 + kg * 8; // this lane's 8 rows of the slab
                bool const k_ok = kk < K;
                if constexpr (PQS)
                    st.sm[j] = buffer_load_x4(pqs_rsrc, (uint32_t) kk * 2u);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                {
                    uint32_t const row = mt * 16 + c;
                    st.a[j][mt]
                        = buffer_load_x4(act_rsrc, k_ok ? (row * AS + (uint32_t) kk) * 2u : kOob);
                }
            }
        }
        if constexpr (GROUP != 0 && !SCLDS)
        {
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                uint32_t const grow = scale_row<GROUP>((uint32_t) (kt * TK + seg * SEG), p.group_magic);
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    uint32_t const off = (grow * (uint32_t) p.n + (uint32_t) (strip_of[s] * 16 + c)) * 2u;
                    st.s[s][seg] = buffer_load_u16(sc_rsrc, off);
                    if constexpr (ZERO)
                        st.z[s][seg] = buffer_load_u16(zr_rsrc, off);
                }
            }
        }
    };

    // Group slots: scales of the SLOTS groups collected in acc_p (window `wnd` of this wavefront's groups).
    // Register r of lane (kg, c) is MFMA row kg*4 + r = slot * R + row: the slot names the group, hence
    // the scale, zero and activation row sum that apply; slots the wavefront never filled read zeros.
    auto flush_slots = [&](int wnd)
    {
        if constexpr (SL)
        {
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                int const i = kg * 4 + r;
                int const gi = wnd * SLOTS + i / R;        // the wavefront's gi-th group
                int const it_i = gi / SEGS, seg_i = gi % SEGS;
                bool const ok = it_i < n_my;
                int const kt_i = wave + it_i * WAVES;
                uint32_t const grow = scale_row<GROUP>((uint32_t) (kt_i * TK + seg_i * SEG), p.group_magic);
                char const* sp = ok ? sc_lds + grow * SC_ROW + (uint32_t) c * 2u : zero_lds;
                char const* zp = ok ? zr_lds + grow * SC_ROW + (uint32_t) c * 2u : zero_lds;
                float const S = *reinterpret_cast<float const*>(
                    ok ? sum_lds + (uint32_t) (kt_i * SEGS + seg_i) * 64u + (uint32_t) (i & (R - 1)) * 4u : zero_lds);
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    float const sc = E::from_bits(*reinterpret_cast<uint16_t const*>(sp + (ok ? s * 32 : 0)));
                    float const zz = ZERO ? E::from_bits(*reinterpret_cast<uint16_t const*>(zp + (ok ? s * 32 : 0))) : 0.f;
                    float const cc = __builtin_fmaf(-OFF, sc, zz);
                    acc_out[s][0][r] = __builtin_fmaf(sc, acc_p[s][0][r], __builtin_fmaf(cc, S, acc_out[s][0][r]));
                }
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
                acc_p[s][0] = zero4;
        }
    };

    auto compute = [&](Stage const& st, int kt, int it)
    {
#pragma unroll
        for (int seg = 0; seg < SEGS; ++seg)
        {
            // group slots: only the lanes of this group's slot read activations, the others zeros
            [[maybe_unused]] char const* a_seg = a_lds;
            if constexpr (SL)
            {
                int const slot = (it * SEGS + seg) & (SLOTS - 1);
                a_seg = (c >> (R == 1 ? 0 : (R == 2 ? 1 : (R == 4 ? 2 : 3)))) == slot
                    ? a_lds + (uint32_t) (kt * TK + seg * SEG) * 2u
                    : zero_lds + (uint32_t) kg * 16u;
            }
#pragma unroll
            for (int js = 0; js < SEG_SLABS; ++js)
            {
                int const j = seg * SEG_SLABS + js;
                u32x4 a[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                {
                    if constexpr (SL)
                        a[mt] = *reinterpret_cast<u32x4 const*>(a_seg + (uint32_t) (js * 32) * 2u);
                    else if constexpr (ALDS)
                        a[mt] = *reinterpret_cast<u32x4 const*>(a_lds + (uint32_t) (kt * TK + j * 32) * 2u);
                    else
                    {
                        a[mt] = st.a[j][mt];
                        if constexpr (PQS)
                        {
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                a[mt][r] = E::mul2(a[mt][r], st.sm[j][r]);
                        }
                    }
                    if constexpr (!SUMLDS)
                        acc_s[mt] = E::mma(a[mt], ones, acc_s[mt]);
                }
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    u32x4 b;
                    if constexpr (BITS == 4)
                        b = expand_int4<DT>(st.w[s][j], nib);
                    else
                        b = expand_int8<DT>(st.w[s][2 * j], st.w[s][2 * j + 1]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc_p[s][mt] = E::mma(a[mt], b, acc_p[s][mt]);
                }
            }
            if constexpr (SL)
            {
                if (((it * SEGS + seg + 1) & (SLOTS - 1)) == 0) // the last slot has been filled
                    flush_slots((it * SEGS + seg) / SLOTS);
            }
            else if constexpr (GROUP != 0)
            {
                // a segment past the end of K carries zero activations, scale 0 and zero 0.
                // Lane (kg, c) register r is output row kg*4 + r: with a single row (decode,
                // m == 1) only r == 0 is ever stored, so the other three are not scaled.
                if constexpr (SUMLDS) // rows kg*4 .. kg*4+3 of this segment's sums
                    acc_s[0] = *reinterpret_cast<f32x4 const*>(sum_lds + (uint32_t) (kt * SEGS + seg) * 64u + kg * 16u);
                auto scale_rows = [&](auto rows_tag)
                {
                    constexpr int ROWS = decltype(rows_tag)::value;
#pragma unroll
                    for (int s = 0; s < NS; ++s)
                    {
                        uint16_t s_raw, z_raw = 0;
                        if constexpr (SCLDS)
                        {
                            uint32_t const at
                                = scale_row<GROUP>((uint32_t) (kt * TK + seg * SEG), p.group_magic) * SC_ROW + (s * 16 + c) * 2u;
                            s_raw = *reinterpret_cast<uint16_t const*>(sc_lds + at);
                            if constexpr (ZERO)
                                z_raw = *reinterpret_cast<uint16_t const*>(zr_lds + at);
                        }
                        else
                        {
                            s_raw = st.s[s][seg];
                            if constexpr (ZERO)
                                z_raw = st.z[s][seg];
                        }
                        float const sc = E::from_bits(s_raw);
                        float const cc = __builtin_fmaf(-OFF, sc, ZERO ? E::from_bits(z_raw) : 0.f);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                        {
#pragma unroll
                            for (int r = 0; r < ROWS; ++r)
                                acc_out[s][mt][r] = __builtin_fmaf(
                                    sc, acc_p[s][mt][r], __builtin_fmaf(cc, acc_s[mt][r], acc_out[s][mt][r]));
                            acc_p[s][mt] = zero4;
                        }
                    }
                };
                if (MT == 1 && p.m == 1)
                    scale_rows(std::integral_constant<int, 1>{});
                else
                    scale_rows(std::integral_constant<int, 4>{});
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc_s[mt] = zero4;
            }
        }
    };

    // tile rows of this wavefront: kt = wave + it * WAVES, it = 0 .. n_my-1 (all scalar).
    // Every load tolerates kt >= KT (returns zeros), so prologue and loop are unconditional and
    // the compiler's wait-count tracking stays exact: compute(st[i]) waits only for its own
    // stage while the PF-1 younger stages stay in flight.  The scheduling barriers keep the
    // compiler from sinking the prefetch below the compute (it would, to save registers).
    auto kt_of = [&](int it) { return wave + it * WAVES; };
    // staging of the group scales / zeros: 16-byte chunks of 8 columns, NS * 2 per group of K
    int const sc_chunks = sc_rows * NS * 2;
    auto sc_offset = [&](int idx, uint32_t& lds_at)
    {
        int const row = idx / (NS * 2), piece = idx - row * (NS * 2); // piece = strip slot * 2 + half
        int strip = strip0 + (piece >> 1);
        if (gated)
        {
            int const pair = strip0 / 2 + (piece >> 2);
            strip = (pair < half_strips ? pair : half_strips - 1) + ((piece >> 1) & 1) * half_strips;
        }
        else if (strip >= p.strips)
            strip = p.strips - 1;
        lds_at = (uint32_t) row * SC_ROW + (uint32_t) piece * 16u;
        return idx < sc_chunks ? ((uint32_t) row * (uint32_t) p.n + (uint32_t) (strip * 16 + (piece & 1) * 8)) * 2u
                               : kOob;
    };
    // chunks past the first 2 * THREADS (long K): a plain loop after the weight prefetch is under way
    auto stage_scales_tail = [&]()
    {
        for (int idx = threadIdx.x + 2 * THREADS; idx < sc_chunks; idx += THREADS)
        {
            uint32_t at;
            uint32_t const off = sc_offset(idx, at);
            *reinterpret_cast<u32x4*>(sc_lds + at) = buffer_load_x4(sc_rsrc, off);
            if constexpr (ZERO)
                *reinterpret_cast<u32x4*>(zr_lds + at) = buffer_load_x4(zr_rsrc, off);
        }
    };
    Stage st[PF];
    if constexpr (!ALDS)
    {
        if constexpr (SCLDS)
        {
            // the staged scales are requested first, the weight and activation prefetch right
            // behind them: loads complete in order, so the barrier waits for the scales only
            uint32_t s_at[2];
            u32x4 sv[2], zv[2];
            [[maybe_unused]] bool const second = sc_chunks > THREADS; // uniform
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                if (u == 1 && !second)
                    continue;
                uint32_t const off = sc_offset(threadIdx.x + u * THREADS, s_at[u]);
                sv[u] = buffer_load_x4(sc_rsrc, off);
                if constexpr (ZERO)
                    zv[u] = buffer_load_x4(zr_rsrc, off);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < P0; ++i)
                fetch(st[i], kt_of(i));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                if (u == 1 && !second)
                    continue;
                if ((int) threadIdx.x + u * THREADS < sc_chunks)
                {
                    *reinterpret_cast<u32x4*>(sc_lds + s_at[u]) = sv[u];
                    if constexpr (ZERO)
                        *reinterpret_cast<u32x4*>(zr_lds + s_at[u]) = zv[u];
                }
            }
            stage_scales_tail();
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = P0; i < PF; ++i)
                fetch(st[i], kt_of(i));
        }
        else
        {
#pragma unroll
            for (int i = 0; i < PF; ++i)
                fetch(st[i], kt_of(i));
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    else
    {
        // Staged operands (activations - smoothed if a pre-quant scale is given - and the group
        // scales / zeros of this workgroup's columns) are requested FIRST, the weight prefetch
        // right behind them: loads complete in order, so the LDS writes and the barrier wait for
        // the small staged loads only while the weights stay in flight.  Each thread holds up to
        // UA + 2 staged chunks in registers across the prefetch (the third and fourth only when the
        // activations are that long: a load issued after the weight prefetch completes after it, so
        // the barrier would wait a whole HBM round trip for it); anything beyond that (long K, many
        // rows) is staged by a plain loop after it.
        constexpr int UA = 4;
        int const chunks_per_row = KT * TK / 8; // 16-byte chunks, including the zero-filled tail of K
        int const act_chunks = act_rows * chunks_per_row;
        auto act_offset = [&](int idx, uint32_t& lds_at, uint32_t& ch, uint32_t& sum_at)
        {
            int const row = act_rows == 1 ? 0 : idx / chunks_per_row;
            ch = (uint32_t) (idx - row * chunks_per_row);
            lds_at = (uint32_t) row * lds_row + ch * 16u;
            sum_at = ch / (SEG / 8) * 64u + (uint32_t) row * 4u;
            bool const ok = idx < act_chunks && (int) ch * 8 < K;
            return ok ? ((uint32_t) row * AS + ch * 8u) * 2u : kOob;
        };
        auto smooth = [&](u32x4 v, u32x4 sm)
        {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[r] = E::mul2(v[r], sm[r]);
            return v;
        };
        // Sum of the SEG activations of one segment: the SEG/8 consecutive lanes that hold its
        // chunks add their eight values each and combine across lanes; every lane of a 16-lane
        // row is active here (rows of lanes enter or leave the staging loops together).
        auto stage_sum = [&](u32x4 v, int idx, uint32_t sum_at)
        {
            float t = 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                t += E::from_bits((uint16_t) (v[r] & 0xFFFFu)) + E::from_bits((uint16_t) (v[r] >> 16));
            t = dpp_add<0xB1>(t);  // quad_perm [1,0,3,2]
            t = dpp_add<0x4E>(t);  // quad_perm [2,3,0,1]
            t = dpp_add<0x141>(t); // row_half_mirror
            if constexpr (SEG == 128)
                t = dpp_add<0x140>(t); // row_mirror
            if ((threadIdx.x & (SEG / 8 - 1)) == 0 && idx < act_chunks)
                *reinterpret_cast<float*>(sum_lds + sum_at) = t;
        };

        u32x4 av[UA], pv[UA], sv[2], zv[2];
        uint32_t a_at[UA], sum_at[UA], s_at[2] = {0, 0};
        [[maybe_unused]] bool const second = sc_chunks > THREADS; // uniform
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            if (u >= 2 && u * THREADS >= act_chunks) // uniform
                continue;
            uint32_t ch;
            av[u] = buffer_load_x4(act_rsrc, act_offset(threadIdx.x + u * THREADS, a_at[u], ch, sum_at[u]));
            if constexpr (PQS)
                pv[u] = buffer_load_x4(pqs_rsrc, ch * 16u);
        }
        if constexpr (SCLDS)
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                if (u == 1 && !second)
                    continue;
                uint32_t const off = sc_offset(threadIdx.x + u * THREADS, s_at[u]);
                sv[u] = buffer_load_x4(sc_rsrc, off);
                if constexpr (ZERO)
                    zv[u] = buffer_load_x4(zr_rsrc, off);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < P0; ++i)
            fetch(st[i], kt_of(i));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UA; ++u)
        {
            if (u >= 2 && u * THREADS >= act_chunks) // uniform
                continue;
            u32x4 const v = PQS ? smooth(av[u], pv[u]) : av[u];
            if ((int) threadIdx.x + u * THREADS < act_chunks)
                *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(act_lds) + a_at[u]) = v;
            if constexpr (SUMLDS)
                stage_sum(v, threadIdx.x + u * THREADS, sum_at[u]);
        }
        if constexpr (SCLDS)
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                if (u == 1 && !second)
                    continue;
                if ((int) threadIdx.x + u * THREADS < sc_chunks)
                {
                    *reinterpret_cast<u32x4*>(sc_lds + s_at[u]) = sv[u];
                    if constexpr (ZERO)
                        *reinterpret_cast<u32x4*>(zr_lds + s_at[u]) = zv[u];
                }
            }
        }
        // (four requests at a time, so that their round trips overlap)
        for (int base = UA * THREADS; base < act_chunks; base += UA * THREADS)
        {
            u32x4 tv[UA], tp[UA];
            uint32_t t_at[UA], t_sum[UA];
#pragma unroll
            for (int u = 0; u < UA; ++u)
            {
                if (base + u * THREADS >= act_chunks) // uniform
                    continue;
                uint32_t ch;
                tv[u] = buffer_load_x4(act_rsrc, act_offset(base + u * THREADS + threadIdx.x, t_at[u], ch, t_sum[u]));
                if constexpr (PQS)
                    tp[u] = buffer_load_x4(pqs_rsrc, ch * 16u);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < UA; ++u)
            {
                if (base + u * THREADS >= act_chunks) // uniform
                    continue;
                int const idx = base + u * THREADS + threadIdx.x;
                u32x4 const v = PQS ? smooth(tv[u], tp[u]) : tv[u];
                if (idx < act_chunks)
                    *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(act_lds) + t_at[u]) = v;
                if constexpr (SUMLDS)
                    stage_sum(v, idx, t_sum[u]);
            }
        }
        if constexpr (SCLDS)
            stage_scales_tail();
        if constexpr (SL)
        {
            if (threadIdx.x < 16)
                *reinterpret_cast<u32x4*>(zero_lds + threadIdx.x * 16u) = u32x4{0u, 0u, 0u, 0u};
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = P0; i < PF; ++i)
            fetch(st[i], kt_of(i));
        __builtin_amdgcn_sched_barrier(0);
    }

    for (int it = 0; it < n_my; it += PF)
    {
#pragma unroll
        for (int i = 0; i < PF; ++i)
        {
            if (it + i < n_my)
                compute(st[i], kt_of(it + i), it + i);
            __builtin_amdgcn_sched_barrier(0);
            fetch(st[i], kt_of(it + i + PF));
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    if constexpr (SL)
    {
        if ((n_my * SEGS) & (SLOTS - 1)) // a last, partly filled window
            flush_slots(n_my * SEGS / SLOTS);
    }
    if constexpr (GROUP == 0)
    {
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            int const col = strip_of[s] * 16 + c;
            float const sc = E::load(p.scales, col);
            float const cc = (ZERO ? E::load(p.zeros, col) : 0.f) - OFF * sc;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc_out[s][mt][r] = __builtin_fmaf(sc, acc_p[s][mt][r], cc * acc_s[mt][r]);
        }
    }

    // ---- cross-wavefront reduction (fixed order) and epilogue -------------------------------
    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    if constexpr (SL)
    {
        // Row `row` of the M-tile is spread over the SLOTS MFMA rows slot * R + row, i.e. over the lane's
        // registers (R < 4) and the lanes kg: folded here in a fixed order, then across wavefronts.
        constexpr int RL = R < 4 ? R : 4; // distinct rows of the M-tile per lane
        __shared__ float red_sl[WAVES][NS][R][16];
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            float v[RL];
            if constexpr (R == 1)
                v[0] = (acc_out[s][0][0] + acc_out[s][0][1]) + (acc_out[s][0][2] + acc_out[s][0][3]);
            else if constexpr (R == 2)
            {
                v[0] = acc_out[s][0][0] + acc_out[s][0][2];
                v[1] = acc_out[s][0][1] + acc_out[s][0][3];
            }
            else
            {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    v[r] = acc_out[s][0][r];
            }
#pragma unroll
            for (int r = 0; r < RL; ++r)
            {
                if constexpr (R <= 4)
                    v[r] += __shfl_xor(v[r], 16);
                v[r] += __shfl_xor(v[r], 32);
                int const row = R <= 4 ? r : (kg & 1) * 4 + r;
                if ((R <= 4 ? kg == 0 : kg < 2) && row < p.m)
                    red_sl[wave][s][row][c] = v[r];
            }
        }
        __syncthreads();
        for (int e = threadIdx.x; e < NS * R * 16; e += WAVES * 64)
        {
            int const s = e / (R * 16), row = (e >> 4) & (R - 1), cc = e & 15;
            if (row >= p.m || strip0 + s >= p.strips)
                continue;
            float sum = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < WAVES; ++w2)
                sum += red_sl[w2][s][row][cc];
            int const ocol = (strip0 + s) * 16 + cc;
            if (p.partial)
            {
                p.partial[(size_t) row * p.n + ocol] = sum; // this K slice's share; the finish pass adds alpha, bias
                continue;
            }
            float v = p.alpha * sum;
            if (p.bias)
                v += E::load(p.bias, ocol);
            out16[(size_t) row * p.n + ocol] = E::store(v);
        }
    }
    else
    {
    constexpr int SLOTS_ = NS * MT * 4;
    __shared__ float red[WAVES][SLOTS_][64];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (mt * 16 + kg * 4 + r < p.m)
                    red[wave][(s * MT + mt) * 4 + r][lane] = acc_out[s][mt][r];
    __syncthreads();

    if (gated)
    {
        // value and gate sums sit in neighbouring strip slots: out = (x + bias_x) * f(g + bias_g)
        if constexpr (ACT && NS % 2 == 0)
        {
            int const n_out = p.n / 2;
            for (int e = threadIdx.x; e < SLOTS_ / 2 * 64; e += WAVES * 64)
            {
                int const pslot = e >> 6, ln = e & 63; // (pair, mt, r)
                int const ps = pslot / (MT * 4), mt = (pslot >> 2) % MT, r = pslot & 3;
                int const row = mt * 16 + (ln >> 4) * 4 + r;
                int const pair = strip0 / 2 + ps;
                if (row >= p.m || pair >= half_strips)
                    continue;
                int const slot_x = ((2 * ps) * MT + mt) * 4 + r, slot_g = ((2 * ps + 1) * MT + mt) * 4 + r;
                float x = 0.f, g = 0.f;
#pragma unroll
                for (int w2 = 0; w2 < WAVES; ++w2)
                {
                    x += red[w2][slot_x][ln];
                    g += red[w2][slot_g][ln];
                }
                int const ocol = pair * 16 + (ln & 15);
                if (p.bias)
                {
                    x += E::load(p.bias, ocol);
                    g += E::load(p.bias, ocol + n_out);
                }
                float v = x * apply_act(p.activation, g);
                if (p.residual)
                    v += E::load(p.residual, (size_t) row * n_out + ocol);
                out16[(size_t) row * n_out + ocol] = E::store(v);
            }
        }
        return;
    }
    for (int e = threadIdx.x; e < SLOTS_ * 64; e += WAVES * 64)
    {
        int const slot = e >> 6, ln = e & 63;
        int const s = slot / (MT * 4), mt = (slot >> 2) % MT, r = slot & 3;
        int const row = mt * 16 + (ln >> 4) * 4 + r;
        if (row >= p.m || strip0 + s >= p.strips)
            continue;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][slot][ln];
        int const ocol = (strip0 + s) * 16 + (ln & 15);
        if (!ACT && p.partial)
        {
            p.partial[(size_t) row * p.n + ocol] = sum; // this K slice's share; the finish pass adds alpha, bias
            continue;
        }
        float v = p.alpha * sum;
        if (p.bias)
            v += E::load(p.bias, ocol);
        if constexpr (ACT)
        {
            v = apply_act(p.activation, v);
            if (p.residual)
                v += E::load(p.residual, (size_t) row * p.n + ocol);
        }
        out16[(size_t) row * p.n + ocol] = E::store(v);
    }
    } // !SL
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int MT, int NS, int WAVES, int PF, int LDS, int SLOTS = 1>
__global__ void __launch_bounds__(WAVES * 64) stream_kernel(StreamParams p)
{
    if (p.k_slices > 1)
    {
        // K split across workgroups: this workgroup's slice becomes the whole problem
        constexpr int TK = BITS == 4 ? 128 : 64;
        int const y = (int) blockIdx.y;
        int const kt0 = y * p.slice_tiles;
        size_t const k0 = (size_t) kt0 * TK;
        p.act = static_cast<char const*>(p.act) + k0 * 2;
        if (PQS)
            p.pqs = static_cast<char const*>(p.pqs) + k0 * 2;
        p.weight = static_cast<char const*>(p.weight) + (size_t) kt0 * 1024;
        if (GROUP != 0)
        {
            size_t const srow = k0 / (GROUP != 0 ? GROUP : 1) * (size_t) p.n * 2;
            p.scales = static_cast<char const*>(p.scales) + srow;
            if (ZERO)
                p.zeros = static_cast<char const*>(p.zeros) + srow;
        }
        if (GROUP != 0)
            p.scale_rows -= (int) (k0 / (GROUP != 0 ? GROUP : 1));
        int const k_left = p.k_total - (int) k0;
        p.k = k_left < p.slice_tiles * TK ? k_left : p.slice_tiles * TK;
        p.k_tiles = (p.k + TK - 1) / TK;
        p.partial += (size_t) y * (size_t) p.m * (size_t) p.n;
    }
    stream_body<DT, BITS, GROUP, PQS, ZERO, MT, NS, WAVES, PF, LDS, false, SLOTS>(p);
}

// Grouped problems: workgroup (x, e) is workgroup x of expert e's own matmul.  The parameters are
// narrowed to that expert's operands and rows; an expert with more than 16 rows streams its
// weights once per 16 rows (this kernel is chosen when that is rare).
template <int DT, int BITS, int GROUP, bool ZERO, int NS, int WAVES, int PF, int LDS>
__global__ void __launch_bounds__(WAVES * 64) stream_grouped_kernel(StreamParams p)
{
    int const e = (int) blockIdx.y;
    int64_t begin = 0;
    int rows_left = p.m; // no prefix sums: one expert owns every row
    if (p.expert_rows)
    {
        begin = e ? p.expert_rows[e - 1] : 0;
        rows_left = __builtin_amdgcn_readfirstlane((int) (p.expert_rows[e] - begin));
    }
    p.act = uniform_ptr(static_cast<char const*>(p.act) + (size_t) begin * (size_t) p.k * 2);
    int const n_out = act_is_gated(p.activation) ? p.n / 2 : p.n;
    p.out = uniform_ptr(static_cast<char*>(p.out) + (size_t) begin * (size_t) n_out * 2);
    if (p.residual)
        p.residual = uniform_ptr(static_cast<char const*>(p.residual) + (size_t) begin * (size_t) n_out * 2);
    p.weight = uniform_ptr(static_cast<char const*>(p.weight) + (size_t) e * p.weight_stride);
    p.scales = uniform_ptr(static_cast<char const*>(p.scales) + (size_t) e * p.scale_stride);
    if (ZERO)
        p.zeros = uniform_ptr(static_cast<char const*>(p.zeros) + (size_t) e * p.scale_stride);
    if (p.bias)
        p.bias = uniform_ptr(static_cast<char const*>(p.bias) + (size_t) e * (size_t) p.n * 2);
    for (; rows_left > 0; rows_left -= 16)
    {
        p.m = rows_left;
        stream_body<DT, BITS, GROUP, false, ZERO, 1, NS, WAVES, PF, LDS, true>(p);
        __syncthreads(); // this pass is done with the LDS areas
        p.act = static_cast<char const*>(p.act) + (size_t) 16 * (size_t) p.k * 2;
        p.out = static_cast<char*>(p.out) + (size_t) 16 * (size_t) n_out * 2;
        if (p.residual)
            p.residual = static_cast<char const*>(p.residual) + (size_t) 16 * (size_t) n_out * 2;
    }
}

// launch shape: NS strips per wavefront, WAVES wavefronts per workgroup, PF tile rows in flight,
// lds = 1: activations, group scales / zeros and activation row sums staged in LDS; lds = 2: only
// the group scales / zeros (activations in registers); lds = 0: nothing staged
struct StreamShape
{
    int ns, waves, pf, lds;
};

// bytes of LDS the staged activations of an m x k problem take (tile_k = 128 int4 / 64 int8)
inline size_t stream_act_lds_bytes(int m, int k, int tile_k)
{
    int const rows = m < 16 ? m : 16;
    return (size_t) rows * ((size_t) ((k + tile_k - 1) / tile_k) * tile_k * 2 + 16);
}

// bytes of LDS the staged group scales (and zeros) of ns strips and, with sums, the activation row
// sums take
// (`group`: the kernel instantiation's, `real_group`: the problem's - they differ for flexible groups)
inline size_t stream_scale_lds_bytes(int k, int tile_k, int group, int real_group, int ns, bool zeros, bool sums)
{
    if (group == 0)
        return 0;
    size_t const k_padded = (size_t) ((k + tile_k - 1) / tile_k) * tile_k;
    size_t const seg = group > tile_k ? tile_k : group; // rows of K per activation row sum
    return (k_padded + real_group - 1) / real_group * (size_t) ns * 32 * (zeros ? 2 : 1) + (sums ? k_padded / seg * 64 : 0);
}


// WOQ_STREAM_SHAPE="ns,waves,pf,lds" overrides the heuristic (for tuning sweeps)
StreamShape pick_stream_shape(int mt, int m, int k, int strips, int k_tiles, int tile_k, int group,
    int const* split_shape = nullptr, bool three_strips = true);
// WOQ_STREAM_SLOTS=0 switches the group-slot variants off (for A/B timing)
bool stream_slots_disabled();
// K slices (1 = none) of a streaming launch with `workspace_bytes` of scratch; WOQ_STREAM_SPLITS overrides
// (shape[0] != 0: the launch shape that goes with the split)
int pick_stream_k_slices(int m, int n, int k, int tile_k, int group, size_t workspace_bytes, int shape[4]);

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO, int MT, int NS, int WAVES, int PF, int LDS,
    bool GROUPED = false, int SLOTS = 1>
int launch_stream_variant(StreamParams sp, hipStream_t stream)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    auto kernel = [] {
        if constexpr (GROUPED)
            return stream_grouped_kernel<DT, BITS, GROUP, ZERO, NS, WAVES, PF, LDS>;
        else
            return stream_kernel<DT, BITS, GROUP, PQS, ZERO, MT, NS, WAVES, PF, LDS, SLOTS>;
    }();
    size_t lds = 0;
    if constexpr (LDS != 0)
    {
        lds = (LDS == 1 ? stream_act_lds_bytes(sp.m, sp.k, TK) : 0) + stream_scale_lds_bytes(sp.k, TK, host_group_rows(GROUP), sp.real_group, NS, ZERO, LDS == 1)
            + (SLOTS > 1 ? 256 : 0); // group slots: a block of zeros behind the staged operands
        // the reduction buffer of the epilogue is static LDS of this variant and shares the CU's 160 KiB
        constexpr size_t kStaticLds = (size_t) WAVES * NS * MT * 4 * 64 * sizeof(float);
        constexpr size_t kMaxDynamic = stream_max_staged_lds(NS * MT, WAVES);
        static_assert(kStaticLds + kMaxDynamic <= 160 * 1024, "LDS of one CU");
        if (lds > kMaxDynamic)
            return fail(WOQ_ERR_UNSUPPORTED, "staged operands of %zu bytes do not fit the LDS staging area", lds);
        static std::atomic<uint64_t> raised{0}; // one bit per device
        if (lds > 32 * 1024)
            if (int rc = raise_lds_once(raised, reinterpret_cast<void const*>(kernel), (int) kMaxDynamic))
                return rc;
    }
    sp.groups = (sp.strips + NS - 1) / NS;
    sp.groups_per_xcd = (sp.groups + 7) / 8;
    dim3 grid(sp.groups_per_xcd * 8, GROUPED ? sp.num_experts : sp.k_slices), block(WAVES * 64);
    note_launch(GROUPED ? "stream grouped mt=%d ns=%d waves=%d pf=%d slots=%d experts=%d"
                        : "stream mt=%d ns=%d waves=%d pf=%d slots=%d k_slices=%d",
        MT, NS, WAVES, PF, SLOTS, GROUPED ? sp.num_experts : sp.k_slices);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, sp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "stream kernel launch failed: %s", hipGetErrorString(err));
    if (!GROUPED && sp.k_slices > 1)
    {
        // out = T(alpha * (slab 0 + slab 1 + ...) + bias), in slice order
        size_t const count = (size_t) sp.m * (size_t) sp.n;
        hipLaunchKernelGGL((gemm_finish_partial<DT>), dim3((unsigned) ((count / 4 + 255) / 256)), dim3(256), 0, stream,
            sp.out, sp.partial, sp.bias, sp.alpha, sp.m, sp.n, sp.k_slices);
        err = hipGetLastError();
        if (err != hipSuccess)
            return fail(WOQ_ERR_RUNTIME, "split-K finish launch failed: %s", hipGetErrorString(err));
    }
    return WOQ_OK;
}

template <int DT, int BITS, int GROUP, bool PQS, bool ZERO>
int launch_stream_shaped(StreamParams const& sp, int mt, hipStream_t s)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    StreamShape sh = pick_stream_shape(mt, sp.m, sp.k, sp.strips, sp.k_tiles, TK, host_group_rows(GROUP), sp.split_shape);
    if (GROUP == 0 && sh.lds == 2)
        sh.lds = 0; // per-channel scales are applied once, in the epilogue: nothing to stage
#define WOQ_SHAPE(MT_, NS_, WAVES_, PF_, LDS_)                                                                         \
    if (mt == MT_ && sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_ && sh.lds == LDS_)                             \
        return launch_stream_variant<DT, BITS, GROUP, PQS, ZERO, MT_, NS_, WAVES_, PF_, LDS_>(sp, s);
    // decode of a single row with staged activations and group scales: 16 groups of K share the MFMA
    // rows and the scales are applied once per 16 groups (the launch shapes the built-in rule picks)
    if constexpr (GROUP != 0)
    {
#define WOQ_SLOT_SHAPE(NS_, WAVES_, PF_)                                                                               \
    if (mt == 1 && sp.m == 1 && sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_ && sh.lds == 1 && slots_ok)          \
        return launch_stream_variant<DT, BITS, GROUP, PQS, ZERO, 1, NS_, WAVES_, PF_, 1, false, 16>(sp, s);
        bool const slots_ok = !stream_slots_disabled();
        WOQ_SLOT_SHAPE(1, 8, 4)
        WOQ_SLOT_SHAPE(2, 8, 4)
        WOQ_SLOT_SHAPE(3, 8, 2)
        WOQ_SLOT_SHAPE(4, 8, 2)
#undef WOQ_SLOT_SHAPE
    }
    // decode (M <= 16), activations in LDS
    WOQ_SHAPE(1, 1, 8, 4, 1)
    WOQ_SHAPE(1, 1, 8, 6, 1)
    WOQ_SHAPE(1, 1, 16, 4, 1)
    WOQ_SHAPE(1, 2, 8, 4, 1)
    WOQ_SHAPE(1, 2, 4, 4, 1)
    WOQ_SHAPE(1, 3, 8, 2, 1)
    WOQ_SHAPE(1, 4, 4, 2, 1)
    WOQ_SHAPE(1, 4, 4, 4, 1)
    WOQ_SHAPE(1, 4, 8, 2, 1)
    WOQ_SHAPE(1, 4, 8, 4, 1)
    // decode, activations in registers (M x K too large for LDS)
    WOQ_SHAPE(1, 1, 8, 4, 0)
    WOQ_SHAPE(1, 2, 8, 2, 0)
    WOQ_SHAPE(1, 4, 4, 2, 0)
    if constexpr (GROUP != 0)
    {
        // decode, activations in registers, group scales / zeros in LDS
        WOQ_SHAPE(1, 1, 8, 4, 2)
        WOQ_SHAPE(1, 2, 8, 2, 2)
        WOQ_SHAPE(1, 4, 4, 2, 2)
    }
    // skinny M
    WOQ_SHAPE(2, 2, 8, 2, 0)
    WOQ_SHAPE(2, 1, 8, 2, 0)
    WOQ_SHAPE(4, 1, 8, 1, 0)
    WOQ_SHAPE(4, 2, 8, 1, 0)
    WOQ_SHAPE(8, 1, 4, 1, 0)
    WOQ_SHAPE(8, 1, 8, 1, 0)
    if constexpr (GROUP != 0)
    {
        // skinny M, group scales / zeros in LDS
        WOQ_SHAPE(2, 2, 8, 2, 2)
        WOQ_SHAPE(2, 1, 8, 2, 2)
        WOQ_SHAPE(4, 1, 8, 1, 2)
        WOQ_SHAPE(4, 2, 8, 1, 2)
    }
#undef WOQ_SHAPE
    return fail(WOQ_ERR_UNSUPPORTED, "stream shape mt=%d ns=%d waves=%d pf=%d lds=%d is not instantiated", mt, sh.ns,
        sh.waves, sh.pf, sh.lds);
}

// grouped problems: the launch shapes the table picks for one 16-row tile
template <int DT, int BITS, int GROUP, bool ZERO>
int launch_stream_grouped(StreamParams const& sp, hipStream_t s)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    // every expert's column groups run side by side: the grid is num_experts times taller
    StreamShape sh = pick_stream_shape(1, sp.m < 16 ? sp.m : 16, sp.k, sp.strips * sp.num_experts, sp.k_tiles, TK, host_group_rows(GROUP), nullptr,
        /*three_strips=*/false); // the grouped kernel comes with one, two or four strips per wavefront
    if (act_is_gated(sp.activation) && sh.ns == 1) // value and gate strips pair up inside a wavefront
        sh = sh.lds == 1 ? StreamShape{2, 8, 4, 1} : StreamShape{2, 8, 2, sh.lds};
    if (GROUP == 0 && sh.lds == 2)
        sh.lds = 0;
#define WOQ_SHAPE(NS_, WAVES_, PF_, LDS_)                                                                              \
    if (sh.ns == NS_ && sh.waves == WAVES_ && sh.pf == PF_ && sh.lds == LDS_)                                          \
        return launch_stream_variant<DT, BITS, GROUP, false, ZERO, 1, NS_, WAVES_, PF_, LDS_, true>(sp, s);
    WOQ_SHAPE(1, 8, 4, 1)
    WOQ_SHAPE(2, 8, 4, 1)
    WOQ_SHAPE(4, 8, 2, 1)
    WOQ_SHAPE(1, 8, 4, 0)
    WOQ_SHAPE(2, 8, 2, 0)
    WOQ_SHAPE(4, 4, 2, 0)
    if constexpr (GROUP != 0)
    {
        WOQ_SHAPE(1, 8, 4, 2)
        WOQ_SHAPE(2, 8, 2, 2)
        WOQ_SHAPE(4, 4, 2, 2)
    }
#undef WOQ_SHAPE
    return fail(WOQ_ERR_UNSUPPORTED, "grouped stream shape ns=%d waves=%d pf=%d lds=%d is not instantiated", sh.ns,
        sh.waves, sh.pf, sh.lds);
}

template <int DT, int BITS>
bool try_launch_stream_wide(MatmulProblem const& p, StreamParams const& sp, hipStream_t s, int& rc);

// the single-row kernel (stream_row.hip) and the rule that picks it and its launch shape (api.cpp)
int launch_stream_row(StreamParams const& sp, int dtype, int group, bool pqs, bool zero, int waves, int tpw, void* stream);
bool pick_row_shape(int m, int n, int k, int group, int bits, int& waves, int& tiles);
// the multi-row kernel without a staging pass (stream_rows_kernel.h) and its rule (api.cpp)
int launch_stream_rows_int4(StreamParams const& sp, int dtype, int group, bool zero, int waves, int ns, int tpw, void* stream);
int launch_stream_rows_int8(StreamParams const& sp, int dtype, int group, bool zero, int waves, int ns, int tpw, void* stream);
bool pick_rows_shape(int m, int n, int k, int group, int bits, bool pqs, int& waves, int& ns, int& tiles);

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
    sp.act_stride = p.k;
    sp.w_strip_tiles = sp.k_tiles;
    sp.k_total = p.k;
    sp.scale_rows = p.group_size ? (p.k + p.group_size - 1) / p.group_size : 1;
    sp.group_magic = scale_row_magic(p.group_size);
    sp.real_group = p.group_size;
    sp.strips = p.n / kTileN;
    sp.groups = sp.groups_per_xcd = 0;
    sp.expert_rows = p.expert_rows;
    sp.num_experts = p.num_experts;
    sp.weight_stride = p.weight_stride;
    sp.scale_stride = p.scale_stride;
    sp.activation = p.activation;
    sp.residual = p.residual;
    auto s = static_cast<hipStream_t>(stream);
    int const mt = p.m <= 16 ? 1 : (p.m <= 32 ? 2 : (p.m <= 64 ? 4 : 8));
    bool const pqs = p.pre_quant_scale != nullptr;
    bool const zero = p.zeros != nullptr;
    if (mt == 1 && !p.num_experts)
    {
        int waves = 0, tiles = 0;
        if (pick_row_shape(p.m, p.n, p.k, p.group_size, BITS, waves, tiles))
        {
            int const rc = launch_stream_row(sp, DT, p.group_size, pqs, zero, waves, tiles, stream);
            if (rc != WOQ_ERR_UNSUPPORTED)
                return rc;
        }
        int ns = 0;
        if (pick_rows_shape(p.m, p.n, p.k, p.group_size, BITS, pqs, waves, ns, tiles))
        {
            int const rc = BITS == 4 ? launch_stream_rows_int4(sp, DT, p.group_size, zero, waves, ns, tiles, stream)
                                     : launch_stream_rows_int8(sp, DT, p.group_size, zero, waves, ns, tiles, stream);
            if (rc != WOQ_ERR_UNSUPPORTED)
                return rc;
        }
    }
    if (mt == 1)
    {
        // wide matrices at decode: the kernel whose wavefronts own whole columns, where the rule picks it
        int rc = WOQ_OK;
        if (try_launch_stream_wide<DT, BITS>(p, sp, s, rc) && rc != WOQ_ERR_UNSUPPORTED)
            return rc;
    }
    if (!p.num_experts && p.group_size <= 128)
    {
        // long K and few columns: split K across workgroups (float32 slabs in the workspace + finish pass)
        int split_shape[4];
        int const slices = pick_stream_k_slices(p.m, p.n, p.k, TK, p.group_size, p.workspace_bytes, split_shape);
        if (slices > 1 && p.workspace)
        {
            sp.slice_tiles = (sp.k_tiles + slices - 1) / slices;
            if (p.group_size > TK) // a slice starts on a group boundary
                sp.slice_tiles = (sp.slice_tiles + p.group_size / TK - 1) / (p.group_size / TK) * (p.group_size / TK);
            sp.k_slices = (sp.k_tiles + sp.slice_tiles - 1) / sp.slice_tiles;
            if (sp.k_slices > 1)
            {
                sp.k_tiles = sp.slice_tiles; // the largest slice: what the launch shape and the LDS areas go by
                sp.k = sp.slice_tiles * TK;
                sp.partial = static_cast<float*>(p.workspace);
                for (int i = 0; i < 4; ++i)
                    sp.split_shape[i] = split_shape[i];
            }
            else
                sp.k_slices = 1;
        }
    }
    if (p.num_experts)
    {
        switch (template_group(p.group_size))
        {
        case 0: return launch_stream_grouped<DT, BITS, 0, false>(sp, s);
        case 64:
            return zero ? launch_stream_grouped<DT, BITS, 64, true>(sp, s)
                        : launch_stream_grouped<DT, BITS, 64, false>(sp, s);
        case 128:
            return zero ? launch_stream_grouped<DT, BITS, 128, true>(sp, s)
                        : launch_stream_grouped<DT, BITS, 128, false>(sp, s);
        case kFlexGroup:
            return zero ? launch_stream_grouped<DT, BITS, kFlexGroup, true>(sp, s)
                        : launch_stream_grouped<DT, BITS, kFlexGroup, false>(sp, s);
        default: return fail(WOQ_ERR_UNSUPPORTED, "group_size %d", p.group_size);
        }
    }

#define WOQ_STREAM_PQS(G)                                                                                              \
    if (pqs)                                                                                                           \
        return zero ? launch_stream_shaped<DT, BITS, G, true, true>(sp, mt, s)                                         \
                    : launch_stream_shaped<DT, BITS, G, true, false>(sp, mt, s);                                       \
    return zero ? launch_stream_shaped<DT, BITS, G, false, true>(sp, mt, s)                                            \
                : launch_stream_shaped<DT, BITS, G, false, false>(sp, mt, s);
    switch (template_group(p.group_size))
    {
    case 0:
        if (pqs)
            return launch_stream_shaped<DT, BITS, 0, true, false>(sp, mt, s);
        return launch_stream_shaped<DT, BITS, 0, false, false>(sp, mt, s);
    case 64: WOQ_STREAM_PQS(64)
    case 128: WOQ_STREAM_PQS(128)
    case kFlexGroup: WOQ_STREAM_PQS(kFlexGroup)
    default: return fail(WOQ_ERR_UNSUPPORTED, "group_size %d", p.group_size);
    }
#undef WOQ_STREAM_PQS
}

} // namespace woq
