// Skinny-M GEMM: the rows-in-the-tens-to-hundreds regime between the streaming GEMV kernel and
// the 256-row prefill GEMM (the reference covers it with CUTLASS tiles of 16..64 rows and split-K,
// cpp/tensorrt_llm/kernels/cutlass_kernels/cutlass_heuristic.cpp:59-140).
//
// Here the work per weight byte is too small to pay for an exact dequantize of every weight (one
// conversion per weight and only a few MFMAs to amortise it), so the kernel uses the streaming
// kernel's arithmetic on a GEMM skeleton:
//   * the packed integers are expanded to the activation type by one bit operation per pair
//     (value q + OFFSET, exact) and multiplied as they are; per scale group the matrix core
//     produces P = sum a * (q + OFFSET) and, against an all-ones operand, S = sum a (the row sums
//     are the same for every wavefront of the workgroup: with group scales each (group, row
//     tile) is summed by ONE wavefront, a step ahead, and shared through LDS);
//   * the scale is applied to the float32 sums, once per group and output element:
//     acc += s * P + (z - OFFSET * s) * S.
// Output tile 64 (32 for M <= 32, int4) rows x 256 columns; 8 wavefronts side by side along N,
// each 32 columns wide, two per SIMD.  Everything a step needs is requested DEPTH steps ahead: the activation
// tile and the group scales go global -> LDS by DMA, packed weights go straight to the registers
// of the lane that feeds them to the matrix core.
#pragma once

#include <type_traits>

#include "gemm_common.h"

namespace woq
{

constexpr int kSkinnyBN = 256;
constexpr int kSkinnyWaves = 8; // two per SIMD: while one waits at the barrier or for LDS the other issues

template <int DT, int BITS, int GROUP, bool ZERO, int RT, bool SPLITK, int DEPTH = (BITS == 4 ? 3 : 5)>
__global__ void __launch_bounds__(kSkinnyWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) skinny_kernel(GemmParams p)
{
    using E = Elem<DT>;
    constexpr int TK = BITS == 4 ? 128 : 64;
    constexpr int SLABS = TK / 32;
    constexpr int kSkinnyBM = RT * 16;                           // RT row tiles per wavefront
    constexpr int NS = kSkinnyBN / 16 / kSkinnyWaves;            // strips (16 columns) per wavefront
    constexpr int SEG = segment_rows<GROUP, TK>(); // rows sharing one scale inside a tile row
    constexpr int SEGS = TK / SEG;
    constexpr int SEG_SLABS = SEG / 32;
    constexpr int A_BYTES = kSkinnyBM * TK * 2;
    constexpr float OFF = Offset<DT, BITS>::value;

    constexpr int SC_SLOTS = GROUP != 0 ? SEGS * (ZERO ? 2 : 1) : 0; // 256-byte scale slots per wavefront and step

    // One LDS object per step in flight.  They are separate variables on purpose: the compiler
    // orders an LDS read after the DMA writes to the SAME variable only, so reading step kt's
    // buffer does not wait for the DMA just issued into another one.
    // (The A tile and the scale slots of a step are separate objects too: the row sums of step kt+1
    // are formed from its A tile while its scales are still in flight.)
    struct StageA
    {
        u32x4 a[A_BYTES / 16];
    };
    struct StageSc
    {
        u32x4 sc[kSkinnyWaves][(SC_SLOTS ? SC_SLOTS : 1) * 16];
    };
    static_assert(DEPTH + 1 <= 7, "seven stage buffers are declared");
    __shared__ StageA lda0, lda1, lda2, lda3, lda4, lda5, lda6;
    __shared__ StageSc ldc0, ldc1, ldc2, ldc3, ldc4, ldc5, ldc6;
    StageA* const stage_a[7] = {&lda0, &lda1, &lda2, &lda3, &lda4, &lda5, &lda6};
    StageSc* const stage_sc[7] = {&ldc0, &ldc1, &ldc2, &ldc3, &ldc4, &ldc5, &ldc6};
    // row sums S of the activations: per step slot, (group of the step, row tile), 16 rows.
    // (Spreading the work over all eight wavefronts - two slabs each, partial sums added by the
    // readers - measured slower than leaving it to SEGS * RT of them.)
    // Per-channel scales need only the sums over the whole of K: every wavefront sums its share of
    // each step's A fragments and the shares are added once, in the epilogue.
    constexpr int SUM_UNITS = GROUP != 0 ? SEGS * RT : kSkinnyWaves;
    static_assert(SUM_UNITS <= kSkinnyWaves, "one wavefront per (group, row tile)");
    __shared__ f32x4 sum_lds[7][SUM_UNITS][4];

    int t;
    if (!xcd_tile(p.tiles_m * p.tiles_n, t))
        return;
    int tm = t % p.tiles_m;
    int const tn = t / p.tiles_m;
    if (p.expert_rows && !select_expert(p, tm, kSkinnyBM))
        return;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15;
    int const kg = lane >> 4;
    int const K = p.k;
    // this workgroup's slice of K, in tile rows; loads outside it return zeros
    int const kt_begin = SPLITK ? (int) blockIdx.y * p.tiles_per_split : 0;
    int const KT = SPLITK ? (kt_begin + p.tiles_per_split < p.k_tiles ? kt_begin + p.tiles_per_split : p.k_tiles)
                          : p.k_tiles;
    int const m0 = tm * kSkinnyBM;
    int const strip0 = tn * (kSkinnyBN / 16) + wave * NS;

    constexpr uint32_t kOob = 0x80000000u;
    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K * 2u);
    uint32_t const sz_bytes = (uint32_t) p.scale_rows * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) p.k_tiles * 1024u);

    bool const gated = !SPLITK && act_is_gated(p.activation);
    bool strip_ok[NS];
    int strip_of[NS];
    uint32_t wlane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        strip_of[s] = paired_strip(gated, strip0, s, p.strips, strip_ok[s]);
        wlane[s] = ((uint32_t) strip_of[s] * (uint32_t) p.k_tiles * 64u + (uint32_t) lane) * 16u;
    }

    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};
    u32x4 const ones = {E::kOnes, E::kOnes, E::kOnes, E::kOnes};
    [[maybe_unused]] NibbleConsts const nib = nibble_consts<DT>();

    // acc: finished sums (GROUP != 0) or the running P (per-channel scales are applied at the end);
    // acc_s: the running S of the per-channel mode
    f32x4 acc[RT][NS];
    f32x4 acc_s[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
    {
        acc_s[rt] = zero4;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc[rt][s] = zero4;
    }

    // A tile -> LDS, same fragment layout as the prefill kernel: fragment f = rt * SLABS + j is the
    // 16 rows x 32 k of one MFMA; lane l = 4*r + q fetches row r's 16-byte chunk q ^ frag_swizzle(r>>2), so
    // quads read contiguous 64 bytes from memory and the fragment read is bank-conflict free.
    constexpr int FRAGS = RT * SLABS;
    static_assert(FRAGS % kSkinnyWaves == 0, "fragments spread evenly over the wavefronts");
    constexpr int DMA_OPS = FRAGS / kSkinnyWaves;
    auto dma_a = [&](int buf, int kt)
    {
        int const r = lane >> 2, chunk = (lane & 3) ^ frag_swizzle(lane >> 4);
#pragma unroll
        for (int i = 0; i < DMA_OPS; ++i)
        {
            int const f = wave + i * kSkinnyWaves;
            int const rt = f / SLABS, j = f % SLABS;
            uint32_t const row = (uint32_t) (m0 + rt * 16 + r);
            int const kk = kt * TK + j * 32 + chunk * 8;
            // out of range (sign bit of K-1-kk or of KT-1-kt set) -> an offset the descriptor rejects
            uint32_t const off
                = ((row * (uint32_t) K + (uint32_t) kk) * 2u) | (((uint32_t) (K - 1 - kk) | (uint32_t) (KT - 1 - kt)) & kOob);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(act_rsrc,
                (__attribute__((address_space(3))) void*) (reinterpret_cast<char*>(stage_a[buf]->a) + f * 1024), 16,
                (int) off, 0, 0, 0);
        }
    };
    int const a_lane_off = (c * 4 + (kg ^ frag_swizzle(c >> 2))) * 16;

    struct Stage
    {
        u32x4 w[NS];
    };
    // vector-memory instructions one fetch_b issues (the explicit wait below counts them)
    constexpr int FETCH_OPS = NS + SC_SLOTS;

    // Scales (and zeros) of the wavefront's 16*NS columns for one group, fetched by the first 8*NS
    // lanes as dwords straight into LDS (the other lanes get zeros from an out-of-range offset).
    static_assert(NS == 2, "the scale fetch below picks between two strips");
    uint32_t const sc_lane_col = (uint32_t) (((lane & 31) < 8 ? strip_of[0] : strip_of[1]) * 16 + 2 * (lane & 7));
    uint32_t const sc_lane_oob = (lane >= 8 * NS || (int) sc_lane_col >= p.n) ? kOob : 0u;

    auto fetch_b = [&](Stage& st, int buf, int kt)
    {
        uint32_t const past = (uint32_t) (KT - 1 - kt) & kOob; // kt >= KT: every load of the step reads zeros
        uint32_t const tile_off = (uint32_t) kt * 1024u | past;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            st.w[s] = buffer_load_x4(w_rsrc, wlane[s] + tile_off);
        if constexpr (GROUP != 0)
        {
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                uint32_t const grow = scale_row<GROUP>((uint32_t) (kt * TK + seg * SEG), p.group_magic);
                uint32_t const off = ((grow * (uint32_t) p.n + sc_lane_col) * 2u) | past | sc_lane_oob;
                char* slot = reinterpret_cast<char*>(stage_sc[buf]->sc[wave]) + seg * (ZERO ? 512 : 256);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    sc_rsrc, (__attribute__((address_space(3))) void*) slot, 4, (int) off, 0, 0, 0);
                if constexpr (ZERO)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(
                        zr_rsrc, (__attribute__((address_space(3))) void*) (slot + 256), 4, (int) off, 0, 0, 0);
            }
        }
    };

    // One step = one tile row of K.  All A fragments of the step are read into registers once; the
    // strips are then processed one after the other, so only one strip's group sums (P) are live
    // at a time.  A single wavefront per SIMD has to overlap its own VALU work with the matrix
    // core, so the step is written as mini-blocks of ONE MFMA plus a few VALU instructions (a
    // scheduling barrier after each keeps them together):
    //   * the B operand of the next 4 MFMAs is expanded one register per mini-block;
    //   * the scale application of strip s-1 is spread over the 16 mini-blocks of strip s; that of
    //     the last strip is carried into the next step, where it runs first and covers the
    //     latency of the fragment reads.
    f32x4 part[2][SEGS][RT];   // P of the strip in flight / of the strip being scaled
    f32x4 part_s[SEGS][RT];    // S of the step's groups
    float sc[NS][SEGS], cc[NS][SEGS]; // s and z - OFFSET * s of the step (strip NS-1: of the pending strip)
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg)
    {
        sc[NS - 1][seg] = cc[NS - 1][seg] = 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
            part[1][seg][rt] = part_s[seg][rt] = zero4;
    }
    static_assert(NS % 2 == 0, "the last strip uses part[1]");

    // unit u of the scale application of strip s: one (group, row tile, register) of acc
    auto apply_unit = [&](int s, int u)
    {
        if constexpr (GROUP != 0)
        {
            int const seg = u % SEGS, rt = (u / SEGS) / 4, r = (u / SEGS) % 4;
            acc[rt][s][r] = __builtin_fmaf(
                sc[s][seg], part[s & 1][seg][rt][r], __builtin_fmaf(cc[s][seg], part_s[seg][rt][r], acc[rt][s][r]));
        }
    };
    constexpr int UNITS = SEGS * RT * 4; // per strip
    constexpr int PER_B = 4 / RT;        // registers of the next B operand expanded per mini-block
    static_assert(RT == 2 || RT == 4, "row tiles per wavefront");

    // register pr (elements 2pr, 2pr+1) of the B operand of slab j of a lane's 16 packed bytes
    auto expand_reg = [&](u32x4 const& w, int j, int pr) -> uint32_t
    {
        if constexpr (BITS == 4)
            return ((w[j] >> (4 * pr)) & nib.mask) | nib.magic;
        else
            return expand_int8_reg<DT>(w[2 * j + pr / 2], pr % 2);
    };

    // Row sums of the step whose A tile sits in buffer `buf`: wavefront w < SUM_UNITS sums (group
    // w / RT, row tile w % RT) against the all-ones operand and leaves the 16 sums in that slot.
    auto form_sums = [&](int buf)
    {
        if constexpr (GROUP != 0)
        {
            if (wave < SUM_UNITS)
            {
                int const seg = wave / RT, rt = wave % RT; // wave-uniform
                char const* frag
                    = reinterpret_cast<char const*>(stage_a[buf]->a) + a_lane_off + (rt * SLABS + seg * SEG_SLABS) * 1024;
                f32x4 sum = zero4;
#pragma unroll
                for (int js = 0; js < SEG_SLABS; ++js)
                    sum = E::mma(*reinterpret_cast<u32x4 const*>(frag + js * 1024), ones, sum);
                if (c == 0) // every column of the block holds the same sums; rows kg*4 .. kg*4+3
                    sum_lds[buf][wave][kg] = sum;
            }
        }
    };

    // With group scales the A tile of the NEXT step has landed when a step starts (its row sums are formed
    // during the step), so the step can also read the next step's A fragments into registers between its
    // matrix instructions: the burst of eight-wavefronts-times-eight LDS reads at the top of every step,
    // and the wait for it, go away.  Two fragment sets alternate (the loop is unrolled by an even number of
    // steps); with four row tiles only half of a second set fits the register file.
    constexpr bool A_AHEAD = (DEPTH + 1) % 2 == 0;
    // slabs read ahead: all with two row tiles; with four, all of them for int8 (two slabs per step), half
    // of them for int4 where the registers allow (group 128), the rest at the top of the step
    constexpr int AH = RT <= 2 ? SLABS : (BITS == 8 ? SLABS : (GROUP == 128 ? SLABS / 2 : 0));
    auto read_frags = [&](int buf, u32x4 (&a)[RT][SLABS])
    {
        char const* a_base = reinterpret_cast<char const*>(stage_a[buf]->a) + a_lane_off;
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                a[rt][j] = *reinterpret_cast<u32x4 const*>(a_base + (rt * SLABS + j) * 1024);
    };
    auto compute = [&](int buf, int buf_next, Stage const& st, u32x4 (&a_have)[RT][SLABS], u32x4 (&a_make)[RT][SLABS])
    {
        [[maybe_unused]] char const* sc_base = reinterpret_cast<char const*>(stage_sc[buf]->sc[wave]) + c * 2;
        [[maybe_unused]] char const* a_next_base = reinterpret_cast<char const*>(stage_a[buf_next]->a) + a_lane_off;
        u32x4 a[RT][SLABS];
        {
            char const* a_base = reinterpret_cast<char const*>(stage_a[buf]->a) + a_lane_off;
#pragma unroll
            for (int j = 0; j < SLABS; ++j)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    a[rt][j] = (A_AHEAD && j < AH) ? a_have[rt][j]
                                                   : *reinterpret_cast<u32x4 const*>(a_base + (rt * SLABS + j) * 1024);
        }
        uint16_t raw_s[NS][SEGS], raw_z[NS][SEGS];
        if constexpr (GROUP != 0)
        {
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int seg = 0; seg < SEGS; ++seg)
                {
                    char const* slot = sc_base + seg * (ZERO ? 512 : 256) + s * 32;
                    raw_s[s][seg] = *reinterpret_cast<uint16_t const*>(slot);
                    raw_z[s][seg] = ZERO ? *reinterpret_cast<uint16_t const*>(slot + 256) : (uint16_t) 0;
                }
        }
        __builtin_amdgcn_sched_barrier(0);

        // pending scale application of the previous step's last strip (uses the previous S)
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
            apply_unit(NS - 1, u);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (GROUP != 0)
        {
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int seg = 0; seg < SEGS; ++seg)
                {
                    sc[s][seg] = E::from_bits(raw_s[s][seg]);
                    cc[s][seg] = __builtin_fmaf(-OFF, sc[s][seg], ZERO ? E::from_bits(raw_z[s][seg]) : 0.f);
                }
        }

        u32x4 b_cur, b_nxt;
        if constexpr (GROUP != 0)
        {
            // this wavefront's share of the NEXT step's S, from the next A tile (it has landed: see
            // WAIT); this step's S was formed during the previous step and is read when the first
            // strip is done (until then the registers still hold the previous step's)
            form_sums(buf_next);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int x = 0; x < 4; ++x)
                b_cur[x] = expand_reg(st.w[0], 0, x);
            __builtin_amdgcn_sched_barrier(0);
        }
        else
        {
            // per-channel mode: this wavefront's share of the running row sums (fragments
            // wave * FPW .. of the step, all of one row tile), kept in acc_s[0] until the epilogue
            // adds the shares up
            constexpr int FPW = FRAGS / kSkinnyWaves;
            static_assert(FPW >= 1 && SLABS % FPW == 0, "a wavefront's fragments belong to one row tile");
            char const* frag = reinterpret_cast<char const*>(stage_a[buf]->a) + a_lane_off + wave * (FPW * 1024);
#pragma unroll
            for (int i = 0; i < FPW; ++i)
                acc_s[0] = E::mma(*reinterpret_cast<u32x4 const*>(frag + i * 1024), ones, acc_s[0]);
#pragma unroll
            for (int x = 0; x < 4; ++x)
                b_cur[x] = expand_reg(st.w[0], 0, x);
            __builtin_amdgcn_sched_barrier(0);
        }

#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
#pragma unroll
            for (int j = 0; j < SLABS; ++j)
            {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                {
                    if constexpr (GROUP != 0)
                        part[s & 1][j / SEG_SLABS][rt] = E::mma(
                            a[rt][j], b_cur, j % SEG_SLABS == 0 ? zero4 : part[s & 1][j / SEG_SLABS][rt]);
                    else
                        acc[rt][s] = E::mma(a[rt][j], b_cur, acc[rt][s]);
                    // this mini-block's share of the next B operand (4 registers per operand)
#pragma unroll
                    for (int x = rt * PER_B; x < (rt + 1) * PER_B; ++x)
                    {
                        if (j + 1 < SLABS)
                            b_nxt[x] = expand_reg(st.w[s], j + 1, x);
                        else if (s + 1 < NS)
                            b_nxt[x] = expand_reg(st.w[s + 1], 0, x);
                    }
                    if constexpr (A_AHEAD)
                    {
                        if (s == 0 && j < AH) // one fragment of the next step per mini-block of the first strip
                            a_make[rt][j] = *reinterpret_cast<u32x4 const*>(a_next_base + (rt * SLABS + j) * 1024);
                    }
                    if constexpr (GROUP != 0)
                    {
                        if (s == 0 && j == SLABS - 1 && rt == RT - 1)
                        {
#pragma unroll
                            for (int seg = 0; seg < SEGS; ++seg)
#pragma unroll
                                for (int rt2 = 0; rt2 < RT; ++rt2)
                                    part_s[seg][rt2] = sum_lds[buf][seg * RT + rt2][kg];
                        }
                    }
                    if (s > 0)
                    {
                        constexpr int BLOCKS = SLABS * RT; // mini-blocks per strip
                        static_assert(UNITS % BLOCKS == 0, "scale units spread evenly");
                        int const blk = j * RT + rt;
#pragma unroll
                        for (int u = blk * (UNITS / BLOCKS); u < (blk + 1) * (UNITS / BLOCKS); ++u)
                            apply_unit(s - 1, u);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                b_cur = b_nxt;
            }
        }
    };

    // ---- four row tiles, int4, group scales: A fragments just in time ----------------------------
    // With four row tiles a step uses 16 A fragments and no second set of them fits the register file, so
    // the step above reads half of them in one burst after the barrier - eight wavefronts at once, the LDS
    // pipe busy for about as long as the step's matrix instructions take, and nothing else running.  Here
    // the loops are ordered (slab, row tile, strip): a fragment feeds the two strips' matrix instructions
    // back to back and is dead afterwards, so a window of WIN fragments, refilled one per pair of
    // mini-blocks (from the next step's tile once this step's are all requested: it has landed, see WAIT),
    // spreads the LDS reads evenly over the step.  The sums P of both strips are live at once; a group's P
    // is applied one mini-block before the next step's first matrix instruction overwrites it.
    constexpr bool JIT = BITS == 4 && GROUP == 128 && RT == 4;
    constexpr int WIN = 4;
    u32x4 awin[WIN];
    f32x4 pj[NS][SEGS][RT];                // P of the step in flight / pending from the previous step
    f32x4 ps_p[SEGS][RT];                  // S that goes with the pending P
    float sc_p[NS][SEGS], cc_p[NS][SEGS];  // s and z - OFFSET * s that go with the pending P
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
        {
            ps_p[seg][rt] = zero4;
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                pj[s][seg][rt] = zero4;
                sc_p[s][seg] = cc_p[s][seg] = 0.f;
            }
        }
    // fragment f in the order of use: slab f / RT, row tile f % RT
    auto frag_at = [&](int buf, int f) -> u32x4
    {
        return *reinterpret_cast<u32x4 const*>(
            reinterpret_cast<char const*>(stage_a[buf]->a) + a_lane_off + ((f % RT) * SLABS + f / RT) * 1024);
    };
    auto apply_group = [&](int s, int seg, int rt)
    {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            acc[rt][s][r] = __builtin_fmaf(
                sc_p[s][seg], pj[s][seg][rt][r], __builtin_fmaf(cc_p[s][seg], ps_p[seg][rt][r], acc[rt][s][r]));
    };
    auto compute_jit = [&](int buf, int buf_next, Stage const& st)
    {
        char const* sc_base = reinterpret_cast<char const*>(stage_sc[buf]->sc[wave]) + c * 2;
        uint16_t raw_s[NS][SEGS], raw_z[NS][SEGS];
        f32x4 ps_n[SEGS][RT];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                char const* slot = sc_base + seg * (ZERO ? 512 : 256) + s * 32;
                raw_s[s][seg] = *reinterpret_cast<uint16_t const*>(slot);
                raw_z[s][seg] = ZERO ? *reinterpret_cast<uint16_t const*>(slot + 256) : (uint16_t) 0;
            }
#pragma unroll
        for (int seg = 0; seg < SEGS; ++seg)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                ps_n[seg][rt] = sum_lds[buf][seg * RT + rt][kg];
        __builtin_amdgcn_sched_barrier(0);
        form_sums(buf_next);
        __builtin_amdgcn_sched_barrier(0);
        u32x4 b_cur[NS], b_nxt[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int x = 0; x < 4; ++x)
                b_cur[s][x] = expand_reg(st.w[s], 0, x);
        apply_group(0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        float sc_n[NS][SEGS], cc_n[NS][SEGS];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                sc_n[s][seg] = E::from_bits(raw_s[s][seg]);
                cc_n[s][seg] = __builtin_fmaf(-OFF, sc_n[s][seg], ZERO ? E::from_bits(raw_z[s][seg]) : 0.f);
            }
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
        {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                int const f = j * RT + rt;
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    int const seg = j / SEG_SLABS;
                    pj[s][seg][rt] = E::mma(awin[f % WIN], b_cur[s], j % SEG_SLABS == 0 ? zero4 : pj[s][seg][rt]);
                    // the pending P that the NEXT mini-block overwrites (runs under this matrix instruction)
                    int const t = (j * RT + rt) * NS + s + 1;
                    int const tj = t / (RT * NS), trt = (t / NS) % RT, ts = t % NS;
                    if (tj < SLABS && tj % SEG_SLABS == 0)
                        apply_group(ts, tj / SEG_SLABS, trt);
                    // one register of this strip's next operand per mini-block
                    if (j + 1 < SLABS)
                        b_nxt[s][rt] = expand_reg(st.w[s], j + 1, rt);
                    if (s == NS - 1)
                        awin[f % WIN] = f + WIN < FRAGS ? frag_at(buf, f + WIN) : frag_at(buf_next, f + WIN - FRAGS);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
                b_cur[s] = b_nxt[s];
        }
#pragma unroll
        for (int seg = 0; seg < SEGS; ++seg)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                ps_p[seg][rt] = ps_n[seg][rt];
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    sc_p[s][seg] = sc_n[s][seg];
                    cc_p[s][seg] = cc_n[s][seg];
                }
            }
    };

    // ---- main loop --------------------------------------------------------------------------
    // Step kt: wait until everything this wavefront requested for step kt has landed, barrier (now
    // all of A(kt) is in LDS and nobody reads A(kt-1) any more), request step kt+DEPTH (its A tile
    // goes into the buffer A(kt-1) used), compute step kt.
    // Vector-memory operations retire in order, so "step kt has landed" is "at most the requests
    // of the DEPTH-1 younger steps are outstanding".
    // With group scales the A tile of step kt+1 must have landed as well (its row sums are formed
    // during step kt): a step's requests are its A DMAs followed by its weight-side requests, so
    // only the weight-side requests of step kt+1 may still be outstanding.
    // (the same when A fragments are read a step ahead)
    constexpr bool NEXT_A_LANDED = GROUP != 0 || (A_AHEAD && AH > 0);
    constexpr int WAIT = NEXT_A_LANDED ? (DEPTH - 2) * (FETCH_OPS + DMA_OPS) + FETCH_OPS : (DEPTH - 1) * (FETCH_OPS + DMA_OPS);
    static_assert(DEPTH >= 2 && WAIT < 64, "vmcnt is a 6-bit counter");
    Stage st[DEPTH + 1];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i)
    {
        dma_a(i, kt_begin + i);
        fetch_b(st[i], i, kt_begin + i);
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (NEXT_A_LANDED)
    {
        // row sums (and fragments) of the first step: its A tile has landed once at most the younger steps
        // and its own weight-side requests are outstanding
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((DEPTH - 1) * (FETCH_OPS + DMA_OPS) + FETCH_OPS) : "memory");
        form_sums(0);
    }
    u32x4 a_set0[RT][SLABS], a_set1[RT][SLABS];
    if constexpr (JIT)
    {
#pragma unroll
        for (int f = 0; f < WIN; ++f)
            awin[f] = frag_at(0, f);
    }
    else if constexpr (A_AHEAD && AH > 0)
    {
        read_frags(0, a_set0);
    }
    for (int kt = kt_begin; kt < KT; kt += DEPTH + 1)
    {
#pragma unroll
        for (int u = 0; u < DEPTH + 1; ++u)
        {
            // (lgkmcnt: the row sums this wavefront wrote for step kt are in LDS before anyone reads them)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(WAIT) : "memory");
            __builtin_amdgcn_sched_barrier(0);
            dma_a((u + DEPTH) % (DEPTH + 1), kt + u + DEPTH);
            fetch_b(st[(u + DEPTH) % (DEPTH + 1)], (u + DEPTH) % (DEPTH + 1), kt + u + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
            if (kt + u < KT) // uniform; the requests above go on (they read zeros past the end of K)
            {
                if constexpr (JIT)
                    compute_jit(u, (u + 1) % (DEPTH + 1), st[u]);
                else
                    compute(u, (u + 1) % (DEPTH + 1), st[u], u % 2 == 0 ? a_set0 : a_set1, u % 2 == 0 ? a_set1 : a_set0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // no DMA may still be writing LDS when the wavefront ends
    if constexpr (GROUP == 0)
    {
        // row sums of the per-channel mode: add the wavefronts' shares (wavefront w summed row tile
        // w * FPW / SLABS)
        constexpr int FPW = FRAGS / kSkinnyWaves;
        if (c == 0)
            sum_lds[0][wave][kg] = acc_s[0];
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
        {
            f32x4 t = zero4;
#pragma unroll
            for (int w = 0; w < kSkinnyWaves; ++w)
                if (w * FPW / SLABS == rt)
                    t += sum_lds[0][w][kg];
            acc_s[rt] = t;
        }
    }
    if constexpr (JIT)
    {
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    apply_group(s, seg, rt); // the last step's sums
    }
    else
    {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
            apply_unit(NS - 1, u); // the last step's last strip
    }

    // ---- epilogue ----------------------------------------------------------------------------
    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    // finished sum of (row tile, strip slot, register): per-channel scales are applied here
    auto finished = [&](int rt, int s, int r, float pc) -> float
    {
        float v = acc[rt][s][r];
        if constexpr (GROUP == 0)
            v = __builtin_fmaf(pc, v, (-OFF * pc) * acc_s[rt][r]);
        return v;
    };
    int const n_out = gated ? p.n / 2 : p.n;
    // The residual is read through a descriptor (rows >= m read zeros, so no branches) and one row
    // tile at a time, all loads of the tile in flight before the first is used.
    auto const res_rsrc = make_rsrc(p.residual ? p.residual : p.out, (uint32_t) p.m * (uint32_t) n_out * 2u);
    if (gated)
    {
        // value and gate sums of an output element sit in the two strip slots of this lane
        if constexpr (!SPLITK)
        {
            auto gated_epilogue = [&](auto act_tag)
            {
                constexpr int ACT = decltype(act_tag)::value;
                if (!strip_ok[0])
                    return;
                int const col = strip_of[0] * 16 + c; // strip_of[0] is the pair index (value half)
                float const bias_x = p.bias ? E::load(p.bias, col) : 0.f;
                float const bias_g = p.bias ? E::load(p.bias, col + n_out) : 0.f;
                [[maybe_unused]] float const pc_x = GROUP == 0 ? E::load(p.scales, col) : 0.f;
                [[maybe_unused]] float const pc_g = GROUP == 0 ? E::load(p.scales, col + n_out) : 0.f;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                {
                    int const row0 = m0 + rt * 16 + kg * 4;
                    float res[4] = {};
                    if (p.residual)
                    {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            res[r] = E::from_bits(buffer_load_u16(
                                res_rsrc, ((uint32_t) (row0 + r) * (uint32_t) n_out + (uint32_t) col) * 2u));
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (row0 + r < p.m)
                            out16[(size_t) (row0 + r) * n_out + col] = E::store((finished(rt, 0, r, pc_x) + bias_x)
                                    * apply_act(ACT, finished(rt, 1, r, pc_g) + bias_g)
                                + res[r]);
                }
            };
            if (p.activation == kActSwiglu)
                gated_epilogue(std::integral_constant<int, kActSwiglu>{});
            else
                gated_epilogue(std::integral_constant<int, kActGeglu>{});
        }
        return;
    }
    int col[NS];
    float bias[NS];
    [[maybe_unused]] float pc[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        col[s] = strip_of[s] * 16 + c;
        bias[s] = (!SPLITK && p.bias) ? E::load(p.bias, col[s]) : 0.f;
        pc[s] = GROUP == 0 ? E::load(p.scales, col[s]) : 0.f;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
    {
        int const row0 = m0 + rt * 16 + kg * 4;
        float res[NS][4] = {};
        if (!SPLITK && p.residual)
        {
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    res[s][r] = E::from_bits(
                        buffer_load_u16(res_rsrc, ((uint32_t) (row0 + r) * (uint32_t) p.n + (uint32_t) col[s]) * 2u));
        }
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                float const v = finished(rt, s, r, pc[s]);
                if (strip_ok[s] && row0 + r < p.m)
                {
                    if constexpr (SPLITK)
                        (p.partial + (size_t) blockIdx.y * ((size_t) p.m * p.n))[(size_t) (row0 + r) * p.n + col[s]] = v;
                    else
                        out16[(size_t) (row0 + r) * p.n + col[s]] = E::store(__builtin_fmaf(p.alpha, v, bias[s]) + res[s][r]);
                }
            }
    }
}

template <int DT, int BITS, int GROUP, bool ZERO, int RT>
int launch_skinny_rt(GemmParams const& gp, hipStream_t stream)
{
    int const total = gp.tiles_m * gp.tiles_n;
    dim3 grid(((total + 7) / 8) * 8, gp.k_splits), block(kSkinnyWaves * 64), block256(256);
    note_launch("gemm skinny rt=%d splits=%d", RT, gp.k_splits);
    if (gp.k_splits > 1)
    {
        size_t const count = (size_t) gp.m * gp.n;
        hipLaunchKernelGGL((skinny_kernel<DT, BITS, GROUP, ZERO, RT, true>), grid, block, 0, stream, gp);
        hipLaunchKernelGGL((gemm_finish_partial<DT>), dim3((unsigned) ((count / 4 + 255) / 256)), block256, 0, stream,
            gp.out, gp.partial, gp.bias, gp.alpha, gp.m, gp.n, gp.k_splits);
    }
    else
        hipLaunchKernelGGL((skinny_kernel<DT, BITS, GROUP, ZERO, RT, false>), grid, block, 0, stream, gp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "skinny gemm kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int DT, int BITS, int GROUP, bool ZERO>
int launch_skinny_variant(GemmParams const& gp, int rt, hipStream_t stream)
{
    if constexpr (BITS == 4)
    {
        if (rt == 2)
            return launch_skinny_rt<DT, BITS, GROUP, ZERO, 2>(gp, stream);
    }
    return launch_skinny_rt<DT, BITS, GROUP, ZERO, 4>(gp, stream);
}

template <int DT, int BITS>
int launch_skinny_typed(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    constexpr int TK = BITS == 4 ? 128 : 64;
    GemmParams gp;
    gp.act = p.act;
    gp.weight = p.weight;
    gp.scales = p.scales;
    gp.zeros = p.zeros;
    gp.bias = p.bias;
    gp.out = p.out;
    gp.alpha = p.alpha;
    gp.m = p.m;
    gp.n = p.n;
    gp.k = p.k;
    gp.k_tiles = (p.k + TK - 1) / TK;
    gp.strips = p.n / kTileN;
    int const rt = (BITS == 4 && plan.rt == 2) ? 2 : 4;
    gp.tiles_m = (p.m + rt * 16 - 1) / (rt * 16);
    gp.tiles_n = (p.n + kSkinnyBN - 1) / kSkinnyBN;
    gp.k_splits = plan.k_splits;
    gp.tiles_per_split = (gp.k_tiles + plan.k_splits - 1) / plan.k_splits;
    gp.partial = static_cast<float*>(p.workspace);
    if (plan.k_splits > 1 && (!p.workspace || p.workspace_bytes < plan.ws_bytes))
        return fail(WOQ_ERR_WORKSPACE, "split-K needs %zu workspace bytes", plan.ws_bytes);
    set_group_fields(gp, p, rt * 16);
    auto s = static_cast<hipStream_t>(stream);
    bool const zero = p.zeros != nullptr;
    switch (template_group(p.group_size))
    {
    case 0: return launch_skinny_variant<DT, BITS, 0, false>(gp, rt, s);
    case 64:
        return zero ? launch_skinny_variant<DT, BITS, 64, true>(gp, rt, s)
                    : launch_skinny_variant<DT, BITS, 64, false>(gp, rt, s);
    case 128:
        return zero ? launch_skinny_variant<DT, BITS, 128, true>(gp, rt, s)
                    : launch_skinny_variant<DT, BITS, 128, false>(gp, rt, s);
    case kFlexGroup:
        return zero ? launch_skinny_variant<DT, BITS, kFlexGroup, true>(gp, rt, s)
                    : launch_skinny_variant<DT, BITS, kFlexGroup, false>(gp, rt, s);
    default: return fail(WOQ_ERR_UNSUPPORTED, "group_size %d", p.group_size);
    }
}

} // namespace woq
