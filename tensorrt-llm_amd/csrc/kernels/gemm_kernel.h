// Prefill GEMM: fp16/bf16 activations x int4/int8 weights on the 16x16x32 matrix core.
//
// Counterpart of the reference's CUTLASS mixed-input GEMM
// (cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h:57-230 and the
// dequantizing main loop in cutlass_extensions/.../gemm/threadblock/dq_mma_multistage_finegrained.h)
// in semantics only: out = T(alpha * A x dequant(W) + bias), float32 accumulation, weights
// dequantized to the activation type by the single definition in dequant_math.h.
//
// Design for CDNA4 (one workgroup of 4 wavefronts per CU, 256 x 256 output tile):
//   * the 4 wavefronts sit side by side along N: each owns 256 rows x 64 columns (16 x 4 MFMA
//     tiles, 256 float32 accumulator registers per lane).  Weight columns are therefore disjoint
//     between wavefronts: every packed weight is loaded from memory once per workgroup, straight
//     into the registers of the lane that feeds it to the matrix core (the tile layout of
//     host_prep.cpp IS the B-operand register layout), and is dequantized exactly once.  Weights
//     never touch LDS.
//   * the activation tile (256 rows x one weight tile row of K) is shared by the 4 wavefronts: it
//     is DMA-ed global -> LDS (buffer_load ... lds, no staging registers) in MFMA-fragment order,
//     so every A-fragment read is one conflict-free ds_read_b128 of consecutive lanes.  Two LDS
//     buffers alternate: the DMA for step k+1 runs under the MFMAs of step k.
//   * rows >= M and the zero-filled tail of K come back as zeros from the buffer descriptor.
#pragma once

#include "dequant_math.h"
#include <type_traits>

#include "gemm_common.h"

namespace woq
{

constexpr int kGemmGroupM = 4; // m-tiles walked together so that concurrent workgroups share panels in L2

// amdgpu_waves_per_eu(1, 1): one wavefront per SIMD is the design point (256 accumulator
// registers per lane); without it the register allocator chases a higher occupancy it cannot
// reach and parks live values in the accumulator file, shuffling them around every step.
//
// RT     row tiles (16 rows) per wavefront: the output tile is 16*RT rows x 256 columns.  16 for
//        prefill; 8 / 4 for skinny M, where a 256-row tile would mostly multiply padding.
// SPLITK several workgroups share one output tile, each covering a slice of K, and add their
//        partial sums into a float32 buffer (skinny M x narrow N would otherwise leave most CUs idle).
// PERSIST one workgroup per CU walks several output tiles (tile b, b + gridDim.x, ...).  The last tile
//        row of a tile already requests the first A tile and weights of the NEXT tile, and the
//        outputs of a finished tile are converted and stored between the matrix instructions of
//        the next tile's first tile row (each accumulator block right before it is cleared for
//        reuse): neither the first-load latency of a tile nor its burst of 128 KiB of stores is
//        paid with the matrix core idle.  Plain epilogue only (bias; no activation, no residual);
//        K must be an even number of tile rows; m * n * 2 < 2 GiB (outputs go through a descriptor).
template <int DT, int BITS, int GROUP, bool ZERO, int RT, bool SPLITK, bool PERSIST = false, int NS_ = 4>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) gemm_kernel(GemmParams p)
{
    static_assert(!(PERSIST && SPLITK), "a persistent workgroup owns whole tiles");
    using E = Elem<DT>;
    constexpr int TK = BITS == 4 ? 128 : 64;
    constexpr int SLABS = TK / 32;
    constexpr int kGemmBM = RT * 16;
    constexpr int NS = NS_;       // strips (16 columns) per wavefront: 4, or 3 for 192-column tiles (not with gated activations)
    constexpr int BN = NS * 64;   // columns of the output tile
    constexpr int SEG = segment_rows<GROUP, TK>(); // rows sharing one scale inside a tile row
    constexpr int SEGS = TK / SEG;
    constexpr int SEG_SLABS = SEG / 32;
    constexpr int A_BYTES = kGemmBM * TK * 2;

    __shared__ u32x4 a_buf0[A_BYTES / 16];
    __shared__ u32x4 a_buf1[A_BYTES / 16];

    // ---- which output tile: XCD-contiguous chunks, m fastest inside groups of kGemmGroupM ------
    // (virtual block vb: the block index itself, or with PERSIST the block index plus a multiple of
    // the grid size, which is a multiple of 8 - a workgroup stays on its XCD's chunk of the order)
    int const total = p.tiles_m * p.tiles_n;
    int const per_xcd = (total + 7) / 8;
    auto tile_of = [&](int vb, int& tm_, int& tn_) -> bool
    {
        int const t = (vb & 7) * per_xcd + (vb >> 3);
        if ((vb >> 3) >= per_xcd || t >= total)
            return false;
        int const in_group = kGemmGroupM * p.tiles_n;
        int const first_m = (t / in_group) * kGemmGroupM;
        int const gsz = p.tiles_m - first_m < kGemmGroupM ? p.tiles_m - first_m : kGemmGroupM;
        tm_ = first_m + (t % in_group) % gsz;
        tn_ = (t % in_group) / gsz;
        return true;
    };
    int vb = (int) blockIdx.x;
    int tm, tn;
    if (!tile_of(vb, tm, tn))
        return;
    if (p.expert_rows && !select_expert(p, tm, kGemmBM))
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
    int m0 = tm * kGemmBM;
    int strip0 = tn * (BN / 16) + wave * NS;
    uint32_t tile_oob = 0; // PERSIST: kOob once there is no further tile (every request reads zeros)

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

    f32x4 acc[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc[rt][s] = f32x4{0.f, 0.f, 0.f, 0.f};

    // per-column scale of the per-channel mode (GROUP == 0) is loaded once
    float pc_scale[NS];
    uint32_t pc_scale2[NS]; // the raw 16-bit value in both halves
    // the same for the tile row after the current one (PERSIST: another tile's columns at a tile boundary)
    float pc_scale_n[NS];
    uint32_t pc_scale2_n[NS];
    if constexpr (GROUP == 0)
    {
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            pc_scale[s] = pc_scale_n[s] = E::load(p.scales, strip_of[s] * 16 + c);
            pc_scale2[s] = pc_scale2_n[s]
                = (uint32_t) static_cast<uint16_t const*>(p.scales)[strip_of[s] * 16 + c] * 0x10001u;
        }
    }

    // A tile -> LDS.  Fragment f = rt * SLABS + j is 1 KiB: the 16 rows x 32 k that one MFMA
    // consumes.  The DMA writes lane l's 16 bytes at offset l*16 of the fragment, so the lane
    // order of the load instruction IS the LDS layout.  Lane l = 4*r + q fetches row r's chunk
    // (q ^ (r>>2)) of the slab (a chunk = 8 k = 16 bytes):
    //   * the 4 lanes of a quad read one contiguous 64-byte piece of a row (the L1 handles a
    //     wavefront quad by quad: per-lane scattered 16-byte reads run 4x slower);
    //   * the XOR spreads the 16 rows that an MFMA lane group (fixed chunk) reads over all 64
    //     banks, so the fragment read below is conflict-free.
    // Wavefront w moves fragments w, w+4, ...
    // Wavefront w moves fragments w, w+4, ...: piece i is fragment f = w + 4i, i.e. slab w % SLABS
    // of row tile i * (4 / SLABS) + w / SLABS - the same slab for every piece, rows a fixed stride
    // apart, so one per-lane base (set once per step, out of range past the end of K) plus a
    // compile-time multiple of the row stride addresses every piece.
    constexpr int FRAGS = RT * SLABS;
    constexpr int DMA_OPS = FRAGS / 4;
    static_assert(4 % SLABS == 0 && FRAGS % 4 == 0, "fragment to wavefront mapping");
    int const dma_j = wave % SLABS;
    uint32_t dma_lane_base = ((uint32_t) (m0 + (wave / SLABS) * 16 + (lane >> 2)) * (uint32_t) K
                                 + (uint32_t) (dma_j * 32 + (((lane & 3) ^ frag_swizzle(lane >> 4)) * 8)))
        * 2u;
    int const dma_lane_k = dma_j * 32 + (((lane & 3) ^ frag_swizzle(lane >> 4)) * 8); // k of this lane inside a tile row
    uint32_t const dma_piece_stride = (uint32_t) (4 / SLABS) * 16u * (uint32_t) K * 2u;
    auto dma_base = [&](int kt) -> uint32_t
    {
        // out of range (sign bit of K-1-k or of KT-1-kt set) -> an offset the descriptor rejects;
        // rows past M fall outside the descriptor by themselves
        int const kk = kt * TK + dma_lane_k;
        return (dma_lane_base + (uint32_t) kt * (uint32_t) (TK * 2))
            | (((uint32_t) (K - 1 - kk) | (uint32_t) (KT - 1 - kt)) & kOob) | tile_oob;
    };
    auto dma_piece = [&](auto* buf, uint32_t base, int i)
    {
        int const f = wave + i * 4;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(act_rsrc,
            (__attribute__((address_space(3))) void*) (reinterpret_cast<char*>(buf) + f * 1024), 16,
            (int) (base + (uint32_t) i * dma_piece_stride), 0, 0, 0);
    };
    auto dma_a = [&](auto* buf, int kt)
    {
        uint32_t const base = dma_base(kt);
#pragma unroll
        for (int i = 0; i < DMA_OPS; ++i)
            dma_piece(buf, base, i);
    };
    // where MFMA lane (kg, c) finds its operand (row c, chunk kg) inside a fragment
    int const a_lane_off = (c * 4 + (kg ^ frag_swizzle(c >> 2))) * 16;

    struct BStage
    {
        u32x4 w[NS];
        uint16_t s[NS][SEGS];
        uint16_t z[NS][SEGS];
    };

    // piece i of the weight-side requests of step kt: the NS packed-weight loads, then the scales
    // and zeros of the step's groups
    constexpr int FETCH_OPS = NS + (GROUP != 0 ? NS * SEGS * (ZERO ? 2 : 1) : 0);
    uint32_t sc_lane[NS]; // byte offset of this lane's column in a scale row
#pragma unroll
    for (int s = 0; s < NS; ++s)
        sc_lane[s] = (uint32_t) (strip_of[s] * 16 + c) * 2u;
    auto fetch_piece = [&](BStage& st, int kt, int i)
    {
        uint32_t const past = ((uint32_t) (KT - 1 - kt) & kOob) | tile_oob; // kt >= KT: every load of the step reads zeros
        if (i < NS)
            st.w[i] = buffer_load_x4(w_rsrc, wlane[i] + ((uint32_t) kt * 1024u | past));
        else if constexpr (GROUP != 0)
        {
            int const q = i - NS, which = q / (NS * SEGS), seg = (q / NS) % SEGS, s = q % NS;
            uint32_t const grow = scale_row<GROUP>((uint32_t) (kt * TK + seg * SEG), p.group_magic);
            uint32_t const off = (grow * (uint32_t) p.n * 2u + sc_lane[s]) | past;
            if (which == 0)
                st.s[s][seg] = buffer_load_u16(sc_rsrc, off);
            else
                st.z[s][seg] = buffer_load_u16(zr_rsrc, off);
        }
    };
    auto fetch_b = [&](BStage& st, int kt)
    {
#pragma unroll
        for (int i = 0; i < FETCH_OPS; ++i)
            fetch_piece(st, kt, i);
    };

    // One tile row of MFMAs.  Hand-pipelined, because left alone the compiler hoists all
    // fragment reads and conversions of the step to its top and runs out of registers:
    //   * iteration (j, rt) issues the A-fragment read that is A_AHEAD iterations away (LDS
    //     latency is a few MFMA groups long), converts 16/RT operand registers of the next slab's
    //     B operands (16 registers per slab) and issues the 4 MFMAs of this row tile;
    //   * the B operands of the first slab of the NEXT tile row are converted during the last
    //     slab of this one (its packed weights were fetched at the start of this step), so the
    //     matrix core never waits for a conversion burst at a step boundary;
    //   * the memory requests of the next step (weight-side loads first: they are converted in this
    //     step's last slab; then the A-tile DMAs) are spread over the iterations as well: a
    //     wavefront that issues them in one burst sits in instruction issue while the matrix core
    //     runs dry;
    //   * a scheduling barrier after every iteration keeps that interleaving intact.
    constexpr int A_AHEAD = 3;
    u32x4 b_cur[NS], b_nxt[NS];

    auto scale_of = [&](BStage const& st, int s, int seg, float& sc, float& zr, bool next_step = false)
    {
        if constexpr (GROUP != 0)
        {
            sc = E::from_bits(st.s[s][seg]);
            zr = ZERO ? E::from_bits(st.z[s][seg]) : 0.f;
        }
        else
        {
            sc = next_step ? pc_scale_n[s] : pc_scale[s];
            zr = 0.f;
        }
    };

    // the same as packed half-precision pairs (s, s) and (z, z), from the raw 16-bit values
    auto scale_pair_of = [&](BStage const& st, int s, int seg, uint32_t& s2, uint32_t& z2, bool next_step = false)
    {
        if constexpr (GROUP != 0)
        {
            s2 = (uint32_t) st.s[s][seg] * 0x10001u;
            z2 = ZERO ? (uint32_t) st.z[s][seg] * 0x10001u : 0u;
        }
        else
        {
            s2 = next_step ? pc_scale2_n[s] : pc_scale2[s];
            z2 = 0u;
        }
    };

    // PERSIST: where the finished tile's outputs go (set when the workgroup moves on to its next tile)
    [[maybe_unused]] auto const out_rsrc = make_rsrc(p.out, (uint32_t) p.m * (uint32_t) p.n * 2u);
    // byte offset of (row m0 + c, column strip0*16 + kg*4) of the tile to store (the launcher only
    // takes this path when N is a multiple of the tile width and there is no bias: every strip of
    // the tile exists, rows past M fall outside the descriptor); kOob: no finished tile yet
    [[maybe_unused]] uint32_t prev_off = kOob;
    [[maybe_unused]] uint32_t const rt_stride = 16u * (uint32_t) p.n * 2u; // bytes between row tiles of the output
    auto store_block = [&](int rt, int s)
    {
        // read out through explicit AGPR-source moves: a plain use of the block by VALU code would make
        // the allocator keep every accumulator in the VGPR half of the file across the whole loop
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[r]) : "a"(acc[rt][s][r]));
        u32x2 const o = {E::pack(p.alpha * v[0], p.alpha * v[1]), E::pack(p.alpha * v[2], p.alpha * v[3])};
        // the row-tile offset belongs in the vector offset: the descriptor's range check does not
        // see the scalar offset, and rows past M must be dropped by it
        __builtin_amdgcn_raw_buffer_store_b64(o, out_rsrc, (int) (prev_off + (uint32_t) rt * rt_stride + (uint32_t) s * 32u), 0, 0);
    };

    auto compute = [&](auto first_tag, auto const* buf, BStage const& st, BStage& st_next, auto* buf_next, int kt_next)
    {
        constexpr bool FIRST = decltype(first_tag)::value; // first tile row of a tile (PERSIST only)
        char const* a_base = reinterpret_cast<char const*>(buf) + a_lane_off;
        constexpr int ITERS = SLABS * RT;
        uint32_t const next_base = dma_base(kt_next);
        auto a_addr = [&](int it) { return a_base + ((it % RT) * SLABS + it / RT) * 1024; };
        u32x4 a_ring[A_AHEAD + 1];
#pragma unroll
        for (int i = 0; i < A_AHEAD; ++i)
            a_ring[i] = *reinterpret_cast<u32x4 const*>(a_addr(i));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
        {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                int const it = j * RT + rt;
                // weight-side pieces all before the last slab (which converts them), DMAs throughout
                // (one per iteration from the start: they travel the farthest, from HBM)
                constexpr int FETCH_WINDOW = (SLABS - 1) * RT < FETCH_OPS ? (SLABS - 1) * RT : FETCH_OPS;
#pragma unroll
                for (int q = 0; q < FETCH_OPS; ++q)
                    if (q * FETCH_WINDOW / FETCH_OPS == it)
                        fetch_piece(st_next, kt_next, q);
                constexpr int DMA_WINDOW = ITERS * 5 / 8 > 0 ? ITERS * 5 / 8 : 1; // leave the tail of the step for them to land
#pragma unroll
                for (int q = 0; q < DMA_OPS; ++q)
                    if (q * DMA_WINDOW / DMA_OPS == it)
                        dma_piece(buf_next, next_base, q);
                if (it + A_AHEAD < ITERS)
                    a_ring[(it + A_AHEAD) % (A_AHEAD + 1)]
                        = *reinterpret_cast<u32x4 const*>(a_addr(it + A_AHEAD));
                // The conversion of this iteration's 16/RT operand registers runs in 4 stages, one
                // after each of the 4 MFMAs: a wavefront issues in order, so VALU work only runs
                // under the matrix core when it sits between the matrix instructions.
                constexpr int CONV = (NS * 4 + RT - 1) / RT; // NS * 4 operand registers per slab over RT iterations
                // bf16: q/16 as float (v_cvt_off_f32_i4 / sign-extending byte converts, with byte
                // selects on the source), float32 FMA with 16*s, packed round to bf16.
                // fp16: the exponent-magic pair (BASE + u), one packed subtract to the exact q and
                // one packed half-precision FMA.
                float t0[CONV], t1[CONV], sc[CONV], zr[CONV];
                uint32_t h2[CONV], s2[CONV], z2[CONV];
                auto conv_stage = [&](int stage)
                {
#pragma unroll
                    for (int x = 0; x < CONV; ++x)
                    {
                        int const ci = rt * CONV + x, s = ci / 4, pr = ci % 4;
                        if (ci >= NS * 4)
                            continue;
                        bool const same_step = j + 1 < SLABS;
                        BStage const& src = same_step ? st : st_next;
                        int const jn = same_step ? j + 1 : 0;
                        if constexpr (DT == WOQ_BF16)
                        {
                            if (stage == 0)
                            {
                                scale_of(src, s, jn / SEG_SLABS, sc[x], zr[x], !same_step);
                                sc[x] *= BITS == 4 ? 16.f : 1.f;
                            }
                            else if (stage == 1)
                            {
                                if constexpr (BITS == 4)
                                    int4_pair_sixteenths(src.w[s][jn] ^ 0x88888888u, pr, t0[x], t1[x]);
                                else
                                    int8_pair_float(src.w[s][2 * jn + pr / 2] ^ 0x80808080u, pr & 1, t0[x], t1[x]);
                            }
                            else if (stage == 2)
                            {
                                t0[x] = __builtin_fmaf(t0[x], sc[x], zr[x]);
                                t1[x] = __builtin_fmaf(t1[x], sc[x], zr[x]);
                            }
                            else
                                b_nxt[s][pr] = E::pack(t0[x], t1[x]);
                        }
                        else
                        {
                            if (stage == 0)
                                scale_pair_of(src, s, jn / SEG_SLABS, s2[x], z2[x], !same_step);
                            else if (stage == 1)
                            {
                                if constexpr (BITS == 4)
                                    h2[x] = ((src.w[s][jn] >> (4 * pr)) & 0x000F000Fu) | E::kMagic4;
                                else
                                    h2[x] = expand_int8_reg<WOQ_FP16>(src.w[s][2 * jn + pr / 2], pr & 1);
                            }
                            else if (stage == 2)
                                h2[x] = half2_add(h2[x], -Offset<DT, BITS>::value);
                            else
                                b_nxt[s][pr] = half2_fma(h2[x], s2[x], z2[x]);
                        }
                    }
                };
                u32x4 const a_cur = a_ring[it % (A_AHEAD + 1)];
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    if constexpr (FIRST)
                    {
                        // the block's sums of the previous tile leave (rows past M and strips past N
                        // fall outside the descriptor) right before the block starts the new tile's sum
                        if (j == 0)
                            store_block(rt, s);
                    }
                    // weights as the first operand: the accumulator holds the TRANSPOSED 16x16 block,
                    // lane (kg, c) the four consecutive columns kg*4 .. kg*4+3 of output row c, so the
                    // epilogue moves 8 bytes per lane and block instead of 2
                    // (the split-K variant keeps the plain orientation: its float32 stores cover
                    // 64 consecutive bytes per row and instruction)
                    if constexpr (SPLITK)
                        E::mma_acc(a_cur, b_cur[s], acc[rt][s]);
                    else if (FIRST && j == 0)
                        E::mma_first(b_cur[s], a_cur, acc[rt][s]); // the block starts the new tile's sum
                    else
                        E::mma_acc(b_cur[s], a_cur, acc[rt][s]);
                    conv_stage(s);
                    if (NS < 4 && s == NS - 1) // fewer matrix instructions than stages: the last one takes the rest
                        for (int rest = NS; rest < 4; ++rest)
                            conv_stage(rest);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
                b_cur[s] = b_nxt[s];
        }
    };

    // ---- main loop: two tile rows per iteration so that each LDS buffer is a distinct object ---
    BStage st0, st1;
    dma_a(a_buf0, kt_begin);
    fetch_b(st0, kt_begin);
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int pr = 0; pr < 4; ++pr)
        {
            float sc, zr;
            scale_of(st0, s, 0, sc, zr);
            b_cur[s][pr] = dequant_operand_reg<DT, BITS>(st0.w[s], 0, pr, sc, zr);
        }
    // Before each barrier a wavefront waits for its own A-tile DMAs explicitly: the wait the
    // compiler derives for them may be placed behind the barrier, where it no longer says anything
    // about the fragments the OTHER wavefronts moved.
    if constexpr (!PERSIST)
    {
        for (int kt = kt_begin; kt < KT; kt += 2)
        {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads(); // A(kt) has landed for every wavefront; everyone is done reading buffer 1
            compute(std::false_type{}, a_buf0, st0, st1, a_buf1, kt + 1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            compute(std::false_type{}, a_buf1, st1, st0, a_buf0, kt + 2); // past the end of K both operands read as zeros: no branch needed
        }
    }
    else
    {
        // Tiles one after the other (KT is even: every tile starts on buffer 0).  The second tile row
        // of a tile's last pair requests tile row 0 of the NEXT tile: the per-tile values are switched
        // over right before it - its own matrix instructions need operands and accumulators only.
        // Straight-line code around a plain inner loop (KT >= 4): the first tile row, the second, the
        // pairs in between, and the last pair with the switch-over.  A branch that chose between the
        // first-tile-row code and the ordinary one inside the loop, or a loop left from its middle,
        // makes the allocator keep second copies of the accumulators, and all 256 AGPRs are theirs.
        auto step_barrier = [&]()
        {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        };
        do
        {
            step_barrier();
            compute(std::true_type{}, a_buf0, st0, st1, a_buf1, 1);
            step_barrier();
            compute(std::false_type{}, a_buf1, st1, st0, a_buf0, 2);
            for (int kt = 2; kt < KT - 2; kt += 2)
            {
                step_barrier();
                compute(std::false_type{}, a_buf0, st0, st1, a_buf1, kt + 1);
                step_barrier();
                compute(std::false_type{}, a_buf1, st1, st0, a_buf0, kt + 2);
            }
            step_barrier();
            compute(std::false_type{}, a_buf0, st0, st1, a_buf1, KT - 1);
            step_barrier();
            {
                {
                    // this tile's outputs: stored during the next tile's first tile row (or below)
                    prev_off = ((uint32_t) (m0 + c) * (uint32_t) p.n + (uint32_t) (strip0 * 16 + kg * 4)) * 2u;
                    vb += (int) gridDim.x;
                    if (tile_of(vb, tm, tn))
                    {
                        m0 = tm * kGemmBM;
                        strip0 = tn * (BN / 16) + wave * NS;
#pragma unroll
                        for (int s = 0; s < NS; ++s)
                        {
                            strip_of[s] = paired_strip(false, strip0, s, p.strips, strip_ok[s]);
                            wlane[s] = ((uint32_t) strip_of[s] * (uint32_t) p.k_tiles * 64u + (uint32_t) lane) * 16u;
                            sc_lane[s] = (uint32_t) (strip_of[s] * 16 + c) * 2u;
                            if constexpr (GROUP == 0)
                            {
                                pc_scale_n[s] = E::load(p.scales, strip_of[s] * 16 + c);
                                pc_scale2_n[s]
                                    = (uint32_t) static_cast<uint16_t const*>(p.scales)[strip_of[s] * 16 + c] * 0x10001u;
                            }
                        }
                        dma_lane_base = ((uint32_t) (m0 + (wave / SLABS) * 16 + (lane >> 2)) * (uint32_t) K
                                            + (uint32_t) (dma_j * 32 + (((lane & 3) ^ frag_swizzle(lane >> 4)) * 8)))
                            * 2u;
                    }
                    else
                        tile_oob = kOob;
                }
                compute(std::false_type{}, a_buf1, st1, st0, a_buf0, 0);
            }
            if constexpr (GROUP == 0)
            {
#pragma unroll
                for (int s = 0; s < NS; ++s)
                {
                    pc_scale[s] = pc_scale_n[s];
                    pc_scale2[s] = pc_scale2_n[s];
                }
            }
        } while (!tile_oob);
        // the last tile's outputs
        mma_drain();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int s = 0; s < NS; ++s)
                store_block(rt, s);
        return;
    }

    // ---- epilogue: out = T(alpha * acc + bias), or partial sums into the float32 buffer --------
    mma_drain();
    if constexpr (SPLITK)
    {
        // plain orientation: acc[rt][s][r] = (row m0 + rt*16 + kg*4 + r, column strip*16 + c);
        // this K slice's own slab of the partial buffer (a slice past the end of K stores zeros)
        float* const slab = p.partial + (size_t) blockIdx.y * ((size_t) p.m * p.n);
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                {
                    int const row = m0 + rt * 16 + kg * 4 + r;
                    if (strip_ok[s] && row < p.m)
                        slab[(size_t) row * p.n + strip_of[s] * 16 + c] = acc[rt][s][r];
                }
        return;
    }
    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    int const n_out = gated ? p.n / 2 : p.n;
    // acc[rt][s][r] = output (row m0 + rt*16 + c, column strip*16 + kg*4 + r): four consecutive
    // columns per lane, moved as one 8-byte access (output, bias and residual alike).
    // The residual is read through a descriptor (rows >= m read zeros, so no branches) and one row
    // tile at a time, all loads of the tile in flight before the first is used.
    auto const res_rsrc = make_rsrc(p.residual ? p.residual : p.out, (uint32_t) p.m * (uint32_t) n_out * 2u);
    auto load4 = [&](void const* base, int col) -> f32x4 // four consecutive 16-bit values as floats
    {
        u32x2 const v = *reinterpret_cast<u32x2 const*>(static_cast<uint16_t const*>(base) + col);
        return f32x4{E::lo(v[0]), E::hi(v[0]), E::lo(v[1]), E::hi(v[1])};
    };
    auto store4 = [&](int row, int col, f32x4 v)
    {
        u32x2 const o = {E::pack(v[0], v[1]), E::pack(v[2], v[3])};
        // the output pointer may have been computed (grouped problems): tell the compiler it is
        // global memory, or it falls back to flat stores
        typedef __attribute__((address_space(1))) u32x2 global_u32x2;
        *(global_u32x2*) (out16 + (size_t) row * n_out + col) = o;
    };
    auto residual4 = [&](int row, int col) -> f32x4
    {
        u32x2 const v = buffer_load_x2(res_rsrc, ((uint32_t) row * (uint32_t) n_out + (uint32_t) col) * 2u);
        return f32x4{E::lo(v[0]), E::hi(v[0]), E::lo(v[1]), E::hi(v[1])};
    };
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};
    if (gated)
    {
        // value and gate sums of an output element sit in neighbouring strip slots of this lane
        if constexpr (!SPLITK)
        {
            // (two instantiations each: without a residual the loop holds no loads at all, so that no
            // wait for a load - which would also wait for the stores before it - sits between stores)
            auto gated_epilogue = [&](auto act_tag, auto residual_tag)
            {
                constexpr int ACT = decltype(act_tag)::value;
                constexpr bool RESIDUAL = decltype(residual_tag)::value;
                int col[NS / 2];
                f32x4 bias_x[NS / 2], bias_g[NS / 2];
#pragma unroll
                for (int i = 0; i < NS / 2; ++i)
                {
                    col[i] = strip_of[2 * i] * 16 + kg * 4; // strip_of[even slot] is the pair index (value half)
                    bias_x[i] = p.bias ? load4(p.bias, col[i]) : zero4;
                    bias_g[i] = p.bias ? load4(p.bias, col[i] + n_out) : zero4;
                }
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                {
                    int const row = m0 + rt * 16 + c;
                    f32x4 res[NS / 2];
#pragma unroll
                    for (int i = 0; i < NS / 2; ++i)
                        res[i] = RESIDUAL ? residual4(row, col[i]) : zero4;
#pragma unroll
                    for (int i = 0; i < NS / 2; ++i)
                    {
                        if (!strip_ok[2 * i] || row >= p.m)
                            continue;
                        f32x4 v;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            v[r] = (acc[rt][2 * i][r] + bias_x[i][r]) * apply_act(ACT, acc[rt][2 * i + 1][r] + bias_g[i][r])
                                + res[i][r];
                        store4(row, col[i], v);
                    }
                }
            };
            bool const swiglu = p.activation == kActSwiglu;
            if (p.residual)
                swiglu ? gated_epilogue(std::integral_constant<int, kActSwiglu>{}, std::true_type{})
                       : gated_epilogue(std::integral_constant<int, kActGeglu>{}, std::true_type{});
            else
                swiglu ? gated_epilogue(std::integral_constant<int, kActSwiglu>{}, std::false_type{})
                       : gated_epilogue(std::integral_constant<int, kActGeglu>{}, std::false_type{});
        }
        return;
    }
    int col[NS];
    f32x4 bias[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        col[s] = strip_of[s] * 16 + kg * 4;
        bias[s] = (!SPLITK && p.bias) ? load4(p.bias, col[s]) : zero4;
    }
    auto plain_epilogue = [&](auto residual_tag)
    {
    constexpr bool RESIDUAL = decltype(residual_tag)::value;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
    {
        int const row = m0 + rt * 16 + c;
        f32x4 res[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s)
            res[s] = RESIDUAL ? residual4(row, col[s]) : zero4;
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            if (!strip_ok[s] || row >= p.m)
                continue;
            f32x4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[r] = __builtin_fmaf(p.alpha, acc[rt][s][r], bias[s][r]) + res[s][r];
            store4(row, col[s], v);
        }
    }
    };
    if (!SPLITK && p.residual)
        plain_epilogue(std::true_type{});
    else
        plain_epilogue(std::false_type{});
}

template <int DT, int BITS, int GROUP, bool ZERO, int RT, int NS = 4>
int launch_gemm_variant(GemmParams const& gp, hipStream_t stream)
{
    static_assert(NS == 4 || RT == 16, "192-column tiles exist for the 256-row kernel only");
    int const total = gp.tiles_m * gp.tiles_n;
    dim3 grid(((total + 7) / 8) * 8, gp.k_splits), block(256);
    if (gp.k_splits > 1)
    {
        size_t const count = (size_t) gp.m * gp.n;
        note_launch("gemm exact rt=%d splits=%d persistent=0", RT, gp.k_splits);
        hipLaunchKernelGGL((gemm_kernel<DT, BITS, GROUP, ZERO, RT, true>), grid, block, 0, stream, gp);
        hipLaunchKernelGGL((gemm_finish_partial<DT>), dim3((unsigned) ((count / 4 + 255) / 256)), block, 0, stream,
            gp.out, gp.partial, gp.bias, gp.alpha, gp.m, gp.n, gp.k_splits);
    }
    else
    {
        // prefill-sized problems: one persistent workgroup per CU when that means at least two tiles each
        int const cus = gemm_persistent_workgroups();
        bool persist = false;
        if constexpr (RT == 16)
            persist = cus > 0 && total > cus && gp.k_tiles % 2 == 0 && gp.k_tiles >= 4 && gp.n % (NS * 64) == 0
                && !gp.bias && !gp.expert_rows && gp.num_experts == 0 && gp.activation == kActIdentity && !gp.residual
                && (uint64_t) gp.m * (uint64_t) gp.n * 2 < ((uint64_t) 1 << 31)
                // byte offsets of the padded last row tile, and of the rejected offset plus 15 row tiles, stay below 2^32
                && (uint64_t) gp.tiles_m * (RT * 16) * (uint64_t) gp.n * 2 < ((uint64_t) 1 << 32) && gp.n < (1 << 22);
        note_launch("gemm exact rt=%d splits=1 persistent=%d columns=%d", RT, (int) persist, NS * 64);
        if (persist)
        {
            if constexpr (RT == 16)
                hipLaunchKernelGGL((gemm_kernel<DT, BITS, GROUP, ZERO, RT, false, true, NS>), dim3(cus), block, 0, stream, gp);
        }
        else
            hipLaunchKernelGGL((gemm_kernel<DT, BITS, GROUP, ZERO, RT, false, false, NS>), grid, block, 0, stream, gp);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "gemm kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int DT, int BITS, int GROUP, bool ZERO>
int launch_gemm_rt(GemmParams const& gp, int rt, hipStream_t s)
{
    switch (rt)
    {
    case 4: return launch_gemm_variant<DT, BITS, GROUP, ZERO, 4>(gp, s);
    case 8: return launch_gemm_variant<DT, BITS, GROUP, ZERO, 8>(gp, s);
    default:
        if (gp.tile_cols == 192)
            return launch_gemm_variant<DT, BITS, GROUP, ZERO, 16, 3>(gp, s);
        return launch_gemm_variant<DT, BITS, GROUP, ZERO, 16>(gp, s);
    }
}

template <int DT, int BITS>
int launch_gemm_typed(MatmulProblem const& p, GemmPlan const& plan, void* stream)
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
    gp.tiles_m = (p.m + plan.rt * 16 - 1) / (plan.rt * 16);
    gp.tiles_n = (p.n + kGemmBN - 1) / kGemmBN;
    // 192-column tiles where 256-column ones leave the last round over the CUs mostly empty (256-row
    // tiles, whole K per workgroup): a 192-column tile costs about 0.8 of a 256-column one
    if (plan.rt == 16 && plan.k_splits == 1 && !act_is_gated(p.activation) && !p.expert_rows && p.n % 192 == 0)
    {
        int const cus = gemm_persistent_workgroups() > 0 ? gemm_persistent_workgroups() : 256;
        int const t256 = gp.tiles_m * gp.tiles_n, t192 = gp.tiles_m * (p.n / 192);
        int const forced = env_overrides().gemm_cols; // WOQ_GEMM_COLS=192|256
        if (forced ? forced == 192 : 0.8 * ((t192 + cus - 1) / cus) < 1.0 * ((t256 + cus - 1) / cus) - 1e-9)
        {
            gp.tile_cols = 192;
            gp.tiles_n = p.n / 192;
        }
    }
    gp.k_splits = plan.k_splits;
    gp.tiles_per_split = (gp.k_tiles + plan.k_splits - 1) / plan.k_splits;
    gp.tiles_per_split += gp.tiles_per_split & 1; // the main loop walks tile rows in pairs
    gp.partial = static_cast<float*>(p.workspace);
    if (plan.k_splits > 1 && (!p.workspace || p.workspace_bytes < plan.ws_bytes))
        return fail(WOQ_ERR_WORKSPACE, "split-K needs %zu workspace bytes", plan.ws_bytes);
    set_group_fields(gp, p, plan.rt * 16);
    auto s = static_cast<hipStream_t>(stream);
    bool const zero = p.zeros != nullptr;
    switch (template_group(p.group_size))
    {
    case 0: return launch_gemm_rt<DT, BITS, 0, false>(gp, plan.rt, s);
    case 64:
        return zero ? launch_gemm_rt<DT, BITS, 64, true>(gp, plan.rt, s)
                    : launch_gemm_rt<DT, BITS, 64, false>(gp, plan.rt, s);
    case 128:
        return zero ? launch_gemm_rt<DT, BITS, 128, true>(gp, plan.rt, s)
                    : launch_gemm_rt<DT, BITS, 128, false>(gp, plan.rt, s);
    case kFlexGroup:
        return zero ? launch_gemm_rt<DT, BITS, kFlexGroup, true>(gp, plan.rt, s)
                    : launch_gemm_rt<DT, BITS, kFlexGroup, false>(gp, plan.rt, s);
    default: return fail(WOQ_ERR_UNSUPPORTED, "group_size %d", p.group_size);
    }
}

} // namespace woq
