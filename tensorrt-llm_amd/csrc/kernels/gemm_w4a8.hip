// W4A8: fp8 (e4m3) activations x int4 weights on the CDNA4 fp8 matrix core.
//
// Semantics of the reference's W4A8 path (fpA_intB runner instantiated for __nv_fp8_e4m3 x uint4
// with half scales, cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h,
// selected by weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): the int4 weight is dequantized
// with fp16 scales/zeros and rounded to e4m3, the MMA accumulates fp8 x fp8 products in float32,
// and the epilogue applies alpha and the bias: out = T(alpha * acc + bias).  Group sizes: 128 and its
// multiples (the reference's pre-Hopper launcher takes 128 only, fpA_intB_gemm_template.h:136-142; its
// Hopper launcher any multiple of the K tile, launchers/fpA_intB_launcher_sm90.inl:190-198).
//
// Same skeleton as the 16-bit prefill kernel (gemm_kernel.h): output tile 16*RT rows x 256
// columns, 4 wavefronts side by side along N with 64 columns each; packed weights go global ->
// registers and are dequantized once per workgroup; the activation tile is DMA-ed
// global -> LDS, double-buffered; the requests of the next step and the conversions are spread
// between the MFMAs; skinny problems split K through the float32 partial buffer.
// The matrix instruction is the CDNA4 v_mfma_f32_16x16x128_f8f6f4 (e4m3 x e4m3): one instruction
// covers a whole 128-deep tile row, twice the rate of the 16x16x32 fp8 form and a quarter of its
// issue slots.  A lane supplies 32 k-values of its row / column; which 32 is free as long as A
// and B agree, so lane (kg, c) keeps the tile layout's own order - its 8 weights of slab 0, of
// slab 1, ... (k = 32 j + 8 kg + e) - and reads the matching four 8-byte pieces of its activation
// row from LDS.
// An fp8 activation fragment is half the size of a 16-bit one, so LDS holds fragment PAIRS: 16
// rows x 64 k = 1 KiB, written by one DMA instruction (lane 4r+q fetches row r's 16-byte chunk
// q ^ (r>>2): quads read 64 contiguous bytes, the XOR spreads an MFMA lane group over the banks).
#include "gemm_common.h"
#include "w4a8_common.h"

namespace woq
{

// PERSIST (256-row tiles, whole K, bf16 output, no bias): one workgroup per CU walks tiles b, b + grid, ...
// as the 16-bit prefill kernel does (gemm_kernel.h): the last two steps of a tile already request the
// first weights and the first A tile of the next one, and a finished tile's outputs are read out of
// the accumulators, scaled, packed and stored right before the matrix instruction that starts each
// block's new sum.  The 8 us or so that a tile spends outside its main loop (first loads, the
// conversion of the first operand set, 128 KiB of stores, the relaunch) weigh twice as much here as
// there: a tile's main loop is half as long.
template <int ODT, bool ZERO, int RT, bool SPLITK, bool PERSIST = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) gemm_w4a8_kernel(GemmParams p)
{
    static_assert(!PERSIST || (RT == 16 && !SPLITK && ODT == WOQ_BF16), "persistent form: 256-row tiles, whole K, bf16 out");
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    constexpr int TK = 128, SLABS = 4, NS = 4;
    constexpr int BM = RT * 16;
    constexpr int PAIRS = RT * 2;      // fragment pairs (1 KiB) of one A tile
    constexpr int A_BYTES = BM * TK;   // e4m3: one byte per element
    static_assert(PAIRS % 4 == 0, "fragment pairs spread evenly over the 4 wavefronts");

    __shared__ u32x4 a_buf0[A_BYTES / 16];
    __shared__ u32x4 a_buf1[A_BYTES / 16];

    // Tile of virtual block vb (the block index, or with PERSIST the block index plus a multiple of the
    // grid size, which is a multiple of 8): XCD-contiguous chunks of the tile order, m fastest inside
    // groups of 4 m-tiles - the 32 workgroups of an XCD then cover about 4 x 8 tiles and share 4
    // activation panels and 8 weight panels in its L2 instead of all 16 activation panels and 2
    int const total = p.tiles_m * p.tiles_n;
    int const per_xcd = (total + 7) / 8;
    auto tile_of = [&](int vb, int& tm_, int& tn_) -> bool
    {
        int const t = (vb & 7) * per_xcd + (vb >> 3);
        if ((vb >> 3) >= per_xcd || t >= total)
            return false;
        constexpr int kGroupM = 4;
        int const in_group = kGroupM * p.tiles_n;
        int const first_m = (t / in_group) * kGroupM;
        int const gsz = p.tiles_m - first_m < kGroupM ? p.tiles_m - first_m : kGroupM;
        tm_ = first_m + (t % in_group) % gsz;
        tn_ = (t % in_group) / gsz;
        return true;
    };
    int vb = (int) blockIdx.x;
    int tm, tn;
    if (!tile_of(vb, tm, tn))
        return;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const K = p.k;
    int const kt_begin = SPLITK ? (int) blockIdx.y * p.tiles_per_split : 0;
    int const KT = SPLITK ? (kt_begin + p.tiles_per_split < p.k_tiles ? kt_begin + p.tiles_per_split : p.k_tiles)
                          : p.k_tiles;
    int m0 = tm * BM;
    int strip0 = tn * (kGemmBN / 16) + wave * NS;

    constexpr uint32_t kOob = 0x80000000u;
    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K);
    uint32_t const sz_bytes = (uint32_t) p.scale_rows * (uint32_t) p.n * 2u;
    uint32_t const magic = p.group_magic; // groups above 128: table row of a tile row (w4a8_scale_row)
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) p.k_tiles * 1024u);

    // per-lane request addresses of one tile (PERSIST keeps those of the next tile beside them)
    struct TileCtx
    {
        uint32_t wlane[NS], sc_lane[NS];
        uint32_t dma_lane_base;
        uint32_t oob; // kOob: there is no such tile, every request reads zeros
    };
    auto make_ctx = [&](int tm_, int tn_, bool valid) -> TileCtx
    {
        TileCtx x;
        int const first = tn_ * (kGemmBN / 16) + wave * NS;
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            int const strip = first + s < p.strips ? first + s : p.strips - 1;
            x.wlane[s] = ((uint32_t) strip * (uint32_t) p.k_tiles * 64u + (uint32_t) lane) * 16u;
            x.sc_lane[s] = (uint32_t) (strip * 16 + c) * 2u;
        }
        // A tile -> LDS: wavefront w moves pairs w, w+4, ...: piece i is pair f = w + 4i = half w % 2 of
        // row tile 2i + w / 2
        x.dma_lane_base = (uint32_t) (tm_ * BM + (wave / 2) * 16 + (lane >> 2)) * (uint32_t) K
            + (uint32_t) ((wave % 2) * 64 + (((lane & 3) ^ ((lane >> 4) & 3)) * 16));
        x.oob = valid ? 0u : 0x80000000u;
        return x;
    };
    TileCtx cur = make_ctx(tm, tn, true);

    f32x4 acc[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc[rt][s] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- A tile -> LDS; K is a multiple of 128, so only kt >= KT falls out of range (rows past M fall
    // outside the descriptor by themselves).
    constexpr int DMA_OPS = PAIRS / 4;
    uint32_t const dma_piece_stride = 32u * (uint32_t) K;
    auto dma_base = [&](int kt, TileCtx const& x) -> uint32_t
    { return (x.dma_lane_base + (uint32_t) kt * (uint32_t) TK) | ((uint32_t) (KT - 1 - kt) & kOob) | x.oob; };
    auto dma_piece = [&](auto* buf, uint32_t base, int i)
    {
        int const f = wave + i * 4;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(act_rsrc,
            (__attribute__((address_space(3))) void*) (reinterpret_cast<char*>(buf) + f * 1024), 16,
            (int) (base + (uint32_t) i * dma_piece_stride), 0, 0, 0);
    };
    // MFMA lane (kg, c), slab j = 2*jp + jj of row tile rt: row c, bytes jj*32 + kg*8 .. +8 of the
    // pair's 64: chunk jj*2 + kg/2 (stored at position chunk ^ (c>>2)), half kg & 1
    uint32_t a_lane_off[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
        a_lane_off[jj] = (uint32_t) ((c * 4 + ((jj * 2 + (kg >> 1)) ^ ((c >> 2) & 3))) * 16 + (kg & 1) * 8);

    struct BStage
    {
        u32x4 w[NS];
        uint16_t s[NS];
        uint16_t z[NS];
    };
    constexpr int FETCH_OPS = NS * (ZERO ? 3 : 2);
    auto fetch_piece = [&](BStage& st, int kt, int i, TileCtx const& x)
    {
        uint32_t const past = ((uint32_t) (KT - 1 - kt) & kOob) | x.oob; // kt >= KT: every load of the step reads zeros
        if (i < NS)
            st.w[i] = buffer_load_x4(w_rsrc, x.wlane[i] + ((uint32_t) kt * 1024u | past));
        else
        {
            int const s = (i - NS) % NS;
            uint32_t const off = (w4a8_scale_row((uint32_t) kt, magic) * (uint32_t) p.n * 2u + x.sc_lane[s]) | past;
            if (i < 2 * NS)
                st.s[s] = buffer_load_u16(sc_rsrc, off);
            else
                st.z[s] = buffer_load_u16(zr_rsrc, off);
        }
    };

    // ---- one step = one tile row of K = RT iterations of 4 MFMAs (one per strip).  Iteration rt
    // issues the activation reads of the row tile A_AHEAD ahead, its share of the memory requests
    // (packed weights of step kt+2, A tile of step kt+1) and of the conversions that build the B
    // operands of step kt+1 (32 half-operands of 4 weights), then the 4 MFMAs of row tile rt.
    constexpr int A_AHEAD = 2;
    auto slab_at = [](int pos) { return ((pos & 1) << 1) | (pos >> 1); }; // its own inverse
    // conversion unit cu = (strip, slab, half, pair): 2 weights -> 16 bits of the operand set.  The
    // same arithmetic as dequant2_fp8 (w4a8_common.h), cut into four stages so that the main loop can
    // run each stage of a unit behind a different matrix instruction: issued back to back, every
    // instruction of the chain mask -> byte-to-float -> FMA -> pack waits for the one before it.
    NibbleConsts const nib = nibble_consts<WOQ_FP16>(); // 0x000F000F in an SGPR, 0x64006400 (1024 as a pair of halves) in a VGPR
    struct ConvState
    {
        uint32_t src[2][2]; // zero-points: sign-flipped source word of (slab parity, pair)
        uint32_t pw[16];    // no zero-points: the unit's two nibbles as a pair of halves 1024 + u (1024 + 16 u for pr = 1)
        uint32_t sh;        // no zero-points: the slab word shifted by 8 (made by the unit h = 1, pr = 0 for both pairs)
        float v[16][2];     // the two values of the units in flight (unit % 16: at most 12 are)
    };
    auto conv_stage = [&](ConvState& cs, u32x8 (&b)[NS], BStage const& st, int cu, int stage)
    {
        int const s = cu / 16, j = (cu / 4) % 4, h = (cu / 2) % 2, pr = cu % 2;
        float(&v)[2] = cs.v[cu % 16];
        if constexpr (ZERO)
        {
            // fma(q, s, z) on the two's-complement nibble: q/16 straight from the nibble, times 16 s
            uint32_t& src = cs.src[j & 1][pr];
            if (stage == 0)
            {
                if (h != 0)
                    return; // the unit with h = 0 made the word for both
                uint32_t const w = st.w[s][j] ^ 0x88888888u; // biased -> two's complement nibbles
                src = pr == 0 ? w : (w >> 4);
                // (here and below: an anchor in the order of the volatile statements, i.e. of the matrix
                // instructions - the next stage's instructions cannot be moved up to this one's)
                asm volatile("" : "+v"(src));
            }
            else if (stage == 1)
            {
                v[0] = cvt_off_f32_i4_byte(src, h);
                v[1] = cvt_off_f32_i4_byte(src, h + 2);
                asm volatile("" : "+v"(v[0]), "+v"(v[1]));
            }
            else if (stage == 2)
            {
                float const sc = EH::from_bits(st.s[s]), zr = EH::from_bits(st.z[s]);
                v[0] = __builtin_fmaf(v[0], 16.f * sc, zr);
                v[1] = __builtin_fmaf(v[1], 16.f * sc, zr);
                asm volatile("" : "+v"(v[0]), "+v"(v[1]));
            }
        }
        else
        {
            // q s = fma(1024 + u, s, -1032 s) on the stored nibble u = q + 8: elements e0 = 4h + 2pr and
            // e0 + 1 sit in nibbles e0/2 and e0/2 + 4, i.e. 16 bits apart - one and-or makes the pair
            // of halves 0x6400 | u = 1024 + u, which the FMA reads directly.  The pair pr = 1 is taken
            // where it sits, four bits up (still inside a half's ten fraction bits): 1024 + 16 u, and
            // q s = fma(1024 + 16 u, s / 16, -72 s); so only the units of h = 1 need a shift, one for
            // both.  The constants and the result (15 significant bits) are exact in float32: the same
            // single rounding to e4m3 as fma(q, s, 0).
            uint32_t& pw = cs.pw[cu % 16];
            if (stage == 0)
            {
                if (h == 1 && pr == 0)
                {
                    cs.sh = st.w[s][j] >> 8;
                    asm volatile("" : "+v"(cs.sh));
                }
                uint32_t const src = h == 0 ? st.w[s][j] : cs.sh;
                pw = (src & (pr == 0 ? nib.mask : nib.mask << 4)) | nib.magic; // one v_and_or_b32
                asm volatile("" : "+v"(pw));
            }
            else if (stage == 2)
            {
                float const sc = EH::from_bits(st.s[s]);
                f16x2 const pair = bit_cast<f16x2>(pw);
                float const mul = pr == 0 ? sc : 0.0625f * sc, add = pr == 0 ? -1032.f * sc : -72.f * sc;
                v[0] = __builtin_fmaf((float) pair[0], mul, add);
                v[1] = __builtin_fmaf((float) pair[1], mul, add);
                asm volatile("" : "+v"(v[0]), "+v"(v[1]));
            }
        }
        if (stage == 3)
        {
            int const idx = slab_at(j) * 2 + h; // slab j sits at operand position slab_at(j)
            b[s][idx] = pr == 0 ? (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], (int) b[s][idx], false)
                                : (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], (int) b[s][idx], true);
        }
    };
    // all four stages of one unit at once (prologue)
    auto convert_unit = [&](u32x8 (&b)[NS], BStage const& st, int cu)
    {
        int const s = cu / 16, j = (cu / 4) % 4, h = (cu / 2) % 2, pr = cu % 2;
        int const idx = slab_at(j) * 2 + h;
        float const sc = EH::from_bits(st.s[s]);
        float const zr = ZERO ? EH::from_bits(st.z[s]) : 0.f;
        b[s][idx] = dequant2_fp8<ZERO, false>(b[s][idx], st.w[s][j], h, pr, sc, zr);
    };
    constexpr int UNITS = NS * SLABS * 4; // 64 per step

    // PERSIST: where the finished tile's outputs go: byte offset of (row m0 + c, column strip0 * 16 + kg * 4)
    // of the tile to store (N is a multiple of the tile width: every strip exists; rows past M fall
    // outside the descriptor); kOob: no finished tile yet
    [[maybe_unused]] auto const out_rsrc = make_rsrc(p.out, (uint32_t) p.m * (uint32_t) p.n * 2u);
    [[maybe_unused]] uint32_t prev_off = kOob;
    [[maybe_unused]] uint32_t const rt_stride = 16u * (uint32_t) p.n * 2u;
    auto store_block = [&](int rt, int s)
    {
        // explicit AGPR-source moves: a plain VALU use of the block would pull every accumulator into the
        // VGPR half of the file for the whole loop.  The pack to bf16 does not depend on the conversion
        // mode the main loop runs in (that concerns fp16 and fp8 results only).
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[r]) : "a"(acc[rt][s][r]));
        u32x2 const o = {EO::pack(p.alpha * v[0], p.alpha * v[1]), EO::pack(p.alpha * v[2], p.alpha * v[3])};
        __builtin_amdgcn_raw_buffer_store_b64(o, out_rsrc, (int) (prev_off + (uint32_t) rt * rt_stride + (uint32_t) s * 32u), 0, 0);
    };

    // One step.  The A tile of step kt_a of tile xa goes to buf_next, the packed weights of step kt_w of
    // tile xw to st_req (the steps after this one and after the next: the same tile's, or with PERSIST
    // the next tile's first ones).  first_tag: the first step of a tile in the persistent loop.
    auto compute = [&](auto first_tag, auto const* buf, u32x8 const (&b_use)[NS], u32x8 (&b_make)[NS],
                       BStage const& st_conv, BStage& st_req, auto* buf_next, int kt_a, TileCtx const& xa, int kt_w,
                       TileCtx const& xw)
    {
        constexpr bool FIRST = decltype(first_tag)::value;
        char const* a_base = reinterpret_cast<char const*>(buf);
        uint32_t const next_base = dma_base(kt_a, xa);
        auto a_read = [&](int rt) -> u32x8
        {
            // operand position pos holds slab slab_at(pos) = 0, 2, 1, 3: the two pieces that sit
            // 1 KiB apart in LDS (same half of the two fragment pairs) come from one two-address read
            u32x8 a;
#pragma unroll
            for (int pos = 0; pos < SLABS; ++pos)
            {
                int const j = slab_at(pos);
                u32x2 const v = *reinterpret_cast<u32x2 const*>(a_base + (rt * 2 + j / 2) * 1024 + a_lane_off[j % 2]);
                a[2 * pos] = v[0];
                a[2 * pos + 1] = v[1];
            }
            return a;
        };
        u32x8 a_ring[A_AHEAD + 1];
#pragma unroll
        for (int i = 0; i < A_AHEAD && i < RT; ++i)
            a_ring[i] = a_read(i);
        // the conversion pipeline's head: the stages that the first matrix instructions expect done
        constexpr int PER0 = UNITS / (RT * NS);
        ConvState cs;
        constexpr bool PIPELINED = RT >= 8; // (64-row tiles measured 2-8 % faster without the stage pipeline, 128-row tiles 3-6 % slower)
#pragma unroll
        for (int lead = 0; PIPELINED && lead < 3; ++lead)
#pragma unroll
            for (int stage = 0; stage < 3 - lead; ++stage)
#pragma unroll
                for (int x = 0; x < PER0; ++x)
                    if (lead * PER0 + x < UNITS)
                        conv_stage(cs, b_make, st_conv, lead * PER0 + x, stage);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
        {
            // the A-tile DMAs first, the weight-side requests of step kt+2 after them: the barrier
            // that ends the step then waits for the DMAs only (vector-memory operations retire in
            // order) and leaves the weight loads, which travel from HBM, a whole further step
            constexpr int DMA_WINDOW = RT / 2 > 0 ? RT / 2 : 1;
#pragma unroll
            for (int q = 0; q < DMA_OPS; ++q)
                if (q * DMA_WINDOW / DMA_OPS == rt)
                    dma_piece(buf_next, next_base, q);
            constexpr int FETCH_FIRST = RT / 2, FETCH_WINDOW = RT - RT / 2 - 1 > 0 ? RT - RT / 2 - 1 : 1;
#pragma unroll
            for (int q = 0; q < FETCH_OPS; ++q)
                if (FETCH_FIRST + q * FETCH_WINDOW / FETCH_OPS == rt)
                    fetch_piece(st_req, kt_w, q, xw);
            if (rt + A_AHEAD < RT)
                a_ring[(rt + A_AHEAD) % (A_AHEAD + 1)] = a_read(rt + A_AHEAD);
            u32x8 const a_cur = a_ring[rt % (A_AHEAD + 1)];
            // one MFMA, then its share of the conversions: a wavefront issues in order, so the
            // VALU work has to sit between the matrix instructions to run under them
#pragma unroll
            for (int s = 0; s < NS; ++s)
            {
                // weights as the first operand: the accumulator holds the TRANSPOSED 16x16 block, lane
                // (kg, c) the four consecutive columns kg*4 .. kg*4+3 of output row c (8-byte epilogue accesses)
                // (the split-K variant keeps the plain orientation: its float32 stores cover 64 consecutive
                // bytes per row and instruction)
                if constexpr (SPLITK)
                    mma_fp8_acc(a_cur, b_use[s], acc[rt][s]);
                else if constexpr (FIRST)
                {
                    store_block(rt, s); // the previous tile's sums leave right before the block starts the new tile's
                    mma_fp8_first(b_use[s], a_cur, acc[rt][s]);
                }
                else
                    mma_fp8_acc(b_use[s], a_cur, acc[rt][s]);
                // behind matrix instruction t: the pack of the units whose FMAs went behind t - 1, the
                // FMAs of those converted behind t - 2, and so on (PER units per instruction)
                constexpr int PER = UNITS / (RT * NS);
                int const t = rt * NS + s;
                if constexpr (PIPELINED)
                {
#pragma unroll
                    for (int stage = 3; stage >= 0; --stage)
#pragma unroll
                        for (int x = 0; x < PER; ++x)
                        {
                            int const cu = (t + 3 - stage) * PER + x;
                            if (cu < UNITS)
                                conv_stage(cs, b_make, st_conv, cu, stage);
                        }
                }
                else
                {
                    // fewer row tiles: several units per matrix instruction, independent of each other -
                    // each goes through its four stages here
#pragma unroll
                    for (int x = 0; x < PER; ++x)
#pragma unroll
                        for (int stage = 0; stage < 4; ++stage)
                            conv_stage(cs, b_make, st_conv, t * PER + x, stage);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // ---- main loop: two steps per iteration so that LDS buffers, operand sets and weight stages
    // are distinct objects.  Step kt multiplies with operand set kt%2 (converted during step kt-1
    // from weight stage kt%2), converts set (kt+1)%2 from stage (kt+1)%2 and refills stage kt%2
    // with the packed weights of step kt+2.  (Requesting the weights a further step ahead - four
    // stages - measured the same.)
    BStage st0, st1;
    u32x8 b0[NS], b1[NS];
    fp8_saturation_on(); // the conversions rely on it; off again before the epilogue
#pragma unroll
    for (int s = 0; s < NS; ++s)
        b0[s] = b1[s] = u32x8{0, 0, 0, 0, 0, 0, 0, 0};
    {
        uint32_t const base = dma_base(kt_begin, cur);
#pragma unroll
        for (int i = 0; i < DMA_OPS; ++i)
            dma_piece(a_buf0, base, i);
    }
#pragma unroll
    for (int i = 0; i < FETCH_OPS; ++i)
        fetch_piece(st0, kt_begin, i, cur);
#pragma unroll
    for (int i = 0; i < FETCH_OPS; ++i)
        fetch_piece(st1, kt_begin + 1, i, cur);
#pragma unroll
    for (int cu = 0; cu < UNITS; ++cu)
        convert_unit(b0, st0, cu);
    // A(kt) has landed for every wavefront (at most the FETCH_OPS weight-side loads issued after its
    // DMAs are still outstanding: loads return in order, and the persistent loop's stores are older than
    // the last of them too); everyone is done reading the other buffer
    auto step_barrier = [&]() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(FETCH_OPS) : "memory"); };
    std::false_type const plain{};
    if constexpr (!PERSIST)
    {
        for (int kt = kt_begin; kt < KT; kt += 2)
        {
            step_barrier();
            compute(plain, a_buf0, b0, b1, st1, st0, a_buf1, kt + 1, cur, kt + 2, cur);
            step_barrier();
            compute(plain, a_buf1, b1, b0, st0, st1, a_buf0, kt + 2, cur, kt + 3, cur); // past the end of K both operands read as zeros
        }
    }
    else
    {
        // Straight-line first, second and last two steps around a plain inner loop (KT even, >= 4; the
        // shape the 16-bit kernel's persistent loop has, for the same reason: all 256 AGPRs are
        // accumulators, and a branch between first-step and ordinary code inside a loop makes the
        // allocator keep second copies of them).  Step kt multiplies operand set kt % 2 (buffer kt % 2),
        // converts the weights of step kt + 1 and requests those of step kt + 2 and the A tile of step
        // kt + 1 - in a tile's last two steps those are the next tile's first ones.
        bool has_next;
        do
        {
            int tmn = 0, tnn = 0;
            has_next = tile_of(vb + (int) gridDim.x, tmn, tnn);
            TileCtx const nxt = make_ctx(tmn, tnn, has_next);
            step_barrier();
            compute(std::true_type{}, a_buf0, b0, b1, st1, st0, a_buf1, 1, cur, 2, cur);
            step_barrier();
            compute(plain, a_buf1, b1, b0, st0, st1, a_buf0, 2, cur, 3, cur);
            for (int kt = 2; kt < KT - 2; kt += 2)
            {
                step_barrier();
                compute(plain, a_buf0, b0, b1, st1, st0, a_buf1, kt + 1, cur, kt + 2, cur);
                step_barrier();
                compute(plain, a_buf1, b1, b0, st0, st1, a_buf0, kt + 2, cur, kt + 3, cur);
            }
            step_barrier();
            compute(plain, a_buf0, b0, b1, st1, st0, a_buf1, KT - 1, cur, 0, nxt);
            step_barrier();
            compute(plain, a_buf1, b1, b0, st0, st1, a_buf0, 0, nxt, 1, nxt);
            // this tile's outputs: stored during the next tile's first step (or below)
            prev_off = ((uint32_t) (m0 + c) * (uint32_t) p.n + (uint32_t) (strip0 * 16 + kg * 4)) * 2u;
            vb += (int) gridDim.x;
            m0 = tmn * BM;
            strip0 = tnn * (kGemmBN / 16) + wave * NS;
            cur = nxt;
        } while (has_next);
        mma_drain();
        fp8_saturation_off();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int s = 0; s < NS; ++s)
                store_block(rt, s);
        return;
    }

    // ---- epilogue: out = T(alpha * acc + bias), or partial sums into the float32 buffer --------
    mma_drain();
    fp8_saturation_off();
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
                    if (strip0 + s < p.strips && row < p.m)
                        slab[(size_t) row * p.n + (strip0 + s) * 16 + c] = acc[rt][s][r];
                }
        return;
    }
    uint16_t* out16 = static_cast<uint16_t*>(p.out);
    // acc[rt][s][r] = output (row m0 + rt*16 + c, column strip*16 + kg*4 + r): four consecutive
    // columns per lane, written as one 8-byte store
    typedef __attribute__((address_space(1))) u32x2 global_u32x2;
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        if (strip0 + s >= p.strips)
            continue;
        int const col = (strip0 + s) * 16 + kg * 4;
        float bias[4] = {0.f, 0.f, 0.f, 0.f};
        if (!SPLITK && p.bias)
        {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                bias[r] = EO::load(p.bias, col + r);
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
        {
            int const row = m0 + rt * 16 + c;
            if (row >= p.m)
                continue;
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[r] = after_mode_change(__builtin_fmaf(p.alpha, acc[rt][s][r], bias[r]));
            u32x2 const o = {EO::pack(v[0], v[1]), EO::pack(v[2], v[3])};
            *(global_u32x2*) (out16 + (size_t) row * p.n + col) = o;
        }
    }
}

template <int ODT, bool ZERO, int RT>
int launch_w4a8_variant(GemmParams const& gp, hipStream_t stream)
{
    int const total = gp.tiles_m * gp.tiles_n;
    dim3 grid(((total + 7) / 8) * 8, gp.k_splits), block(256);
    note_launch("gemm w4a8 rt=%d splits=%d", RT, gp.k_splits);
    if (gp.k_splits > 1)
    {
        size_t const count = (size_t) gp.m * gp.n;
        hipLaunchKernelGGL((gemm_w4a8_kernel<ODT, ZERO, RT, true>), grid, block, 0, stream, gp);
        hipLaunchKernelGGL((gemm_finish_partial<ODT>), dim3((unsigned) ((count / 4 + 255) / 256)), block, 0, stream,
            gp.out, gp.partial, gp.bias, gp.alpha, gp.m, gp.n, gp.k_splits);
    }
    else
    {
        // 256-row tiles, bf16 out: one persistent workgroup per CU when that means at least two tiles each
        int const cus = gemm_persistent_workgroups();
        bool persist = false;
        if constexpr (RT == 16 && ODT == WOQ_BF16)
            persist = cus > 0 && total > cus && gp.k_tiles % 2 == 0 && gp.k_tiles >= 4 && gp.n % kGemmBN == 0 && !gp.bias
                && (uint64_t) gp.m * (uint64_t) gp.n * 2 < ((uint64_t) 1 << 31)
                // byte offsets of the padded last row tile, and of the rejected offset plus 15 row tiles, stay below 2^32
                && (uint64_t) gp.tiles_m * 256 * (uint64_t) gp.n * 2 < ((uint64_t) 1 << 32) && gp.n < (1 << 22);
        note_launch("gemm w4a8 rt=%d splits=1 persistent=%d", RT, (int) persist);
        if (persist)
        {
            if constexpr (RT == 16 && ODT == WOQ_BF16)
                hipLaunchKernelGGL((gemm_w4a8_kernel<ODT, ZERO, RT, false, true>), dim3(cus), block, 0, stream, gp);
        }
        else
            hipLaunchKernelGGL((gemm_w4a8_kernel<ODT, ZERO, RT, false>), grid, block, 0, stream, gp);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "W4A8 gemm kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int ODT, bool ZERO>
int launch_w4a8_rt(GemmParams const& gp, int rt, hipStream_t s)
{
    switch (rt)
    {
    case 4: return launch_w4a8_variant<ODT, ZERO, 4>(gp, s);
    case 8: return launch_w4a8_variant<ODT, ZERO, 8>(gp, s);
    default: return launch_w4a8_variant<ODT, ZERO, 16>(gp, s);
    }
}

int launch_gemm_w4a8(MatmulProblem const& p, void* stream)
{
    GemmPlan const plan = plan_gemm_w4a8(p.m, p.n, p.k);
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
    gp.k_tiles = (p.k + 127) / 128;
    gp.strips = p.n / kTileN;
    gp.scale_rows = (p.k + p.group_size - 1) / p.group_size;
    gp.group_magic = w4a8_scale_row_magic(p.group_size);
    gp.tiles_m = (p.m + plan.rt * 16 - 1) / (plan.rt * 16);
    gp.tiles_n = (p.n + kGemmBN - 1) / kGemmBN;
    gp.k_splits = plan.k_splits;
    gp.tiles_per_split = (gp.k_tiles + plan.k_splits - 1) / plan.k_splits;
    gp.tiles_per_split += gp.tiles_per_split & 1; // the main loop walks tile rows in pairs
    gp.partial = static_cast<float*>(p.workspace);
    if (plan.k_splits > 1 && (!p.workspace || p.workspace_bytes < plan.ws_bytes))
        return fail(WOQ_ERR_WORKSPACE, "split-K needs %zu workspace bytes", plan.ws_bytes);
    auto s = static_cast<hipStream_t>(stream);
    bool const zero = p.zeros != nullptr;
    if (p.out_dtype == WOQ_BF16)
        return zero ? launch_w4a8_rt<WOQ_BF16, true>(gp, plan.rt, s) : launch_w4a8_rt<WOQ_BF16, false>(gp, plan.rt, s);
    return zero ? launch_w4a8_rt<WOQ_FP16, true>(gp, plan.rt, s) : launch_w4a8_rt<WOQ_FP16, false>(gp, plan.rt, s);
}

} // namespace woq
