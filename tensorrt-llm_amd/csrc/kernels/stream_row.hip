// Single-row decode (M = 1, int4 weights, group scales): short-lived wavefronts in address order.
//
// Counterpart of the reference's small-M kernel at batch 1
// (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernel.h:57-118) in purpose only.  What HBM rewards on
// this part is many short-lived wavefronts that each read a few contiguous KiB, neighbours reading
// neighbouring addresses at the same time.  So: one workgroup per strip of 16 columns (its tiles are
// contiguous in the gfx950 layout), wavefront w reads the TPW consecutive 1 KiB tiles w * TPW .. of that
// strip with all its loads issued at once, and there is no staging pass and no barrier before the
// arithmetic - every wavefront fetches the few activations and scales it needs itself:
//   * lane (kg, c) of the 16x16x32 matrix instruction supplies row c of the A operand.  Row c carries the
//     activations of the wavefront's c-th group of K (c < ROWS = groups per wavefront, at most 16) and
//     nothing else, so one instruction multiplies every group's activations with one group's weights;
//     D_g = A x W_g is kept per group g and only its row g is used: no masking, no zero operands;
//   * A x ones gives the activation sum S_g of every group in the same register layout;
//   * register r of lane (kg, c) is row kg * 4 + r: that lane loads the scale and zero of groups
//     kg * 4 + r for its column c (2-byte loads, 32 contiguous bytes per group and strip) and forms
//     s * P + (z - OFFSET * s) * S in float32, as the other streaming kernels do;
//   * the wavefronts of a workgroup (different ranges of K) are added through LDS in wavefront order:
//     results are bit-reproducible.
#include "stream_kernel.h"

namespace woq
{

#ifdef WOQ_TIMELINE
// per-wavefront time stamps (100 MHz constant clock) for `bench.py --mode timeline`: a build of its own
#define WOQ_TR(i)                                                                                                      \
    do                                                                                                                 \
    {                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
        tr[i] = __builtin_amdgcn_s_memrealtime();                                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
    } while (0)
#else
#define WOQ_TR(i)                                                                                                      \
    do                                                                                                                 \
    {                                                                                                                  \
    } while (0)
#endif

// what the epilogue and the optional smoothing need: read late, off the critical path
struct RowTail
{
    void const* pqs;
    void const* bias;
    unsigned long long* trace; // WOQ_TIMELINE builds only
};

// The first fourteen dwords of the arguments are what the requests need.  They are plain scalars so that
// the wavefront finds them in SGPRs when it starts (kernel-argument preloading; this file is compiled with
// -amdgpu-kernarg-preload-count=16, of which the hardware's sixteen user SGPRs leave fourteen): a by-value
// struct is fetched with scalar loads from the argument buffer instead, 0.2-0.3 us per dependent batch,
// before the first address can be formed.
template <int DT, int GROUP, bool PQS, bool ZERO, int WAVES, int TPW, bool MULTI>
__global__ void __launch_bounds__(WAVES * 64) stream_row_kernel(void const* weight, void const* act, void const* scales,
    void const* zeros, int k_tiles, int strips, int groups_per_xcd, int n, int k, float alpha, void* out, RowTail tail)
{
    using E = Elem<DT>;
    constexpr int TK = 128;
    constexpr int SEGS = TK / GROUP, SEG_SLABS = GROUP / 32;
    constexpr int ROWS = TPW * SEGS; // groups of K per wavefront and pass = rows of the M-tile in use
    static_assert(GROUP == 64 || GROUP == 128, "group scales of 64 or 128 rows");
    static_assert(ROWS == 4 || ROWS == 8 || ROWS == 16, "whole quads of MFMA rows");
    constexpr float OFF = Offset<DT, 4>::value;
    constexpr uint32_t kOob = 0x80000000u;

#ifdef WOQ_TIMELINE
    unsigned long long tr[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#endif
    WOQ_TR(0);
    int const strip = xcd_strip(blockIdx.x, groups_per_xcd);
    if (strip >= strips)
        return; // whole workgroup leaves together

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const KT = k_tiles;
    auto const w_rsrc = make_rsrc(weight, (uint32_t) strips * (uint32_t) KT * 1024u);
    uint32_t const wlane = ((uint32_t) strip * (uint32_t) KT * 64u + (uint32_t) lane) * 16u;
    int const c = lane & 15, kg = lane >> 4;
    int const groups_k = k / GROUP;
    auto const act_rsrc = make_rsrc(act, (uint32_t) k * 2u);

    // One pass of the workgroup covers WAVES * TPW tiles of K; wavefront w takes the TPW consecutive tiles
    // w * TPW .. of it.  MULTI (K longer than one pass): the passes follow one another, each with all its
    // requests issued at once - the other resident workgroups fill the gaps.  (Two passes in flight per
    // wavefront through two register stages measured 25-50 % slower: more requests in flight per CU than
    // the memory system rewards, as with deeper prefetch in the other streaming kernels.)
    struct Stage
    {
        u32x4 w[TPW], a[SEG_SLABS], pq[PQS ? SEG_SLABS : 1];
        uint16_t s[4], z[4];
    };
    // the activations (a few hundred bytes from the L2: back before the first weights, so that each tile is
    // multiplied as it arrives) and the weights: needed first, requested before anything else is worked out
    auto fetch_operands = [&](Stage& st, int kt0)
    {
        int const g_mine = kt0 * SEGS + c; // the group whose activations this lane holds
        bool const a_ok = c < ROWS && g_mine < groups_k;
#pragma unroll
        for (int js = 0; js < SEG_SLABS; ++js)
            st.a[js] = buffer_load_x4(act_rsrc, a_ok ? (uint32_t) (g_mine * GROUP + js * 32 + kg * 8) * 2u : kOob);
#pragma unroll
        for (int i = 0; i < TPW; ++i)
            st.w[i] = buffer_load_x4(w_rsrc, kt0 + i < KT ? wlane + (uint32_t) (kt0 + i) * 1024u : kOob);
    };
    auto kt_of = [&](int pass) { return (pass * WAVES + wave) * TPW; };
    Stage st[1];
    fetch_operands(st[0], kt_of(0));
    __builtin_amdgcn_sched_barrier(0);
    WOQ_TR(1);

    auto const pqs_rsrc = make_rsrc(PQS ? tail.pqs : act, (uint32_t) k * 2u);
    uint32_t const sz_bytes = (uint32_t) groups_k * (uint32_t) n * 2u;
    auto const sc_rsrc = make_rsrc(scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? zeros : scales, sz_bytes);
    uint32_t const sc_lane = (uint32_t) (strip * 16 + c) * 2u;
    u32x4 const ones = {E::kOnes, E::kOnes, E::kOnes, E::kOnes};
    NibbleConsts const nib = nibble_consts<DT>();
    f32x4 const zero4 = {0.f, 0.f, 0.f, 0.f};
    // what the end of a pass needs: the scale and zero of groups kg * 4 + r for this lane's column (and the
    // smoothing factors of the lane's activations)
    auto fetch_scales = [&](Stage& st, int kt0)
    {
        int const g0 = kt0 * SEGS;
        if constexpr (PQS)
        {
            int const g_mine = g0 + c;
            bool const a_ok = c < ROWS && g_mine < groups_k;
#pragma unroll
            for (int js = 0; js < SEG_SLABS; ++js)
                st.pq[js] = buffer_load_x4(pqs_rsrc, a_ok ? (uint32_t) (g_mine * GROUP + js * 32 + kg * 8) * 2u : kOob);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            int const row = kg * 4 + r;
            bool const ok = row < ROWS && g0 + row < groups_k;
            uint32_t const off = ok ? (uint32_t) (g0 + row) * (uint32_t) n * 2u + sc_lane : kOob;
            st.s[r] = buffer_load_u16(sc_rsrc, off);
            st.z[r] = ZERO ? buffer_load_u16(zr_rsrc, off) : (uint16_t) 0;
        }
    };
    fetch_scales(st[0], kt_of(0));
    __builtin_amdgcn_sched_barrier(0);
    WOQ_TR(2);

    float total = 0.f; // this lane's share of output column c
    auto compute = [&](Stage& st)
    {
        // ---- products: D_g = A x W_g for every group g of the pass, S = A x ones ----
        f32x4 acc[TPW][SEGS], acc_s = zero4;
#pragma unroll
        for (int js = 0; js < SEG_SLABS; ++js)
        {
            if constexpr (PQS)
            {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    st.a[js][r] = E::mul2(st.a[js][r], st.pq[js][r]);
            }
            acc_s = E::mma(st.a[js], ones, acc_s);
        }
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int seg = 0; seg < SEGS; ++seg)
            {
                acc[i][seg] = zero4;
#pragma unroll
                for (int js = 0; js < SEG_SLABS; ++js)
                    acc[i][seg] = E::mma(st.a[js], expand_int4<DT>(st.w[i][seg * SEG_SLABS + js], nib), acc[i][seg]);
            }
        // ---- row kg * 4 + r of D_(kg * 4 + r), scaled ----
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float P = 0.f;
#pragma unroll
            for (int q = 0; q < ROWS / 4; ++q)
            {
                int const g = q * 4 + r;
                float const v = acc[g / SEGS][g % SEGS][r];
                P = kg == q ? v : P;
            }
            float const sc = E::from_bits(st.s[r]);
            float const cc = __builtin_fmaf(-OFF, sc, ZERO ? E::from_bits(st.z[r]) : 0.f);
            total = __builtin_fmaf(sc, P, __builtin_fmaf(cc, acc_s[r], total));
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

    // ---- rows (lanes kg) of a wavefront, then the wavefronts, in fixed order ----
    WOQ_TR(6);
    total += __shfl_xor(total, 16);
    total += __shfl_xor(total, 32);
    __shared__ float red[WAVES][16];
    if (kg == 0)
        red[wave][c] = total;
    WOQ_TR(7);
    __syncthreads();
    WOQ_TR(8);
    if (threadIdx.x < 16)
    {
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][c];
        int const ocol = strip * 16 + c;
        float v = alpha * sum;
        if (tail.bias)
            v += E::load(tail.bias, ocol);
        static_cast<uint16_t*>(out)[ocol] = E::store(v);
    }
#ifdef WOQ_TIMELINE
    WOQ_TR(9);
    if (tail.trace && lane == 0)
    {
        unsigned long long* t = tail.trace + ((size_t) blockIdx.x * WAVES + wave) * 10;
        for (int i = 0; i < 10; ++i)
            t[i] = tr[i];
    }
#endif
}

namespace
{
template <int DT, int GROUP, bool PQS, bool ZERO, int WAVES, int TPW>
int launch_row_variant(StreamParams sp, hipStream_t stream)
{
    bool const multi = sp.k_tiles > WAVES * TPW; // K longer than one pass of the workgroup
    sp.groups = sp.strips; // one workgroup per strip
    sp.groups_per_xcd = (sp.groups + 7) / 8;
    dim3 grid(sp.groups_per_xcd * 8), block(WAVES * 64);
    note_launch("stream row waves=%d tpw=%d passes=%d", WAVES, TPW, (sp.k_tiles + WAVES * TPW - 1) / (WAVES * TPW));
    RowTail tail{sp.pqs, sp.bias, nullptr};
#ifdef WOQ_TIMELINE
    if (char const* e = std::getenv("WOQ_TRACE_PTR"))
        tail.trace = reinterpret_cast<unsigned long long*>(std::strtoull(e, nullptr, 16));
#endif
    if (multi)
        hipLaunchKernelGGL((stream_row_kernel<DT, GROUP, PQS, ZERO, WAVES, TPW, true>), grid, block, 0, stream, sp.weight,
            sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, sp.groups_per_xcd, sp.n, sp.k, sp.alpha, sp.out, tail);
    else
        hipLaunchKernelGGL((stream_row_kernel<DT, GROUP, PQS, ZERO, WAVES, TPW, false>), grid, block, 0, stream, sp.weight,
            sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, sp.groups_per_xcd, sp.n, sp.k, sp.alpha, sp.out, tail);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(WOQ_ERR_RUNTIME, "row stream kernel launch failed: %s", hipGetErrorString(err));
    return WOQ_OK;
}

template <int DT, int GROUP, bool PQS, bool ZERO>
int launch_row_shaped(StreamParams const& sp, int waves, int tpw, hipStream_t s)
{
#define WOQ_ROW(WAVES_, TPW_)                                                                                          \
    if (waves == WAVES_ && tpw == TPW_)                                                                                \
        return launch_row_variant<DT, GROUP, PQS, ZERO, WAVES_, TPW_>(sp, s);
    WOQ_ROW(8, 4)
    WOQ_ROW(16, 4)
    WOQ_ROW(8, 8)
    WOQ_ROW(16, 8)
    WOQ_ROW(4, 8)
#undef WOQ_ROW
    return fail(WOQ_ERR_UNSUPPORTED, "row stream shape waves=%d tpw=%d is not instantiated", waves, tpw);
}

template <int DT, int GROUP>
int launch_row_flags(StreamParams const& sp, bool pqs, bool zero, int waves, int tpw, hipStream_t s)
{
    if (pqs)
        return zero ? launch_row_shaped<DT, GROUP, true, true>(sp, waves, tpw, s)
                    : launch_row_shaped<DT, GROUP, true, false>(sp, waves, tpw, s);
    return zero ? launch_row_shaped<DT, GROUP, false, true>(sp, waves, tpw, s)
                : launch_row_shaped<DT, GROUP, false, false>(sp, waves, tpw, s);
}
} // namespace

int launch_stream_row(StreamParams const& sp, int dtype, int group, bool pqs, bool zero, int waves, int tpw, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    if (sp.m != 1 || (group != 64 && group != 128) || sp.k % group)
        return fail(WOQ_ERR_UNSUPPORTED, "row stream kernel: one row, int4, group size 64 or 128");
    if (dtype == WOQ_BF16)
        return group == 64 ? launch_row_flags<WOQ_BF16, 64>(sp, pqs, zero, waves, tpw, s)
                           : launch_row_flags<WOQ_BF16, 128>(sp, pqs, zero, waves, tpw, s);
    return group == 64 ? launch_row_flags<WOQ_FP16, 64>(sp, pqs, zero, waves, tpw, s)
                       : launch_row_flags<WOQ_FP16, 128>(sp, pqs, zero, waves, tpw, s);
}

} // namespace woq
