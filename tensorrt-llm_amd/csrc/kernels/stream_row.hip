// Decode of one to four rows (int4 weights, group scales): short-lived wavefronts in address order.
//
// Counterpart of the reference's small-M kernel at batch 1
// (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernel.h:57-118) in purpose only.  What HBM rewards on
// this part is many short-lived wavefronts that each read a few contiguous KiB, neighbours reading
// neighbouring addresses at the same time.  So: one workgroup per strip of 16 columns (its tiles are
// contiguous in the gfx950 layout), wavefront w reads the TPW consecutive 1 KiB tiles w * TPW .. of that
// strip with all its loads issued at once, and there is no staging pass and no barrier before the
// arithmetic - every wavefront fetches the few activations and scales it needs itself:
//   * lane (kg, c) of the 16x16x32 matrix instruction supplies row c of the A operand.  Row c carries the
//     activations of activation row c % R of the wavefront's (c / R)-th group of K (R = 1, 2 or 4 rows of
//     the problem; groups per wavefront x R <= 16) and nothing else, so one instruction multiplies every
//     group's activations with one group's weights; D_g = A x W_g is kept per group g and only its rows
//     g * R .. g * R + R - 1 are used: no masking, no zero operands;
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
// per-wavefront time stamps (100 MHz constant clock) for `bench.py --mode timeline`: a library of its own
// (`build.py --timeline`), whose launcher takes the address of the stamp buffer from WOQ_TRACE_PTR
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
    float alpha;
    int m;
    unsigned long long* trace; // WOQ_TIMELINE builds only
};

// The first fourteen dwords of the arguments are what the requests need.  They are plain scalars so that
// the wavefront finds them in SGPRs when it starts (kernel-argument preloading; this file is compiled with
// -amdgpu-kernarg-preload-count=16, of which the hardware's sixteen user SGPRs leave fourteen): a by-value
// struct is fetched with scalar loads from the argument buffer instead, 0.2-0.3 us per dependent batch,
// before the first address can be formed.  `act_bytes` = m * k * 2: rows of the M-tile past m start
// outside the descriptor, read zeros and cost no traffic.
template <int DT, int GROUP, bool PQS, bool ZERO, int WAVES, int TPW, bool MULTI, int R>
__global__ void __launch_bounds__(WAVES * 64) stream_row_kernel(void const* weight, void const* act, void const* scales,
    void const* zeros, int k_tiles, int strips, int groups_per_xcd, int n, int k, int act_bytes, void* out, RowTail tail)
{
    using E = Elem<DT>;
    constexpr int TK = 128;
    constexpr int SEGS = TK / GROUP, SEG_SLABS = GROUP / 32;
    constexpr int GROUPS = TPW * SEGS; // groups of K per wavefront and pass
    constexpr int ROWS = GROUPS * R;   // rows of the M-tile in use
    static_assert(GROUP == 64 || GROUP == 128, "group scales of 64 or 128 rows");
    static_assert(R == 1 || R == 2 || R == 4, "one, two or four activation rows");
    static_assert(ROWS <= 16, "the M-tile has 16 rows");
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
    auto const act_rsrc = make_rsrc(act, (uint32_t) act_bytes);
    // this lane's activations: row c % R of the problem, group c / R of the pass
    uint32_t const a_lane = (uint32_t) (c % R) * (uint32_t) k * 2u + (uint32_t) (kg * 8) * 2u;

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
        int const g_mine = kt0 * SEGS + c / R; // the group whose activations this lane holds
        bool const a_ok = c < ROWS && g_mine < groups_k;
#pragma unroll
        for (int js = 0; js < SEG_SLABS; ++js)
            st.a[js] = buffer_load_x4(act_rsrc, a_ok ? a_lane + (uint32_t) (g_mine * GROUP + js * 32) * 2u : kOob);
#pragma unroll
        for (int i = 0; i < TPW; ++i)
            st.w[i] = buffer_load_x4_once(w_rsrc, kt0 + i < KT ? wlane + (uint32_t) (kt0 + i) * 1024u : kOob);
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
    // what the end of a pass needs: register r of lane (kg, c) is row kg * 4 + r of the M-tile, i.e. group
    // (kg * 4 + r) / R - the lane loads that group's scale and zero for its column c (and the smoothing
    // factors of the lane's activations)
    auto fetch_scales = [&](Stage& st, int kt0)
    {
        int const g0 = kt0 * SEGS;
        if constexpr (PQS)
        {
            int const g_mine = g0 + c / R;
            bool const a_ok = c < ROWS && g_mine < groups_k;
#pragma unroll
            for (int js = 0; js < SEG_SLABS; ++js)
                st.pq[js] = buffer_load_x4(pqs_rsrc, a_ok ? (uint32_t) (g_mine * GROUP + js * 32 + kg * 8) * 2u : kOob);
        }
#pragma unroll
        for (int r = 0; r < 4; r += R)
        {
            int const gl = (kg * 4 + r) / R;
            bool const ok = gl < GROUPS && g0 + gl < groups_k;
            uint32_t const off = ok ? (uint32_t) (g0 + gl) * (uint32_t) n * 2u + sc_lane : kOob;
            st.s[r] = buffer_load_u16(sc_rsrc, off);
            st.z[r] = ZERO ? buffer_load_u16(zr_rsrc, off) : (uint16_t) 0;
        }
    };
    fetch_scales(st[0], kt_of(0));
    __builtin_amdgcn_sched_barrier(0);
    WOQ_TR(2);

    float total[R]; // this lane's share of output column c, per activation row
#pragma unroll
    for (int i = 0; i < R; ++i)
        total[i] = 0.f;
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
        // ---- row kg * 4 + r of D_g, g = (kg * 4 + r) / R, scaled ----
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            float P = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                int const g = (q * 4 + r) / R;
                if (g < GROUPS)
                {
                    float const v = acc[g / SEGS][g % SEGS][r];
                    P = kg == q ? v : P;
                }
            }
            float const sc = E::from_bits(st.s[r - r % R]);
            float const cc = __builtin_fmaf(-OFF, sc, ZERO ? E::from_bits(st.z[r - r % R]) : 0.f);
            total[r % R] = __builtin_fmaf(sc, P, __builtin_fmaf(cc, acc_s[r], total[r % R]));
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
    __shared__ float red[WAVES][R][16];
#pragma unroll
    for (int i = 0; i < R; ++i)
    {
        total[i] += __shfl_xor(total[i], 16);
        total[i] += __shfl_xor(total[i], 32);
        if (kg == 0)
            red[wave][i][c] = total[i];
    }
    WOQ_TR(7);
    __syncthreads();
    WOQ_TR(8);
    if (threadIdx.x < 16 * R)
    {
        int const row = threadIdx.x >> 4;
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
            sum += red[w2][row][c];
        int const ocol = strip * 16 + c;
        float v = tail.alpha * sum;
        if (tail.bias)
            v += E::load(tail.bias, ocol);
        if (row < tail.m)
            static_cast<uint16_t*>(out)[(size_t) row * n + ocol] = E::store(v);
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
template <int DT, int GROUP, bool PQS, bool ZERO, int WAVES, int TPW, int R>
int launch_row_variant(StreamParams sp, hipStream_t stream)
{
    if constexpr (TPW * (128 / GROUP) * R > 16)
        return fail(WOQ_ERR_UNSUPPORTED, "row stream shape: %d tiles of %d groups x %d rows do not fit the 16 MFMA rows", TPW,
            128 / GROUP, R);
    else
    {
        bool const multi = sp.k_tiles > WAVES * TPW; // K longer than one pass of the workgroup
        sp.groups = sp.strips;                       // one workgroup per strip
        sp.groups_per_xcd = (sp.groups + 7) / 8;
        dim3 grid(sp.groups_per_xcd * 8), block(WAVES * 64);
        note_launch("stream row waves=%d tpw=%d passes=%d rows=%d", WAVES, TPW, (sp.k_tiles + WAVES * TPW - 1) / (WAVES * TPW),
            R);
        RowTail tail{sp.pqs, sp.bias, sp.alpha, sp.m, nullptr};
#ifdef WOQ_TIMELINE
        if (char const* e = std::getenv("WOQ_TRACE_PTR"))
            tail.trace = reinterpret_cast<unsigned long long*>(std::strtoull(e, nullptr, 16));
#endif
        int const act_bytes = sp.m * sp.k * 2;
        if (multi)
            hipLaunchKernelGGL((stream_row_kernel<DT, GROUP, PQS, ZERO, WAVES, TPW, true, R>), grid, block, 0, stream,
                sp.weight, sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, sp.groups_per_xcd, sp.n, sp.k, act_bytes,
                sp.out, tail);
        else
            hipLaunchKernelGGL((stream_row_kernel<DT, GROUP, PQS, ZERO, WAVES, TPW, false, R>), grid, block, 0, stream,
                sp.weight, sp.act, sp.scales, sp.zeros, sp.k_tiles, sp.strips, sp.groups_per_xcd, sp.n, sp.k, act_bytes,
                sp.out, tail);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess)
            return fail(WOQ_ERR_RUNTIME, "row stream kernel launch failed: %s", hipGetErrorString(err));
        return WOQ_OK;
    }
}

template <int DT, int GROUP, bool PQS, bool ZERO, int R>
int launch_row_shaped(StreamParams const& sp, int waves, int tpw, hipStream_t s)
{
#define WOQ_ROW(WAVES_, TPW_)                                                                                          \
    if (waves == WAVES_ && tpw == TPW_)                                                                                \
        return launch_row_variant<DT, GROUP, PQS, ZERO, WAVES_, TPW_, R>(sp, s);
    WOQ_ROW(4, 8)
    WOQ_ROW(8, 8)
    WOQ_ROW(16, 8)
    WOQ_ROW(4, 4)
    WOQ_ROW(8, 4)
    WOQ_ROW(16, 2)
    WOQ_ROW(8, 7) // K = 14336 is 112 tiles: passes that K divides evenly, every wavefront with a full share
    WOQ_ROW(7, 4)
#undef WOQ_ROW
    return fail(WOQ_ERR_UNSUPPORTED, "row stream shape waves=%d tpw=%d is not instantiated", waves, tpw);
}

template <int DT, int GROUP, int R>
int launch_row_flags(StreamParams const& sp, bool pqs, bool zero, int waves, int tpw, hipStream_t s)
{
    if (pqs)
        return zero ? launch_row_shaped<DT, GROUP, true, true, R>(sp, waves, tpw, s)
                    : launch_row_shaped<DT, GROUP, true, false, R>(sp, waves, tpw, s);
    return zero ? launch_row_shaped<DT, GROUP, false, true, R>(sp, waves, tpw, s)
                : launch_row_shaped<DT, GROUP, false, false, R>(sp, waves, tpw, s);
}

template <int DT, int GROUP>
int launch_row_rows(StreamParams const& sp, bool pqs, bool zero, int waves, int tpw, hipStream_t s)
{
    if (sp.m == 1)
        return launch_row_flags<DT, GROUP, 1>(sp, pqs, zero, waves, tpw, s);
    if (sp.m == 2)
        return launch_row_flags<DT, GROUP, 2>(sp, pqs, zero, waves, tpw, s);
    return launch_row_flags<DT, GROUP, 4>(sp, pqs, zero, waves, tpw, s);
}
} // namespace

int launch_stream_row(StreamParams const& sp, int dtype, int group, bool pqs, bool zero, int waves, int tpw, void* stream)
{
    auto s = static_cast<hipStream_t>(stream);
    if (sp.m < 1 || sp.m > 4 || (group != 64 && group != 128) || sp.k % group)
        return fail(WOQ_ERR_UNSUPPORTED, "row stream kernel: one to four rows, int4, group size 64 or 128");
    if ((uint64_t) sp.m * (uint64_t) sp.n * 2 >= ((uint64_t) 1 << 31))
        return fail(WOQ_ERR_UNSUPPORTED, "row stream kernel: output beyond 2 GiB");
    if (dtype == WOQ_BF16)
        return group == 64 ? launch_row_rows<WOQ_BF16, 64>(sp, pqs, zero, waves, tpw, s)
                           : launch_row_rows<WOQ_BF16, 128>(sp, pqs, zero, waves, tpw, s);
    return group == 64 ? launch_row_rows<WOQ_FP16, 64>(sp, pqs, zero, waves, tpw, s)
                       : launch_row_rows<WOQ_FP16, 128>(sp, pqs, zero, waves, tpw, s);
}

} // namespace woq
