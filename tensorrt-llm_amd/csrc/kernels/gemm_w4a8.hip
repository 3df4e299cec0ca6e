// W4A8: fp8 (e4m3) activations x int4 weights on the CDNA4 fp8 matrix core.
//
// Semantics of the reference's W4A8 path (fpA_intB runner instantiated for __nv_fp8_e4m3 x uint4
// with half scales, cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h,
// selected by weightOnlyGroupwiseQuantMatmulPlugin.cpp:203-276): the int4 weight is dequantized
// with fp16 scales/zeros and rounded to e4m3, the MMA accumulates fp8 x fp8 products in float32,
// and the epilogue applies alpha and the bias: out = T(alpha * acc + bias).  Group size 128 only.
//
// Same skeleton as the 16-bit prefill kernel (gemm_kernel.h): output tile 16*RT rows x 256
// columns, 4 wavefronts side by side along N with 64 columns each; packed weights go global ->
// registers (the tile layout is the B-operand layout of v_mfma_f32_16x16x32_fp8_fp8 as well: 8
// consecutive k per lane) and are dequantized once per workgroup; the activation tile is DMA-ed
// global -> LDS, double-buffered; the requests of the next step and the conversions are spread
// between the MFMAs; skinny problems split K through the float32 partial buffer.
// An fp8 activation fragment is half the size of a 16-bit one, so LDS holds fragment PAIRS: 16
// rows x 64 k = 1 KiB, written by one DMA instruction (lane 4r+q fetches row r's 16-byte chunk
// q ^ (r>>2): quads read 64 contiguous bytes, the XOR spreads an MFMA lane group over the banks).
#include "dequant_math.h"
#include "gemm_common.h"

namespace woq
{

// elements 4h .. 4h+3 of slab dword `w` -> 4 e4m3 bytes, element order preserved
__device__ __forceinline__ uint32_t dequant4_fp8(uint32_t w, int h, float s, float z)
{
    uint32_t const t = w ^ 0x88888888u; // biased -> two's complement nibbles
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        int const e = 4 * h + i;
        int const slot = (e & 1) ? 4 + (e >> 1) : (e >> 1);
        int const q = (int) (t << (28 - 4 * slot)) >> 28;
        v[i] = clamp_e4m3(__builtin_fmaf((float) q, s, z));
    }
    uint32_t r = 0;
    r = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], (int) r, false);
    r = (uint32_t) __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], (int) r, true);
    return r;
}

// c += a x b (8 e4m3 values per lane each), accumulator tied to one AGPR quad (see Elem::mma_acc)
__device__ __forceinline__ void mma_fp8_acc(u32x2 a, u32x2 b, f32x4& c)
{
    asm volatile("v_mfma_f32_16x16x32_fp8_fp8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

template <int ODT, bool ZERO, int RT, bool SPLITK>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) gemm_w4a8_kernel(GemmParams p)
{
    using EO = Elem<ODT>;
    using EH = Elem<WOQ_FP16>;
    constexpr int TK = 128, SLABS = 4, NS = 4;
    constexpr int BM = RT * 16;
    constexpr int PAIRS = RT * 2;      // fragment pairs (1 KiB) of one A tile
    constexpr int A_BYTES = BM * TK;   // e4m3: one byte per element
    static_assert(PAIRS % 4 == 0, "fragment pairs spread evenly over the 4 wavefronts");

    __shared__ u32x4 a_buf0[A_BYTES / 16];
    __shared__ u32x4 a_buf1[A_BYTES / 16];

    int t;
    if (!xcd_tile(p.tiles_m * p.tiles_n, t))
        return;
    int const tm = t % p.tiles_m, tn = t / p.tiles_m;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const c = lane & 15, kg = lane >> 4;
    int const K = p.k;
    int const kt_begin = SPLITK ? (int) blockIdx.y * p.tiles_per_split : 0;
    int const KT = SPLITK ? (kt_begin + p.tiles_per_split < p.k_tiles ? kt_begin + p.tiles_per_split : p.k_tiles)
                          : p.k_tiles;
    int const m0 = tm * BM;
    int const strip0 = tn * (kGemmBN / 16) + wave * NS;

    constexpr uint32_t kOob = 0x80000000u;
    auto const act_rsrc = make_rsrc(p.act, (uint32_t) p.m * (uint32_t) K);
    uint32_t const sz_bytes = (uint32_t) (K / 128) * (uint32_t) p.n * 2u;
    auto const sc_rsrc = make_rsrc(p.scales, sz_bytes);
    auto const zr_rsrc = make_rsrc(ZERO ? p.zeros : p.scales, sz_bytes);
    auto const w_rsrc = make_rsrc(p.weight, (uint32_t) p.strips * (uint32_t) p.k_tiles * 1024u);

    int strip_of[NS];
    uint32_t wlane[NS], sc_lane[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        strip_of[s] = strip0 + s < p.strips ? strip0 + s : p.strips - 1;
        wlane[s] = ((uint32_t) strip_of[s] * (uint32_t) p.k_tiles * 64u + (uint32_t) lane) * 16u;
        sc_lane[s] = (uint32_t) (strip_of[s] * 16 + c) * 2u;
    }

    f32x4 acc[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            acc[rt][s] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- A tile -> LDS: wavefront w moves pairs w, w+4, ...: piece i is pair f = w + 4i = half
    // w % 2 of row tile 2i + w / 2; K is a multiple of 128, so only kt >= KT falls out of range
    // (rows past M fall outside the descriptor by themselves).
    constexpr int DMA_OPS = PAIRS / 4;
    uint32_t const dma_lane_base = (uint32_t) (m0 + (wave / 2) * 16 + (lane >> 2)) * (uint32_t) K
        + (uint32_t) ((wave % 2) * 64 + (((lane & 3) ^ ((lane >> 4) & 3)) * 16));
    uint32_t const dma_piece_stride = 32u * (uint32_t) K;
    auto dma_base = [&](int kt) -> uint32_t
    { return (dma_lane_base + (uint32_t) kt * (uint32_t) TK) | ((uint32_t) (KT - 1 - kt) & kOob); };
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
    auto fetch_piece = [&](BStage& st, int kt, int i)
    {
        uint32_t const past = (uint32_t) (KT - 1 - kt) & kOob; // kt >= KT: every load of the step reads zeros
        if (i < NS)
            st.w[i] = buffer_load_x4(w_rsrc, wlane[i] + ((uint32_t) kt * 1024u | past));
        else
        {
            int const s = (i - NS) % NS;
            uint32_t const off = ((uint32_t) kt * (uint32_t) p.n * 2u + sc_lane[s]) | past;
            if (i < 2 * NS)
                st.s[s] = buffer_load_u16(sc_rsrc, off);
            else
                st.z[s] = buffer_load_u16(zr_rsrc, off);
        }
    };

    // ---- one tile row of MFMAs, hand-pipelined like the 16-bit kernel: iteration (j, rt) issues
    // the fragment read A_AHEAD iterations away, its share of the next step's requests and of the
    // next slab's conversions (8 half-operands of 4 weights per slab), and the 4 MFMAs of row tile rt.
    constexpr int A_AHEAD = 3;
    u32x2 b_cur[NS], b_nxt[NS];
    auto half_operand = [&](BStage const& st, int j, int ci) -> uint32_t
    {
        int const s = ci / 2, h = ci % 2;
        float const sc = EH::from_bits(st.s[s]);
        float const zr = ZERO ? EH::from_bits(st.z[s]) : 0.f;
        return dequant4_fp8(st.w[s][j], h, sc, zr);
    };

    auto compute = [&](auto const* buf, BStage const& st, BStage& st_next, auto* buf_next, int kt_next)
    {
        char const* a_base = reinterpret_cast<char const*>(buf);
        constexpr int ITERS = SLABS * RT;
        uint32_t const next_base = dma_base(kt_next);
        auto a_read = [&](int it) -> u32x2
        {
            int const rt = it % RT, j = it / RT;
            return *reinterpret_cast<u32x2 const*>(a_base + (rt * 2 + j / 2) * 1024 + a_lane_off[j % 2]);
        };
        u32x2 a_ring[A_AHEAD + 1];
#pragma unroll
        for (int i = 0; i < A_AHEAD; ++i)
            a_ring[i] = a_read(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < SLABS; ++j)
        {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                int const it = j * RT + rt;
                constexpr int FETCH_WINDOW = (SLABS - 1) * RT < FETCH_OPS ? (SLABS - 1) * RT : FETCH_OPS;
#pragma unroll
                for (int q = 0; q < FETCH_OPS; ++q)
                    if (q * FETCH_WINDOW / FETCH_OPS == it)
                        fetch_piece(st_next, kt_next, q);
                constexpr int DMA_WINDOW = ITERS * 5 / 8 > 0 ? ITERS * 5 / 8 : 1;
#pragma unroll
                for (int q = 0; q < DMA_OPS; ++q)
                    if (q * DMA_WINDOW / DMA_OPS == it)
                        dma_piece(buf_next, next_base, q);
                if (it + A_AHEAD < ITERS)
                    a_ring[(it + A_AHEAD) % (A_AHEAD + 1)] = a_read(it + A_AHEAD);
                // 8 half-operands per slab over RT iterations
#pragma unroll
                for (int ci = 0; ci < 8; ++ci)
                    if (ci * RT / 8 == rt)
                    {
                        if (j + 1 < SLABS)
                            b_nxt[ci / 2][ci % 2] = half_operand(st, j + 1, ci);
                        else
                            b_nxt[ci / 2][ci % 2] = half_operand(st_next, 0, ci);
                    }
                u32x2 const a_cur = a_ring[it % (A_AHEAD + 1)];
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    mma_fp8_acc(a_cur, b_cur[s], acc[rt][s]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int s = 0; s < NS; ++s)
                b_cur[s] = b_nxt[s];
        }
    };

    // ---- main loop: two tile rows per iteration so that each LDS buffer is a distinct object ---
    BStage st0, st1;
    {
        uint32_t const base = dma_base(kt_begin);
#pragma unroll
        for (int i = 0; i < DMA_OPS; ++i)
            dma_piece(a_buf0, base, i);
    }
#pragma unroll
    for (int i = 0; i < FETCH_OPS; ++i)
        fetch_piece(st0, kt_begin, i);
#pragma unroll
    for (int ci = 0; ci < 8; ++ci)
        b_cur[ci / 2][ci % 2] = half_operand(st0, 0, ci);
    for (int kt = kt_begin; kt < KT; kt += 2)
    {
        __syncthreads(); // A(kt) has landed for every wavefront; everyone is done reading buffer 1
        compute(a_buf0, st0, st1, a_buf1, kt + 1);
        __syncthreads();
        compute(a_buf1, st1, st0, a_buf0, kt + 2); // past the end of K both operands read as zeros
    }

    // ---- epilogue: out = T(alpha * acc + bias), or partial sums into the float32 buffer --------
    mma_drain();
    uint16_t* out16 = static_cast<uint16_t*>(p.out);
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        if (strip0 + s >= p.strips)
            continue;
        int const col = (strip0 + s) * 16 + c;
        float const bias = (!SPLITK && p.bias) ? EO::load(p.bias, col) : 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                int const row = m0 + rt * 16 + kg * 4 + r;
                if (row < p.m)
                {
                    if constexpr (SPLITK)
                        unsafeAtomicAdd(p.partial + (size_t) row * p.n + col, acc[rt][s][r]);
                    else
                        out16[(size_t) row * p.n + col] = EO::store(__builtin_fmaf(p.alpha, acc[rt][s][r], bias));
                }
            }
    }
}

template <int ODT, bool ZERO, int RT>
int launch_w4a8_variant(GemmParams const& gp, hipStream_t stream)
{
    int const total = gp.tiles_m * gp.tiles_n;
    dim3 grid(((total + 7) / 8) * 8, gp.k_splits), block(256);
    if (gp.k_splits > 1)
    {
        size_t const count = (size_t) gp.m * gp.n;
        hipLaunchKernelGGL((gemm_zero_partial<ODT>), dim3((unsigned) ((count / 4 + 255) / 256)), block, 0, stream,
            gp.partial, count);
        hipLaunchKernelGGL((gemm_w4a8_kernel<ODT, ZERO, RT, true>), grid, block, 0, stream, gp);
        hipLaunchKernelGGL((gemm_finish_partial<ODT>), dim3((unsigned) ((count + 255) / 256)), block, 0, stream, gp.out,
            gp.partial, gp.bias, gp.alpha, gp.m, gp.n);
    }
    else
        hipLaunchKernelGGL((gemm_w4a8_kernel<ODT, ZERO, RT, false>), grid, block, 0, stream, gp);
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
