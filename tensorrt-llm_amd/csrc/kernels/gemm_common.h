// Pieces shared by the two MFMA GEMM kernels (exact-dequantize prefill kernel, deferred-scale
// skinny kernel): the parameter block, the workgroup -> tile order and the split-K helpers.
#pragma once

#include "device_common.h"

namespace woq
{

struct GemmParams
{
    void const* act;
    void const* weight;
    void const* scales;
    void const* zeros;
    void const* bias;
    void* out;
    float alpha;
    int m, n, k;
    int k_tiles; // ceil(k / TILE_K)
    int strips;  // n / 16
    int scale_rows = 1;       // rows of the scale / zero tables: ceil(k / group_size)
    uint32_t group_magic = 0; // see scale_row()
    int tiles_m, tiles_n;
    int k_splits;        // workgroups along K per output tile (blockIdx.y)
    int tiles_per_split; // tile rows of K each of them covers
    float* partial;      // [k_splits, m, n] float32 when k_splits > 1: slab y holds K slice y's sums
    // grouped problems (see MatmulProblem): m is the total row count, tiles_m an upper bound of
    // the row tiles of all experts together
    int64_t const* expert_rows = nullptr;
    int num_experts = 0;
    size_t weight_stride = 0, scale_stride = 0;
    // kActSwiglu / kActGeglu: the epilogue multiplies value column j with f(gate column j + n/2)
    // and writes [m, n/2]; the strips of a wavefront then alternate between the two halves of N
    // (see paired_strip).  Other activations are applied by a separate pass.
    int activation = kActIdentity;
    int tile_cols = 256; // columns of an output tile of the exact-dequantize kernel (256, or 192 for 256-row tiles)
    void const* residual = nullptr; // [m, n_out] in the output type, added last (no split-K with it)
};

// A fragments (16 rows x 32 k of 16-bit values, 1 KiB) in LDS.  The DMA that fills a fragment writes lane l's
// 16 bytes at position l, and lane l = 4 * row + q fetches a 16-byte chunk of `row`, so that quads read
// 64 contiguous bytes from memory; the matrix core wants lane (kg, row) to read chunk kg of `row`.  Which
// chunk sits at position 4 * row + q is chosen so that those reads do not collide on LDS banks: a 128-bit
// LDS read is served in four phases of 16 lanes, and the phases are NOT runs of consecutive lanes - phase 0
// takes lanes 0-3, 12-15, 20-23, 24-27, phase 1 lanes 4-7, 8-11, 16-19, 28-31, phases 2 and 3 the same plus
// 32 - so the four lanes of a phase that share (row mod 4) come from row blocks 0, 3 (chunk kg) and 1, 2
// (chunk kg + 1).  With chunk kg of a row in block b at q = kg ^ frag_swizzle(b) they land on four different
// bank groups.  (kg ^ b, conflict-free if phases were runs of 16 lanes, measures two-way conflicts on
// every read.)
__device__ __forceinline__ int frag_swizzle(int row_block)
{
    return (4 - row_block) & 3;
}

// Strip slot s of a wavefront whose first slot is `first` (even): without a gated activation strip
// first + s; with one, slots pair up - even slot: pair (first + s) / 2 in the value half, odd
// slot: the same pair in the gate half, `half` strips further.  `valid`: the slot's strip exists.
__device__ __forceinline__ int paired_strip(bool gated, int first, int s, int strips, bool& valid)
{
    if (!gated)
    {
        valid = first + s < strips;
        return valid ? first + s : strips - 1;
    }
    int const half = strips / 2, pair = first / 2 + s / 2;
    valid = pair < half;
    return (valid ? pair : half - 1) + (s & 1) * half;
}

inline void set_group_fields(GemmParams& gp, MatmulProblem const& p, int tile_rows)
{
    gp.scale_rows = p.group_size ? (p.k + p.group_size - 1) / p.group_size : 1;
    gp.group_magic = scale_row_magic(p.group_size);
    gp.activation = act_is_gated(p.activation) ? p.activation : kActIdentity;
    // behind a non-gated activation the residual is added by the activation pass, not here
    gp.residual = (p.activation == kActIdentity || act_is_gated(p.activation)) ? p.residual : nullptr;
    gp.expert_rows = p.expert_rows;
    gp.num_experts = p.num_experts;
    gp.weight_stride = p.weight_stride;
    gp.scale_stride = p.scale_stride;
    if (p.expert_rows) // every expert may end with a partly filled tile
        gp.tiles_m = p.m / tile_rows + p.num_experts;
}

// Grouped problems: row tile `tm` counts through the row tiles of expert 0, 1, ... in turn.
// Finds the expert it belongs to, narrows the parameter block to that expert's operands and rows
// (so that the kernel proceeds as for an ordinary problem) and makes tm the tile index inside
// the expert.  False when tm is past the last tile.  All values are wavefront-uniform.
__device__ __forceinline__ bool select_expert(GemmParams& p, int& tm, int tile_rows)
{
    int64_t begin = 0;
    int first_tile = 0;
    for (int e = 0; e < p.num_experts; ++e)
    {
        int64_t const end = p.expert_rows[e];
        int const rows = (int) (end - begin);
        int const tiles = (rows + tile_rows - 1) / tile_rows;
        if (tm < first_tile + tiles)
        {
            p.act = uniform_ptr(static_cast<char const*>(p.act) + (size_t) begin * (size_t) p.k * 2);
            size_t const out_off = (size_t) begin * (size_t) (act_is_gated(p.activation) ? p.n / 2 : p.n) * 2;
            p.out = uniform_ptr(static_cast<char*>(p.out) + out_off);
            if (p.residual)
                p.residual = uniform_ptr(static_cast<char const*>(p.residual) + out_off);
            p.weight = uniform_ptr(static_cast<char const*>(p.weight) + (size_t) e * p.weight_stride);
            p.scales = uniform_ptr(static_cast<char const*>(p.scales) + (size_t) e * p.scale_stride);
            if (p.zeros)
                p.zeros = uniform_ptr(static_cast<char const*>(p.zeros) + (size_t) e * p.scale_stride);
            if (p.bias)
                p.bias = uniform_ptr(static_cast<char const*>(p.bias) + (size_t) e * (size_t) p.n * 2);
            p.m = __builtin_amdgcn_readfirstlane(rows);
            tm = __builtin_amdgcn_readfirstlane(tm - first_tile);
            return true;
        }
        first_tile += tiles;
        begin = end;
    }
    return false;
}

constexpr int kGemmBN = 256; // columns of an output tile (4 wavefronts x 64)

// Workgroups of a persistent launch: the CU count of the current device rounded down to a multiple
// of 8 (one per CU, the same number on every XCD); 0 switches the persistent kernels off
// (WOQ_GEMM_PERSIST=0).
int gemm_persistent_workgroups();

// Output tiles are numbered m-fastest inside a column panel; the 8 XCDs each take one contiguous
// chunk of that order (workgroup i runs on XCD i % 8), so the workgroups that share weight
// columns or activation rows also share an L2.
__device__ __forceinline__ bool xcd_tile(int total, int& t)
{
    int const per_xcd = (total + 7) / 8;
    t = (int) (blockIdx.x & 7) * per_xcd + (int) (blockIdx.x >> 3);
    return (int) (blockIdx.x >> 3) < per_xcd && t < total;
}

// split-K finish: the workgroups of K slice y store their float32 partial sums in slab y of the
// workspace ([splits][m][n], every element of every slab written exactly once per call, so nothing
// needs clearing); out = T(alpha * (slab 0 + slab 1 + ...) + bias), summed in slab order: the result
// does not depend on which workgroup finished first.  Four consecutive columns per thread
// (n is a multiple of 16).
template <int DT>
__global__ void __launch_bounds__(256) gemm_finish_partial(
    void* out, float const* partial, void const* bias, float alpha, int m, int n, int splits)
{
    using E = Elem<DT>;
    size_t const count = (size_t) m * n;
    size_t const i = ((size_t) blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count)
        return;
    // eight slabs are requested at a time (a loop of one dependent load after another paid a memory round
    // trip per slab: 4-5 us for the 6-12 slabs of a skinny problem), then added in slab order; a request
    // past the last slab re-reads that slab and is not added
    f32x4 sum = *reinterpret_cast<f32x4 const*>(partial + i);
    for (int y = 1; y < splits; y += 8)
    {
        f32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
        {
            int const yy = y + u < splits ? y + u : splits - 1;
            v[u] = *reinterpret_cast<f32x4 const*>(partial + (size_t) yy * count + i);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (y + u < splits)
                sum[0] += v[u][0], sum[1] += v[u][1], sum[2] += v[u][2], sum[3] += v[u][3];
    }
    int const col = (int) (i % n);
    f32x4 b = {0.f, 0.f, 0.f, 0.f};
    if (bias)
    {
        u32x2 const v = *reinterpret_cast<u32x2 const*>(static_cast<uint16_t const*>(bias) + col);
        b = f32x4{E::lo(v[0]), E::hi(v[0]), E::lo(v[1]), E::hi(v[1])};
    }
    u32x2 const o = {E::pack(__builtin_fmaf(alpha, sum[0], b[0]), __builtin_fmaf(alpha, sum[1], b[1])),
        E::pack(__builtin_fmaf(alpha, sum[2], b[2]), __builtin_fmaf(alpha, sum[3], b[3]))};
    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + i) = o;
}

} // namespace woq
