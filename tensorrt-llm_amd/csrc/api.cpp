// The matmul entry points of libwoq: argument validation, M-regime selection and dispatch to the
// kernel launchers.  This is the counterpart of the two plugins' enqueue()
// (cpp/tensorrt_llm/plugins/weightOnlyQuantMatmulPlugin/weightOnlyQuantMatmulPlugin.cpp:283-339,
// cpp/tensorrt_llm/plugins/weightOnlyGroupwiseQuantMatmulPlugin/weightOnlyGroupwiseQuantMatmulPlugin.cpp:407-495),
// of the small-M dispatcher (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernelDispatcher.h:30-166)
// and of the runner's argument checks
// (cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h:129-196).
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <initializer_list>

#include <hip/hip_runtime.h>

#include "woq_internal.h"

namespace woq
{
int launch_stream_BF16_4(MatmulProblem const& p, void* stream);
int launch_stream_BF16_8(MatmulProblem const& p, void* stream);
int launch_stream_FP16_4(MatmulProblem const& p, void* stream);
int launch_stream_FP16_8(MatmulProblem const& p, void* stream);

int launch_gemm_BF16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_gemm_BF16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_gemm_FP16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_gemm_FP16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_skinny_BF16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_skinny_BF16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_skinny_FP16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_skinny_FP16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream);
int launch_gemm_w4a8(MatmulProblem const& p, void* stream);
int launch_stream_w4a8(MatmulProblem const& p, void* stream);

int launch_gemm_planned(MatmulProblem const& p, GemmPlan const& plan, void* stream);

// plan of a plain (not grouped) 16-bit GEMM-regime call: the tactic in force, else the cost model's
GemmPlan planned_gemm(int m, int n, int k, int bits, int group)
{
    Tactic const* t = current_tactic();
    if (t && t->regime == WOQ_REGIME_GEMM && t->rt != 0 && (t->rt != 2 || (t->skinny && bits == 4)))
    {
        GemmPlan pl{};
        pl.skinny = t->skinny != 0;
        pl.rt = t->rt;
        int const k_tiles = (k + tile_k_of_bits(bits) - 1) / tile_k_of_bits(bits);
        pl.k_splits = t->k_splits < 1 ? 1 : (t->k_splits > k_tiles ? k_tiles : t->k_splits);
        pl.ws_bytes = split_partial_bytes(m, n, pl.k_splits);
        return pl;
    }
    return plan_gemm(m, n, k, bits, true, 1, group);
}

int launch_gemm(MatmulProblem const& p, void* stream)
{
    if (p.w4a8)
        return launch_gemm_w4a8(p, stream);
    return launch_gemm_planned(p, planned_gemm(p.m, p.n, p.k, p.bits, p.group_size), stream);
}

int launch_gemm_planned(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    bool const bf16 = p.out_dtype == WOQ_BF16;
    if (plan.skinny)
    {
        if (bf16)
            return p.bits == 4 ? launch_skinny_BF16_4(p, plan, stream) : launch_skinny_BF16_8(p, plan, stream);
        return p.bits == 4 ? launch_skinny_FP16_4(p, plan, stream) : launch_skinny_FP16_8(p, plan, stream);
    }
    if (bf16)
        return p.bits == 4 ? launch_gemm_BF16_4(p, plan, stream) : launch_gemm_BF16_8(p, plan, stream);
    return p.bits == 4 ? launch_gemm_FP16_4(p, plan, stream) : launch_gemm_FP16_8(p, plan, stream);
}

int launch_stream(MatmulProblem const& p, void* stream)
{
    if (p.w4a8)
        return launch_stream_w4a8(p, stream);
    if (!p.num_experts && p.m > kStreamMaxM) // a grouped problem runs 16-row passes per expert
        return fail(WOQ_ERR_UNSUPPORTED, "unsupported m: the streaming kernel covers m <= %d (got %d)", kStreamMaxM,
            p.m);
    if (p.out_dtype == WOQ_BF16)
        return p.bits == 4 ? launch_stream_BF16_4(p, stream) : launch_stream_BF16_8(p, stream);
    return p.bits == 4 ? launch_stream_FP16_4(p, stream) : launch_stream_FP16_8(p, stream);
}

// Launch shape of the streaming kernel.  More strips per wavefront amortise the activation
// fragments and the row-sum MFMA; more wavefronts per workgroup split K further so that small
// problems still fill 256 CUs.
struct StreamShape
{
    int ns, waves, pf, lds;
};

StreamShape pick_stream_shape(int mt, int m, int k, int strips, int k_tiles, int tile_k, int group, int const* split_shape,
    bool three_strips)
{
    if (split_shape && split_shape[0] != 0) // the K split's own launch shape
        return {split_shape[0], split_shape[1], split_shape[2], split_shape[3]};
    EnvOverrides const& env = env_overrides();
    if (env.has_stream_shape)
        return {env.stream_shape[0], env.stream_shape[1], env.stream_shape[2], env.stream_shape[3]};
    (void) k_tiles;
    if (Tactic const* t = current_tactic())
    {
        if (t->regime == WOQ_REGIME_STREAM && t->ns != 0 && t->mt == mt)
            return {t->ns, t->waves, t->pf, t->lds};
    }
    if (mt == 1)
    {
        int const rows = m < 16 ? m : 16;
        size_t const act_lds = (size_t) rows * ((size_t) ((k + tile_k - 1) / tile_k) * tile_k * 2 + 16);
        // the group scales and zeros are staged next to the activations (at most k * ns bytes, and k more
        // for the activation row sums).  Staging the activations pays for a single row (the kernel
        // then scales one output row only) up to ~48 KiB, for more rows up to ~20 KiB (M = 2 at
        // K = 4096; beyond that register-held fragments with staged scales measure faster: the
        // staging pass and the resident workgroups it costs outweigh the shared reads), and with
        // few column groups and at most 3 rows (4 rows while K <= 4096: o_proj 4096x4096 at M = 4
        // 5.9 -> 5.3 us), where one workgroup per CU covers the whole problem anyway (the down
        // projections: long K, N <= 4096)
        // strips per workgroup: one up to 256 column strips, two up to 512, three up to 768, else four, so
        // that no launch has between 256 and 512 workgroups (a partly filled second round over the 256
        // CUs measured 10-70 % slower than half as many workgroups of twice the width); three strips
        // keep 214-256 CUs busy where four would leave 129-192 (3-6 % on N = 9216 ... 12288)
        StreamShape sh = strips > 768 || (strips > 512 && !three_strips)
            ? StreamShape{4, 8, 2, 1}
            : (strips > 512 ? StreamShape{3, 8, 2, 1}
                            : (strips > 256 ? StreamShape{2, 8, 4, 1} : StreamShape{1, 8, 4, 1}));
        // LDS of one workgroup of the staged variants: activations, group scales + zeros and row sums
        // (at most k * ns + k bytes, group 64 with zeros), the epilogue's reduction buffer
        size_t const scale_unit = group == 0 ? 0 : (size_t) k * 64 / group;
        auto footprint = [&](StreamShape const& v) {
            return act_lds + scale_unit * (v.ns + 1) + (size_t) v.waves * v.ns * 1024;
        };
        // a launch of more workgroups than CUs wants two of them resident per CU
        if (sh.ns == 4 && strips > 4 * 256 && 2 * footprint(sh) > (size_t) 160 * 1024)
            sh = StreamShape{2, 8, 4, 1};
        if (act_lds <= (size_t) (rows == 1 ? 48 : 20) * 1024)
        {
            if (act_lds + (size_t) k * (sh.ns + 1) <= stream_max_staged_lds(sh.ns, sh.waves))
                return sh;
            if (act_lds + (size_t) k * 2 <= stream_max_staged_lds(1, 8))
                return {1, 8, 4, 1};
        }
        else if (strips <= 256 && (rows <= 3 || (rows == 4 && act_lds <= (size_t) 33 * 1024))
            && act_lds + (size_t) k * 2 <= stream_max_staged_lds(1, 8))
            return {1, 8, 4, 1};
        // 513..1024 strips run as at most 256 workgroups of four strips: with one workgroup per CU the
        // eight wavefronts of the staged variant keep more loads in flight than the four of the
        // register variant, for up to four rows
        else if (strips > 512 && strips <= 1024 && rows <= 4
            && act_lds + (size_t) k * (sh.ns + 1) <= stream_max_staged_lds(sh.ns, 8))
            return sh;
        // activations stay in registers; the group scales / zeros (at most k * ns bytes) are still
        // staged while that leaves room for the resident workgroups the shape counts on
        StreamShape reg = strips > 512 ? StreamShape{4, 4, 2, 0}
                                       : (strips > 256 ? StreamShape{2, 8, 2, 0} : StreamShape{1, 8, 4, 0});
        if ((size_t) k * reg.ns <= (size_t) (reg.waves == 4 ? 32 : 64) * 1024)
            reg.lds = 2;
        return reg;
    }
    if (mt == 2 || mt == 4)
    {
        // the group scales / zeros (at most k * ns bytes) are staged in LDS while they are small
        int const ns = stream_mid_ns(strips);
        int const lds = group != 0 && (size_t) k * ns <= (size_t) 48 * 1024 ? 2 : 0;
        return {ns, 8, mt == 2 ? 2 : 1, lds};
    }
    return {1, 8, 1, 0};
}

int raise_lds_once(std::atomic<uint64_t>& raised, void const* kernel, int bytes)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess)
    {
        // device ordinals from 64 on have no bit of their own: the (idempotent) call is made every time there
        uint64_t const bit = dev < 64 ? (uint64_t) 1 << dev : 0;
        if (raised.load(std::memory_order_relaxed) & bit)
            return WOQ_OK;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess)
        {
            raised.fetch_or(bit, std::memory_order_relaxed);
            return WOQ_OK;
        }
    }
    (void) hipGetLastError(); // do not leave the error for the caller's next runtime call
    return fail(WOQ_ERR_RUNTIME, "raising the dynamic LDS limit failed: %s", hipGetErrorString(e));
}

struct WideShape
{
    int ns, waves, pf;
};

// The wide streaming kernel (a wavefront per NS strips over all of K) for this problem, and its launch
// shape.  WOQ_WIDE_SHAPE="ns,waves,pf" forces it, "0" switches it off.
bool pick_wide_shape(int m, int n, int k, int group, int bits, WideShape& out)
{
    (void) group;
    (void) bits;
    if (Tactic const* t = current_tactic())
        if (t->regime == WOQ_REGIME_STREAM && t->ns != 0)
            return false; // a tuned launch shape of the strip-group kernel
    EnvOverrides const& env = env_overrides();
    if (env.wide_mode == 0 || (env.has_stream_shape && env.wide_mode != 1))
        return false; // switched off, or a launch shape of the strip-group kernel is forced
    if (env.wide_mode == 1)
    {
        out = WideShape{env.wide_shape[0], env.wide_shape[1], env.wide_shape[2]};
        return true;
    }
    // Measured on MI355X (one row, int4): with K up to 4096 and at least 1536 column strips (the
    // Llama-3-8B gate_up, 4096 x 28672) two strips per wavefront, four wavefronts, four tile rows in
    // flight run 5-7 % faster than the strip-group kernel (13.5 against 14.3 us); with longer K or
    // fewer columns the strip-group kernel is as fast or faster.
    if (m == 1 && k <= 4096 && n >= 1536 * 16)
    {
        out = WideShape{2, 4, 4};
        return true;
    }
    return false;
}

// The single-row streaming kernel (one workgroup per strip, short-lived wavefronts) for this problem, and
// its launch shape: wavefronts per workgroup and tiles (1 KiB, 128 rows of K) per wavefront and pass.
// WOQ_ROW_SHAPE="waves,tiles" forces it, "0" switches it off.
bool pick_row_shape(int m, int n, int k, int group, int bits, int& waves, int& tiles)
{
    (void) n;
    if (m < 1 || m > 4 || bits != 4 || (group != 64 && group != 128))
        return false;
    if (Tactic const* t = current_tactic())
        if (t->regime == WOQ_REGIME_STREAM && t->ns != 0)
            return false; // a tuned launch shape of the strip-group kernel
    EnvOverrides const& env = env_overrides();
    if (env.row_mode == 0 || env.has_stream_shape || env.wide_mode == 1)
        return false;
    if (env.row_mode == 1)
    {
        waves = env.row_shape[0], tiles = env.row_shape[1];
        return true;
    }
    // Measured on MI355X (int4 with group scales and zeros, against the strip-group and wide kernels).
    // One row: 4096 x 6144 5.69 -> 4.74 us, 4096 x 4096 4.64 -> 3.91, 4096 x 28672 13.74 -> 12.85,
    // 14336 x 4096 8.43 -> 8.28, 8192 x 10240 11.15 -> 10.97, 8192 x 8192 9.34 -> 8.93, 8192 x 57344
    // 45.79 -> 44.34, 28672 x 8192 26.90 -> 24.61.  Launch shape: one pass over K where a workgroup of
    // at most sixteen wavefronts x eight tiles reaches that far (few wavefronts with eight tiles each up to
    // K = 4096, eight up to 8192, sixteen up to 16384), else passes of four wavefronts x eight tiles.
    // Two rows (two rows of the M-tile per group, so at most eight groups per wavefront): 4096 x 6144
    // 5.89 -> 5.17, 4096 x 4096 4.58 -> 4.31, 4096 x 28672 14.06 -> 13.49, 14336 x 4096 10.02 -> 8.51,
    // 28672 x 8192 27.63 -> 24.67; nothing to gain at K = 8192.  Three and four rows (four groups per
    // wavefront): the narrow matrices only - 4096 x 6144 6.33 -> 5.84, 4096 x 4096 5.25 -> 4.51, 14336 x 4096
    // 12.14 -> 10.07; the wide ones and K >= 8192 with 512 strips or more are 5-15 % slower than on the
    // strip-group kernel, which shares each activation fragment among more strips.
    int const k_tiles = (k + 127) / 128;
    int const strips = n / 16;
    int const segs = 128 / group;
    // K = 14336 (112 tiles) does not fill sixteen wavefronts x eight tiles - two wavefronts idle, the others with
    // the longest share - and takes shapes that divide it instead: one row, two passes of eight wavefronts x seven
    // tiles, 7.78 -> 7.28 us; four rows (g128), four passes of seven wavefronts x four tiles, 9.03 -> 8.63
    // (two and three rows: within the noise).
    // With the weights read non-temporally, smaller requests per wavefront win on three classes (one row): K = 4096 on
    // wide matrices, eight wavefronts x four tiles (4096 x 28672 11.85 -> 11.47 us; level on 384 strips, 3.7 -> 4.1 on
    // 256); K = 8192 on up to 512 strips, two passes of eight x four (8192 x 8192 8.0 -> 7.75; level on 640 strips
    // and on 3584); K beyond 16384, passes of four x four (28672 x 8192 21.7 -> 21.0).
    if (m == 1)
    {
        tiles = 8;
        waves = k_tiles <= 32 ? 4 : (k_tiles <= 64 ? 8 : (k_tiles <= 128 ? 16 : 4));
        if (k_tiles > 64 && k_tiles <= 128 && k_tiles % 56 == 0)
            waves = 8, tiles = 7;
        else if ((k_tiles <= 32 && strips >= 1024) || (k_tiles > 32 && k_tiles <= 64 && strips <= 512))
            waves = 8, tiles = 4;
        else if (k_tiles > 128)
            waves = 4, tiles = 4;
        return true;
    }
    // (two rows, with the weights read non-temporally: 4096 x 4096 with four wavefronts x eight tiles 4.22 -> 3.96 us;
    // 8192 x 8192 in passes of four x four 8.74 (strip-group kernel) -> 8.05; level on 8192 x 10240)
    if (m == 2)
    {
        if (k_tiles > 32 && k_tiles <= 64 && strips <= 512)
            return waves = 4, tiles = 4, true;
        if (k_tiles > 32 && k_tiles <= 64 && strips < 2048)
            return false;
        tiles = 4;
        waves = k_tiles <= 128 ? 8 : 4;
        if (k_tiles <= 32 && strips <= 256 && segs == 1)
            waves = 4, tiles = 8;
        return true;
    }
    if (strips > 512 || k_tiles > 128 || (k_tiles > 32 && k_tiles <= 64))
        return false;
    tiles = 4 / segs;
    waves = segs == 1 ? 8 : 16;
    if (m == 4 && segs == 1 && k_tiles > 64 && k_tiles % 28 == 0)
        waves = 7;
    return true;
}

// The multi-row streaming kernel (stream_rows_kernel.h: up to sixteen rows, no staging pass) for this problem, and
// its launch shape: wavefronts per workgroup, strips per workgroup, tile rows per wavefront and pass.
// WOQ_ROWS_SHAPE="waves,ns,tiles" forces it, "0" switches it off.
bool pick_rows_shape(int m, int n, int k, int group, int bits, bool pqs, int& waves, int& ns, int& tiles)
{
    (void) pqs; // smoothed activations cost four more requests per tile row: same classes
    if (m < 1 || m > 16 || (group != 0 && group != 64 && group != 128) || (group && k % group))
        return false;
    if (Tactic const* t = current_tactic())
        if (t->regime == WOQ_REGIME_STREAM && t->ns != 0)
            return false; // a tuned launch shape of the strip-group kernel
    EnvOverrides const& env = env_overrides();
    if (env.rows_mode == 0 || env.has_stream_shape || env.wide_mode == 1 || env.stream_splits > 0)
        return false;
    if (env.rows_mode == 1)
    {
        waves = env.rows_shape[0], ns = env.rows_shape[1], tiles = env.rows_shape[2];
        return true;
    }
    // Measured on MI355X against the staged strip-group kernels (bf16, scales + zeros; 2 tile rows per
    // wavefront and pass, 8 wavefronts; us, staged -> this kernel).  K = 4096, 256 strips, one strip per
    // workgroup: 5 rows 5.64 -> 4.64, 8 6.11 -> 4.95, 12 6.60 -> 5.56, 16 7.25 -> 6.05 (g64: 6.54 -> 5.17 at 8 rows);
    // 384 strips, two strips: 5 rows 6.19 -> 5.68, 8 6.56 -> 5.88, 16 7.68 -> 7.10 (g64 6.95 -> 6.59 at 8);
    // 1792 strips, four strips (g128 only): 3 rows 14.73 -> 13.86, 4 15.31 -> 14.14, 8 15.17 -> 14.44, 10 15.14 ->
    // 14.85, from 12 rows on slower.  K = 8192, 640 strips, four strips (g128): 5 rows 13.89 -> 12.91, 8 14.09 ->
    // 13.31, 10 14.21 -> 13.78, slower below 5 and above 10 rows.  Elsewhere (K = 8192 with up to 512 strips:
    // within 5 % either way; the widest matrices; K beyond 8192, where the staged kernel splits K across
    // workgroups) the staged kernels stay.
    int const strips = n / 16;
    waves = 8, tiles = 2;
    if (bits == 8 && group == 0)
    {
        // int8 per-channel (fp16 / bf16, no zeros), same comparison: K = 4096, 256 strips, one strip per
        // workgroup: 8 rows 6.36 -> 5.90, 16 rows 7.51 -> 6.77 (one row: 5.37 -> 5.52, not taken); 384 strips, two
        // strips: 8 rows 7.57 -> 7.09, 16 rows 8.70 -> 8.12; wide matrices, sixteen wavefronts x two strips: 8192 x
        // 57344 at 1 / 4 / 8 rows 83.3 -> 75.4 / 82.4 -> 75.9 / 84.7 -> 78.0, 4096 x 28672 21.3 -> 21.0 / 22.4 -> 21.1 /
        // 22.7 -> 22.3, slower at 16 rows; K = 14336 x 256 strips and 8192 x 640 strips: no gain.
        if (k <= 4096 && strips <= 256 && m >= 5)
            return ns = 1, true;
        if (k <= 4096 && strips <= 512 && m >= 5)
            return ns = 2, true;
        if (k <= 8192 && strips >= 1024 && m <= 8)
            return waves = 16, ns = 2, true;
        return false;
    }
    if (bits != 4 || group == 0 || m < 2)
        return false; // int8 with group scales, int4 per-channel: not measured, the staged kernels serve them
    int const k_tiles = (k + 127) / 128;
    if (k_tiles <= 32)
    {
        if (strips <= 256 && m >= 5)
            return ns = 1, true;
        if (strips <= 512 && m >= 5)
            return ns = 2, true;
        if (strips >= 1024 && group == 128 && m >= 3 && m <= 10)
            return ns = 4, true;
        return false;
    }
    if (k_tiles <= 64 && strips > 512 && strips <= 1024 && group == 128 && m >= 5 && m <= 10)
        return ns = 4, true;
    return false;
}

// The W4A8 multi-row kernel (stream_rows_w4a8.hip) for this problem and its launch shape; WOQ_ROWS_SHAPE as above.
bool pick_rows_w4a8_shape(int m, int n, int k, int& waves, int& ns, int& tiles)
{
    if (m < 1 || m > 16)
        return false;
    EnvOverrides const& env = env_overrides();
    if (env.rows_mode == 0 || env.has_stream_shape)
        return false;
    if (env.rows_mode == 1)
    {
        waves = env.rows_shape[0], ns = env.rows_shape[1], tiles = env.rows_shape[2];
        return true;
    }
    // Measured on MI355X against the staged W4A8 streaming kernel (bf16 output, symmetric g128; us, staged ->
    // this kernel; eight wavefronts, two tile rows per wavefront and pass).  K = 4096: 256 strips, one strip per
    // workgroup, 5 rows 5.48 -> 5.23, 10 5.98 -> 5.50, 16 6.99 -> 6.52; 384 strips, two strips, 5 rows 7.43 -> 6.46,
    // 8 7.78 -> 6.65, 10 7.96 -> 6.72, 16 7.95 -> 7.25; 1792 strips, two strips up to 8 rows (5 rows 16.3 -> 15.2,
    // 8 19.7 -> 16.1), four strips at 9 ... 11 (10 rows 20.4 -> 16.4), slower from 12 rows on.  K = 8192, 640 strips,
    // four strips from 12 rows on: 12 rows 17.6 -> 16.9, 16 20.2 -> 17.2 (10 rows: 16.1 -> 16.7 since the staged
    // kernel reads its weights non-temporally); slower below.  Elsewhere
    // (K = 8192 with up to 512 strips, the widest matrices, K beyond 8192) the staged kernel stays.
    int const k_tiles = k / 128;
    int const strips = n / 16;
    waves = 8, tiles = 2;
    if (m < 5)
        return false;
    if (k_tiles <= 32)
    {
        if (strips <= 256)
            return ns = 1, true;
        if (strips <= 512)
            return ns = 2, true;
        if (strips >= 1024 && m <= 11)
            return ns = m <= 8 ? 2 : 4, true;
        return false;
    }
    if (k_tiles <= 64 && strips > 512 && strips <= 1024 && m >= 12)
        return ns = 4, true;
    return false;
}

// The W4A8 row kernel (stream_row_w4a8.hip) for this problem and its launch shape; WOQ_ROW_SHAPE as above.
bool pick_row_w4a8_shape(int m, int n, int k, int& waves, int& tiles)
{
    (void) n;
    if (m < 1 || m > 4)
        return false;
    EnvOverrides const& env = env_overrides();
    if (env.row_mode == 0 || env.has_stream_shape)
        return false;
    if (env.row_mode == 1)
    {
        waves = env.row_shape[0], tiles = env.row_shape[1];
        return true;
    }
    // Measured on MI355X against the strip-group W4A8 kernel (both convert through the table): with K up to
    // 4096 eight wavefronts x four tiles (4096 x 28672 at one row 15.9 -> 14.3 us, 4096 x 4096 5.08 -> 4.86);
    // with K up to 8192 and at most 1024 strips sixteen x four (8192 x 8192 10.4 -> 9.7 us, at four rows
    // 11.6 -> 10.8; 8192 x 10240 at four rows 14.6 -> 13.4).  The conversion, not the memory system, bounds
    // this kernel (about 80 VALU instructions per KiB of weights), so the wide and long matrices, where the
    // strip-group kernel's deeper pipeline keeps more of it under the loads, stay there.
    // K = 14336 (112 tiles) on a narrow matrix, with shapes that divide it: 14336 x 4096 at two rows, sixteen
    // wavefronts x seven tiles, 9.21 -> 8.74 us; at four rows, two passes of fourteen x four, 10.77 -> 9.80
    // (one row: level with the strip-group kernel, which keeps it).
    int const k_tiles = (k + 127) / 128;
    if (k_tiles > 64 && k_tiles <= 128 && k_tiles % 56 == 0 && n <= 256 * 16 && m >= 2)
    {
        waves = m == 2 ? 16 : 14, tiles = m == 2 ? 7 : 4;
        return true;
    }
    if (k_tiles <= 32)
        waves = 8;
    else if (k_tiles <= 64 && n <= 1024 * 16)
        waves = 16;
    else
        return false;
    tiles = 4;
    return true;
}

// bytes of float32 slabs a streaming launch of m rows splitting K into `slices` needs
static size_t stream_slab_bytes(int m, int n, int slices)
{
    return slices > 1 ? (size_t) slices * (size_t) m * (size_t) n * 4 : 0;
}

// K slices of a streaming launch (1 = none) and, with a split, the launch shape that goes with it.
// Splitting pays where the activations, re-read by every workgroup, outweigh the weights on the way
// from the L2 to the CUs: several rows, long K, few columns (the down projections).  A workgroup then
// covers more strips over a slice of K, so each activation fragment meets 2-4 times as many weights.
// Measured on MI355X (int4 g128): 14336 x 4096 at M = 16 18.4 -> 12.8 us, M = 8 14.0 -> 12.2, M = 4
// 12.3 -> 11.4; 28672 x 8192 at M = 16 39.9 -> 33.5, M = 8 32.5 -> 29.4; nothing to gain at K <= 8192
// with N >= K or below 4 rows (the finish pass costs ~2.5 us).
int pick_stream_k_slices(int m, int n, int k, int tile_k, int group, size_t workspace_bytes, int shape[4])
{
    (void) group;
    int const k_tiles = (k + tile_k - 1) / tile_k;
    int const strips = n / kTileN;
    shape[0] = 0; // no shape of its own
    int slices = env_overrides().stream_splits;
    if (slices <= 0)
    {
        slices = 1;
        Tactic const* t = current_tactic();
        bool const tuned = t && t->regime == WOQ_REGIME_STREAM && t->ns != 0;
        if (!tuned && !env_overrides().has_stream_shape && m <= 16 && k >= 8192 && k >= 2 * n)
        {
            if (m >= 8 && strips <= 512)
            {
                slices = 4;
                shape[0] = 4, shape[1] = 4, shape[2] = 2, shape[3] = 2;
            }
            else if (m >= 4 && strips <= 256)
            {
                slices = 2;
                shape[0] = 2, shape[1] = 8, shape[2] = 2, shape[3] = 2;
            }
        }
    }
    if (slices > k_tiles)
        slices = k_tiles;
    if (m > 16 || stream_slab_bytes(m, n, slices) > workspace_bytes)
        return 1;
    return slices;
}

int gemm_persistent_workgroups()
{
    if (env_overrides().persist_off)
        return 0;
    // CU count per device ordinal, asked once (0: not yet known)
    static std::atomic<int> cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    {
        (void) hipGetLastError();
        return 0;
    }
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0)
    {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        {
            (void) hipGetLastError();
            return 0;
        }
        n = n / 8 * 8;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool stream_slots_disabled()
{
    return env_overrides().slots_off;
}

namespace
{
EnvOverrides read_env()
{
    EnvOverrides o;
    if (char const* e = std::getenv("WOQ_FORCE_REGIME"))
        o.regime = !std::strcmp(e, "stream") ? WOQ_REGIME_STREAM : (!std::strcmp(e, "gemm") ? WOQ_REGIME_GEMM : 0);
    if (char const* e = std::getenv("WOQ_STREAM_SHAPE"))
        o.has_stream_shape = std::sscanf(e, "%d,%d,%d,%d", &o.stream_shape[0], &o.stream_shape[1], &o.stream_shape[2],
                                 &o.stream_shape[3])
            == 4;
    if (char const* e = std::getenv("WOQ_WIDE_SHAPE"))
        o.wide_mode = std::sscanf(e, "%d,%d,%d", &o.wide_shape[0], &o.wide_shape[1], &o.wide_shape[2]) == 3 ? 1 : 0;
    if (char const* e = std::getenv("WOQ_ROW_SHAPE"))
        o.row_mode = std::sscanf(e, "%d,%d", &o.row_shape[0], &o.row_shape[1]) == 2 ? 1 : 0;
    if (char const* e = std::getenv("WOQ_ROWS_SHAPE"))
        o.rows_mode = std::sscanf(e, "%d,%d,%d", &o.rows_shape[0], &o.rows_shape[1], &o.rows_shape[2]) == 3 ? 1 : 0;
    if (char const* e = std::getenv("WOQ_STREAM_SLOTS"))
        o.slots_off = e[0] == '0';
    if (char const* e = std::getenv("WOQ_GEMM_KERNEL"))
        o.gemm_kernel = !std::strcmp(e, "skinny") ? 2 : 1;
    if (char const* e = std::getenv("WOQ_GEMM_COLS"))
    {
        int const v = std::atoi(e);
        o.gemm_cols = (v == 192 || v == 256) ? v : 0;
    }
    if (char const* e = std::getenv("WOQ_GEMM_RT"))
    {
        int const v = std::atoi(e);
        o.gemm_rt = (v == 4 || v == 8 || v == 16) ? v : 0;
    }
    if (char const* e = std::getenv("WOQ_GEMM_SPLITS"))
        o.gemm_splits = std::atoi(e);
    if (char const* e = std::getenv("WOQ_STREAM_SPLITS"))
        o.stream_splits = std::atoi(e);
    if (char const* e = std::getenv("WOQ_GEMM_PERSIST"))
        o.persist_off = e[0] == '0';
    return o;
}

// the overrides in force: replaced as a whole by woq_reload_env (the old set is left in place for
// calls that still read it; reloading is a test and tuning facility, not a hot path)
std::atomic<EnvOverrides const*> g_env{nullptr};
} // namespace

EnvOverrides const& env_overrides()
{
    EnvOverrides const* e = g_env.load(std::memory_order_acquire);
    if (!e)
    {
        EnvOverrides const* fresh = new EnvOverrides(read_env());
        if (g_env.compare_exchange_strong(e, fresh, std::memory_order_acq_rel))
            return *fresh;
        delete fresh; // another thread was first
    }
    return *e;
}

namespace
{

// Environment override of the regime, for experiments: WOQ_FORCE_REGIME=stream|gemm
int env_regime()
{
    return env_overrides().regime;
}

int validate(woq_matmul_args const* a, MatmulProblem& p)
{
    if (!a)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "args is NULL");
    if (a->m < 0 || a->n <= 0 || a->k <= 0)
        return fail(WOQ_ERR_BAD_SHAPE, "m, n, k must be non-negative / positive (got %d, %d, %d)", a->m, a->n, a->k);
    if (a->out_dtype != WOQ_FP16 && a->out_dtype != WOQ_BF16)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "No valid weightOnlyQuantMatmul configuration: out_dtype must be fp16 or bf16");
    int const algo = a->quant_algo;
    if (algo & ~(WOQ_ALGO_BIAS | WOQ_ALGO_ZERO | WOQ_ALGO_PRE_QUANT_SCALE | WOQ_ALGO_FP8_ALPHA | WOQ_ALGO_INT8_WEIGHT))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_algo bits 0x%x", algo);
    bool const w4a8 = algo & WOQ_ALGO_FP8_ALPHA;
    if (w4a8 && (algo & WOQ_ALGO_INT8_WEIGHT))
        return fail(WOQ_ERR_UNSUPPORTED, "W4A(fp)8 kernel requires INT4 weight!");
    if (a->act_dtype == WOQ_FP8_E4M3)
    {
        if (!w4a8)
            return fail(WOQ_ERR_INVALID_ARGUMENT, "fp8 activations need quant_algo FP8_ALPHA");
        if (algo & WOQ_ALGO_PRE_QUANT_SCALE)
            return fail(WOQ_ERR_INVALID_ARGUMENT, "fp8 activations are already smoothed: PRE_QUANT_SCALE not allowed");
    }
    else if (a->act_dtype != a->out_dtype)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "activation dtype must equal out_dtype (or be fp8 for W4A8)");
    else if (w4a8 && !(algo & WOQ_ALGO_PRE_QUANT_SCALE))
        return fail(WOQ_ERR_INVALID_ARGUMENT,
            "W4A8 with fp16/bf16 activations needs PRE_QUANT_SCALE (the smoothing pass is what casts to fp8)");
    // 64 and 128 as the reference's kernels for every SM; larger multiples of 64 as its Hopper kernels
    // ("The group size must a multiple of <K tile>", launchers/fpA_intB_launcher_sm90.inl:191-198)
    if (a->group_size < 0 || a->group_size % 64)
        return fail(WOQ_ERR_UNSUPPORTED, "group_size must be 0 (per-channel) or a multiple of 64 (got %d)", a->group_size);
    // e4m3 activations: 128 as the reference's pre-Hopper launcher (fpA_intB_gemm_template.h:136-142) and
    // every further multiple of 128 as its Hopper one (launchers/fpA_intB_launcher_sm90.inl:190-198,
    // tests/quantization/test_weight_only_groupwise_quant_matmul.py:429-455)
    if (w4a8 && (a->group_size < 128 || a->group_size % 128))
        return fail(WOQ_ERR_UNSUPPORTED, "W4A8 supports group sizes that are multiples of 128 only (got %d)", a->group_size);
    // m == 0 is a no-op (weightOnlyQuantMatmulPlugin.cpp:303): empty tensors may carry null pointers
    if (a->m > 0 && (!a->act || !a->weight || !a->out))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "act, weight and out must not be NULL");
    if (!a->scales)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "Weight scales must always be set to a non-null value.");
    if (a->group_size == 0 && (a->zeros || (algo & WOQ_ALGO_ZERO)))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "Weight zero pointer must be a nullptr for scale only ops");
    if (((algo & WOQ_ALGO_ZERO) != 0) != (a->zeros != nullptr))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "zeros must be given exactly when quant_algo has ZERO");
    if (((algo & WOQ_ALGO_BIAS) != 0) != (a->bias != nullptr))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "bias must be given exactly when quant_algo has BIAS");
    if (((algo & WOQ_ALGO_PRE_QUANT_SCALE) != 0) != (a->pre_quant_scale != nullptr))
        return fail(WOQ_ERR_INVALID_ARGUMENT, "pre_quant_scale must be given exactly when quant_algo has PRE_QUANT_SCALE");
    int const k_align = w4a8 ? 128 : 64;
    if (a->k % k_align)
        return fail(WOQ_ERR_BAD_SHAPE, "k must be a multiple of %d (got %d)", k_align, a->k);
    // a group size above 128 may leave a shorter last group: the tables then hold ceil(k / group_size) rows
    // (tests/quantization/test_weight_only_groupwise_quant_matmul.py:155, 405-420)
    if (a->group_size && a->group_size <= 128 && a->k % a->group_size)
        return fail(WOQ_ERR_BAD_SHAPE, "k must be a multiple of group_size (got %d, %d)", a->k, a->group_size);
    if (a->n % kTileN)
        return fail(WOQ_ERR_BAD_SHAPE, "n must be a multiple of %d (got %d)", kTileN, a->n);
    if (a->regime != WOQ_REGIME_AUTO && a->regime != WOQ_REGIME_STREAM && a->regime != WOQ_REGIME_GEMM)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown regime %d", a->regime);
    {
        // the kernels address every operand through buffer descriptors with 31-bit byte offsets
        // (the top bit marks a deliberately out-of-range access)
        uint64_t const limit = (uint64_t) 1 << 31;
        uint64_t const act_bytes = (uint64_t) a->m * a->k * (a->act_dtype == WOQ_FP8_E4M3 ? 1 : 2);
        uint64_t const weight_bytes = (uint64_t) a->k * a->n * ((algo & WOQ_ALGO_INT8_WEIGHT) ? 2 : 1) / 2;
        uint64_t const scale_bytes
            = (uint64_t) (a->group_size ? (a->k + a->group_size - 1) / a->group_size : 1) * a->n * 2;
        if (act_bytes >= limit || weight_bytes >= limit || scale_bytes >= limit)
            return fail(WOQ_ERR_UNSUPPORTED,
                "operand too large: activations, one weight matrix and its scales must each stay below 2 GiB "
                "(m=%d n=%d k=%d)", a->m, a->n, a->k);
    }

    p.act = a->act;
    p.pre_quant_scale = a->pre_quant_scale;
    p.weight = a->weight;
    p.scales = a->scales;
    p.zeros = a->zeros;
    p.bias = a->bias;
    p.out = a->out;
    p.alpha = w4a8 ? a->alpha : 1.f;
    p.m = a->m;
    p.n = a->n;
    p.k = a->k;
    p.group_size = a->group_size;
    p.bits = (algo & WOQ_ALGO_INT8_WEIGHT) ? 8 : 4;
    p.out_dtype = a->out_dtype;
    p.act_dtype = a->act_dtype;
    p.w4a8 = w4a8;
    p.workspace = a->workspace;
    p.workspace_bytes = a->workspace_bytes;
    return WOQ_OK;
}

int pick_regime(woq_matmul_args const* a)
{
    int r = a->regime != WOQ_REGIME_AUTO ? a->regime : env_regime();
    if (r == WOQ_REGIME_AUTO && current_tactic())
        r = current_tactic()->regime;
    if (r == WOQ_REGIME_AUTO)
        r = woq_select_regime(a->m, a->n, a->k, a->quant_algo);
    return r;
}

} // namespace
} // namespace woq

using namespace woq;

extern "C" void woq_reload_env(void)
{
    g_env.store(new EnvOverrides(read_env()), std::memory_order_release);
}

extern "C" int woq_select_regime(int32_t m, int32_t n, int32_t k, int32_t quant_algo)
{
    // W4A8: the streaming kernel converts every weight to e4m3 in registers and still runs at
    // memory speed for one 16-row tile; with two tiles per wavefront (17..32 rows) it still beats the
    // fp8 GEMM kernel, whose 64-row tiles convert the same weights for a quarter of the rows, by 8-39 %
    // on the Llama-3-8B / 70B shapes - except on the long-K, narrow-N ones from some row count on (below);
    // beyond that the GEMM kernel
    if (quant_algo & WOQ_ALGO_FP8_ALPHA)
    {
        if (m <= kStreamW4a8AutoMaxM)
            return WOQ_REGIME_STREAM;
        // (long K on few columns: 28672 x 8192 streams up to 30 rows - 28 rows 52.2 against 57.0 us - 14336 x 4096
        // up to 19: 24 rows 25.8 against 22.7)
        if (m <= kStreamW4a8MaxM && !(m > (n <= 4096 ? 19 : 30) && k >= 2 * n))
            return WOQ_REGIME_STREAM;
        return WOQ_REGIME_GEMM;
    }
    // Measured crossover on MI355X: one 16-row tile streams weights at GEMV speed.  With 17..64 rows
    // the streaming kernel (no split-K passes) still wins on small matrices with short K: whichever
    // the two fitted cost models estimate cheaper.  Beyond that the MFMA GEMM kernels are faster.
    if (m <= 16)
        return WOQ_REGIME_STREAM;
    if (m <= 64)
    {
        int const bits = (quant_algo & WOQ_ALGO_INT8_WEIGHT) ? 8 : 4;
        if (stream_cost_us(m, n, k) < plan_gemm(m, n, k, bits).cost_us)
            return WOQ_REGIME_STREAM;
    }
    return WOQ_REGIME_GEMM;
}

namespace
{
inline size_t align256(size_t v)
{
    return (v + 255) & ~(size_t) 255;
}

// bytes of the smoothed-activation region at the front of the workspace
size_t smooth_bytes(int m, int k, int quant_algo)
{
    return (quant_algo & WOQ_ALGO_PRE_QUANT_SCALE) ? align256((size_t) m * (size_t) k * 2) : 0;
}
} // namespace

// float32 slabs the streaming kernel may use for a K split with at most m rows
static size_t stream_workspace_bytes(int m, int n, int k, int quant_algo)
{
    if (quant_algo & WOQ_ALGO_FP8_ALPHA)
        return 0;
    int const tile_k = tile_k_of_bits((quant_algo & WOQ_ALGO_INT8_WEIGHT) ? 8 : 4);
    size_t need = 0;
    for (int rows = 1; rows <= (m < 16 ? m : 16); ++rows)
    {
        int shape[4];
        size_t const b = stream_slab_bytes(rows, n, pick_stream_k_slices(rows, n, k, tile_k, 0, (size_t) -1, shape));
        need = b > need ? b : need;
    }
    return need;
}

// float32 partial buffer of one GEMM-regime call with exactly m rows
// (group: the problem's group size, or -1 for a caller that does not know it - the plan may depend on
// it, so such a caller gets the larger of the candidates)
static size_t split_bytes(int m, int n, int k, int quant_algo, int group = -1)
{
    if (quant_algo & WOQ_ALGO_FP8_ALPHA)
        return plan_gemm_w4a8(m, n, k).ws_bytes;
    int const bits = (quant_algo & WOQ_ALGO_INT8_WEIGHT) ? 8 : 4;
    if (group >= 0)
        return planned_gemm(m, n, k, bits, group).ws_bytes;
    size_t const a = planned_gemm(m, n, k, bits, -1).ws_bytes, b = planned_gemm(m, n, k, bits, 128).ws_bytes;
    return a > b ? a : b;
}

// what one GEMM-regime call with exactly m rows uses
static size_t gemm_workspace_bytes(int m, int n, int k, int quant_algo, int group = -1)
{
    return smooth_bytes(m, k, quant_algo) + split_bytes(m, n, k, quant_algo, group);
}

extern "C" size_t woq_workspace_bytes(int32_t m, int32_t n, int32_t k, int32_t quant_algo, int32_t act_dtype)
{
    (void) act_dtype;
    if (m <= 0 || k <= 0 || n <= 0)
        return 0;
    // Enough for every call with at most m rows (the reference sizes its workspace for the
    // profile's largest M the same way), in either regime.  The smoothing region grows with m;
    // the split-K region does not (large m does not split, small m splits most), so take its
    // maximum over the row counts up to m.
    size_t bytes = smooth_bytes(m, k, quant_algo);
    // A plan splits K only while tiles * splits <= 512, which even the tallest (256-row) tiles exceed
    // beyond 256 * (256 / column tiles) rows; below that the plan may change at any row count.
    // Within a class of 16 rows every candidate has the same tiles, and the partial traffic, which
    // grows with the rows, only ever favours fewer splits: the splits of the class's first row count
    // times its last row count bound the class.
    size_t split = split_bytes(m, n, k, quant_algo);
    int const col_tiles = (n + 255) / 256;
    int const cap = 256 * (col_tiles >= 256 ? 1 : 256 / col_tiles);
    int const top = m - 1 < cap ? m - 1 : cap;
    for (int lo = 1; lo <= top; lo += 16)
    {
        int const hi = lo + 15 < top ? lo + 15 : top;
        size_t const per_row = split_bytes(lo, n, k, quant_algo) / (size_t) lo;
        split = per_row * hi > split ? per_row * hi : split;
    }
    size_t const tuned = tuned_split_bytes(m, n, k, quant_algo);
    bytes += split > tuned ? split : tuned;
    // the streaming regime's own K split (16-bit activations, at most 16 rows)
    size_t const stream = stream_workspace_bytes(m, n, k, quant_algo);
    return bytes > stream ? bytes : stream;
}

extern "C" int woq_matmul_check(const woq_matmul_args* args)
{
    MatmulProblem p;
    if (int rc = validate(args, p))
        return rc;
    int const regime = pick_regime(args);
    int const stream_max_m = p.w4a8 ? kStreamW4a8MaxM : kStreamMaxM;
    if (regime == WOQ_REGIME_STREAM && args->m > stream_max_m)
        return fail(WOQ_ERR_UNSUPPORTED, "unsupported m: the streaming kernel covers m <= %d (got %d)", stream_max_m,
            args->m);
    if (p.m > 0 && (regime == WOQ_REGIME_GEMM || p.w4a8))
    {
        // the W4A8 streaming kernel reads e4m3 activations: 16-bit ones go through the smoothing
        // pass (and its workspace region) in either regime
        size_t const need = regime == WOQ_REGIME_GEMM ? gemm_workspace_bytes(p.m, p.n, p.k, args->quant_algo, p.group_size)
                                                      : smooth_bytes(p.m, p.k, args->quant_algo);
        if (need && (!p.workspace || p.workspace_bytes < need))
            return fail(WOQ_ERR_WORKSPACE, "workspace of %zu bytes required, %zu given", need,
                p.workspace ? p.workspace_bytes : (size_t) 0);
    }
    return WOQ_OK;
}

static int run_matmul(const woq_matmul_args* args, void* stream);

extern "C" int woq_matmul(const woq_matmul_args* args, void* stream)
{
    // a tuned tactic for this problem, unless the caller, the environment or a profiling run
    // already fixed the choice, or the workspace given is too small for it
    Tactic tuned;
    if (args && args->regime == WOQ_REGIME_AUTO && !current_tactic() && env_regime() == WOQ_REGIME_AUTO
        && find_tactic(*args, tuned))
    {
        TacticScope scope(&tuned);
        if (woq_matmul_check(args) == WOQ_OK)
        {
            // an imported entry may name a launch shape this build does not have: nothing has been
            // launched then, and the heuristics take over
            int const rc = run_matmul(args, stream);
            if (rc != WOQ_ERR_UNSUPPORTED)
                return rc;
        }
    }
    return run_matmul(args, stream);
}

static int run_matmul(const woq_matmul_args* args, void* stream)
{
    if (int rc = woq_matmul_check(args))
        return rc;
    MatmulProblem p;
    validate(args, p);
    if (p.m == 0)
        return WOQ_OK;
    bool const streaming = pick_regime(args) == WOQ_REGIME_STREAM;
    if (streaming && !p.w4a8)
        return launch_stream(p, stream); // smoothing is fused into the 16-bit streaming kernel
    if (p.pre_quant_scale)
    {
        // smoothing pass into the workspace, then the GEMM reads the smoothed activations
        int const smoothed_dtype = p.w4a8 ? WOQ_FP8_E4M3 : p.out_dtype;
        if (int rc = launch_prequant(
                p.workspace, p.act, p.pre_quant_scale, p.m, p.k, p.out_dtype, smoothed_dtype, stream))
            return rc;
        p.act = p.workspace;
        p.act_dtype = smoothed_dtype;
        p.pre_quant_scale = nullptr;
        size_t const used = smooth_bytes(p.m, p.k, args->quant_algo);
        p.workspace = static_cast<char*>(p.workspace) + used;
        p.workspace_bytes -= used;
    }
    return streaming ? launch_stream(p, stream) : launch_gemm(p, stream);
}

// ---- woq_matmul_static: the matmul for callers that cannot allocate ----------------------------
// The split-K partial sums and the smoothed activations of the GEMM regime live in a file-scope
// device array instead of a caller workspace.  In host code the array's NAME is only a stand-in
// for the symbol: its device address is looked up once per device (every GPU holds its own copy
// at its own address) and that pointer is what the kernels, through the workspace fields, receive.
static __device__ __align__(256) unsigned char scratch[WOQ_STATIC_SCRATCH_BYTES];

namespace
{
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device (looked up on the first call there)
int static_scratch_ptr(void** out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
    {
        (void) hipGetLastError();
        return fail(WOQ_ERR_RUNTIME, "hipGetDevice failed: %s", hipGetErrorString(e));
    }
    if (dev < 0 || dev >= kMaxDevices)
        return fail(WOQ_ERR_RUNTIME, "device ordinal %d is beyond the %d this library keeps scratch pointers for", dev,
            kMaxDevices);
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr)
    {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
        {
            (void) hipGetLastError();
            return fail(WOQ_ERR_RUNTIME, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
        }
        g_scratch_ptr[dev].store(ptr, std::memory_order_release); // racing first calls store the same address
    }
    *out = ptr;
    return WOQ_OK;
}
} // namespace

extern "C" size_t woq_static_scratch_bytes(void)
{
    return WOQ_STATIC_SCRATCH_BYTES;
}

extern "C" int woq_static_init(void)
{
    (void) env_overrides(); // read (and allocate, on the host) once, here rather than inside a first call
    void* ptr = nullptr;
    return static_scratch_ptr(&ptr);
}

extern "C" int woq_matmul_static(const woq_matmul_args* args, void* stream)
{
    if (!args)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "args is NULL");
    woq_matmul_args a = *args;
    a.workspace = nullptr;
    a.workspace_bytes = 0;
    // what this very call needs (the regime and plan woq_matmul would take without a tuned table
    // entry that wants more room: with too little workspace it falls back to the built-in choice)
    MatmulProblem p;
    if (int rc = validate(&a, p))
        return rc;
    if (p.m == 0)
        return WOQ_OK;
    int const regime = pick_regime(&a);
    size_t need = 0;
    if (regime == WOQ_REGIME_GEMM)
        need = gemm_workspace_bytes(p.m, p.n, p.k, a.quant_algo, p.group_size);
    else if (p.w4a8)
        need = smooth_bytes(p.m, p.k, a.quant_algo);
    else
    {
        // the streaming kernel splits K only if it is given room for the slabs: offer the scratch
        // when they fit, else it runs without the split
        need = stream_workspace_bytes(p.m, p.n, p.k, a.quant_algo);
        if (need > (size_t) WOQ_STATIC_SCRATCH_BYTES)
            need = 0;
    }
    if (need > (size_t) WOQ_STATIC_SCRATCH_BYTES)
        return fail(WOQ_ERR_WORKSPACE,
            "woq_matmul_static: this call needs %zu bytes of scratch, the static scratch holds %zu; use woq_matmul "
            "with a caller workspace",
            need, (size_t) WOQ_STATIC_SCRATCH_BYTES);
    if (need)
    {
        void* ptr = nullptr;
        if (int rc = static_scratch_ptr(&ptr))
            return rc;
        a.workspace = ptr;
        a.workspace_bytes = WOQ_STATIC_SCRATCH_BYTES;
    }
    return woq_matmul(&a, stream);
}

namespace
{
// Kernel family of a grouped problem.  Only the total row count is known on the host, so the choice
// goes by the average expert: streaming passes of 16 rows while that is at most 16 rows, else the
// tiled kernels (kernel and tile height by plan_gemm's estimate for the average expert; K is
// never split).
int grouped_regime(woq_grouped_matmul_args const* a)
{
    int r = a->base.regime != WOQ_REGIME_AUTO ? a->base.regime : env_regime();
    if (r == WOQ_REGIME_AUTO)
        r = (int64_t) a->base.m <= (int64_t) 16 * a->num_experts ? WOQ_REGIME_STREAM : WOQ_REGIME_GEMM;
    return r;
}

} // namespace

extern "C" int woq_grouped_matmul_check(const woq_grouped_matmul_args* args)
{
    if (!args)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "args is NULL");
    MatmulProblem p;
    if (int rc = validate(&args->base, p))
        return rc;
    if (p.w4a8 || p.pre_quant_scale)
        return fail(WOQ_ERR_UNSUPPORTED, "grouped matmul: FP8_ALPHA and PRE_QUANT_SCALE are not supported");
    if (args->num_experts <= 0)
        return fail(WOQ_ERR_BAD_SHAPE, "num_experts must be positive (got %d)", args->num_experts);
    if (p.m > 0 && !args->total_rows_before_expert && args->num_experts != 1)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "total_rows_before_expert must not be NULL (unless num_experts is 1)");
    int const act = args->activation;
    if (act < WOQ_ACT_GELU || act > WOQ_ACT_IDENTITY)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown activation %d", act);
    bool const gated = act == WOQ_ACT_SWIGLU || act == WOQ_ACT_GEGLU;
    if (gated && p.n % 32)
        return fail(WOQ_ERR_BAD_SHAPE, "a gated activation needs n %% 32 == 0 (got %d)", p.n);
    int const r = args->base.regime;
    if (r != WOQ_REGIME_AUTO && r != WOQ_REGIME_STREAM && r != WOQ_REGIME_GEMM)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown regime %d", r);
    // the kernels address the residual with 32-bit byte offsets
    if (args->residual && (uint64_t) p.m * (uint64_t) p.n * 2 >= ((uint64_t) 1 << 32))
        return fail(WOQ_ERR_UNSUPPORTED, "residual: total_rows * n * 2 must stay below 4 GiB (got %d x %d)", p.m, p.n);
    return WOQ_OK;
}

extern "C" int woq_grouped_matmul(const woq_grouped_matmul_args* args, void* stream)
{
    if (int rc = woq_grouped_matmul_check(args))
        return rc;
    MatmulProblem p;
    validate(&args->base, p);
    if (p.m == 0)
        return WOQ_OK;
    p.weight_stride = woq_preprocessed_bytes(p.k, p.n, p.bits == 8 ? WOQ_W8_A16 : WOQ_W4_A16);
    p.scale_stride = (size_t) (p.group_size ? (p.k + p.group_size - 1) / p.group_size : 1) * (size_t) p.n * 2;
    int const act = args->activation;
    bool const gated = act == WOQ_ACT_SWIGLU || act == WOQ_ACT_GEGLU;
    // without the prefix sums (one expert owning every row) the kernels take the row count from m
    bool const single = !args->total_rows_before_expert;
    p.expert_rows = args->total_rows_before_expert;
    p.num_experts = args->num_experts;
    p.workspace = nullptr; // K is never split here
    p.workspace_bytes = 0;
    // every kernel applies a gated activation in its epilogue; the streaming kernel the others too
    bool const streaming = grouped_regime(args) == WOQ_REGIME_STREAM;
    p.activation = (streaming || gated) ? act : WOQ_ACT_IDENTITY;
    p.residual = args->residual;
    if (streaming)
        return launch_stream(p, stream);
    // no K split: the tiles of one expert are not what is short here, and the epilogue fusions need the sums
    GemmPlan const plan = plan_gemm(p.m, p.n, p.k, p.bits, false, single ? 1 : p.num_experts, p.group_size);
    bool const two_pass = act != WOQ_ACT_IDENTITY && !gated;
    if (two_pass)
        p.residual = nullptr; // added behind the activation, by the pass below
    if (int rc = launch_gemm_planned(p, plan, stream))
        return rc;
    if (!two_pass)
        return WOQ_OK;
    return launch_activation(p.out, p.out, args->residual, p.m, p.n, act, p.out_dtype, stream); // in place
}

extern "C" int woq_apply_per_channel_scale(void* out, const void* act, const void* per_channel_scale, int32_t m,
    int32_t k, int32_t in_dtype, int32_t out_dtype, void* stream)
{
    if (!out || !act || !per_channel_scale)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_apply_per_channel_scale: null pointer");
    if (in_dtype != WOQ_FP16 && in_dtype != WOQ_BF16)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "input dtype must be fp16 or bf16");
    if (out_dtype != in_dtype && out_dtype != WOQ_FP8_E4M3)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "output dtype must be the input dtype or fp8 e4m3");
    if (m < 0 || k <= 0 || k % 8)
        return fail(WOQ_ERR_BAD_SHAPE, "m >= 0 and k %% 8 == 0 required (got %d, %d)", m, k);
    if (m == 0)
        return WOQ_OK;
    return launch_prequant(out, act, per_channel_scale, m, k, in_dtype, out_dtype, stream);
}

extern "C" int woq_rmsnorm_prequant(void* out, const void* x, const void* gamma, const void* beta,
    const void* pre_quant_scale, float eps, int32_t m, int32_t k, int32_t dtype, int32_t out_dtype, void* stream)
{
    if (!out || !x || !gamma)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_rmsnorm_prequant: null pointer");
    if (dtype != WOQ_FP16 && dtype != WOQ_BF16)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "input dtype must be fp16 or bf16");
    if (out_dtype != dtype && out_dtype != WOQ_FP8_E4M3)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "output dtype must be the input dtype or fp8 e4m3");
    if (m < 0 || k <= 0 || k % 8)
        return fail(WOQ_ERR_BAD_SHAPE, "m >= 0 and k %% 8 == 0 required (got %d, %d)", m, k);
    if (m == 0)
        return WOQ_OK;
    return launch_rmsnorm_prequant(out, x, gamma, beta, pre_quant_scale, eps, m, k, dtype, out_dtype, stream);
}

extern "C" int woq_dequantize(void* out, const void* weight, const void* scales, const void* zeros, int32_t k,
    int32_t n, int32_t group_size, int32_t quant_type, int32_t dtype, void* stream)
{
    if (!out || !weight || !scales)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_dequantize: null pointer");
    if (quant_type != WOQ_W8_A16 && quant_type != WOQ_W4_A16 && quant_type != WOQ_W4_AFP8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_type %d", quant_type);
    if (dtype != WOQ_FP16 && dtype != WOQ_BF16 && dtype != WOQ_FP8_E4M3)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "dtype must be fp16, bf16 or fp8 e4m3");
    if (k <= 0 || n <= 0 || n % kTileN || k % 32)
        return fail(WOQ_ERR_BAD_SHAPE, "k %% 32 == 0 and n %% 16 == 0 required (got %d, %d)", k, n);
    if (group_size < 0 || group_size % 64)
        return fail(WOQ_ERR_UNSUPPORTED, "group_size must be 0 or a multiple of 64 (got %d)", group_size);
    if (group_size && group_size <= 128 && k % group_size)
        return fail(WOQ_ERR_BAD_SHAPE, "k must be a multiple of group_size");
    return launch_dequant(out, weight, scales, zeros, k, n, group_size, bits_of(quant_type), dtype, stream);
}
