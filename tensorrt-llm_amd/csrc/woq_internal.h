// Internal declarations shared by the host code and the kernel launchers of libwoq.
#pragma once

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <initializer_list>

#include "../../include/woq.h"

namespace woq
{

// records a message for woq_last_error() on this thread and returns `code`
int fail(int code, char const* fmt, ...) __attribute__((format(printf, 2, 3)));

// remembers what woq_last_launch() reports for this thread (`fmt` must be a string literal with up
// to six %d; formatted only when asked for)
void note_launch(char const* fmt, int a = 0, int b = 0, int c = 0, int d = 0, int e = 0, int f = 0);

inline int bits_of(int quant_type)
{
    return quant_type == WOQ_W8_A16 ? 8 : 4;
}

// Experiment overrides from the environment, read once (at first use) and again by woq_reload_env():
//   WOQ_FORCE_REGIME=stream|gemm      WOQ_STREAM_SHAPE=ns,waves,pf,lds   WOQ_WIDE_SHAPE=ns,waves,pf | 0
//   WOQ_STREAM_SLOTS=0                WOQ_GEMM_KERNEL=exact|skinny       WOQ_GEMM_RT=4|8|16
//   WOQ_GEMM_SPLITS=<n>               WOQ_STREAM_SPLITS=<n>              WOQ_GEMM_PERSIST=0
//   WOQ_GEMM_COLS=192|256             WOQ_ROW_SHAPE=waves,tiles | 0      WOQ_ROWS_SHAPE=waves,ns,tiles | 0
struct EnvOverrides
{
    int regime = 0;                // woq_regime; 0 = none
    bool has_stream_shape = false; // streaming kernels: strips per wavefront, wavefronts, tile rows in flight, LDS mode
    int stream_shape[4] = {0, 0, 0, 0};
    int wide_mode = -1;            // wide streaming kernel: -1 built-in rule, 0 off, 1 forced shape
    int wide_shape[3] = {0, 0, 0};
    int row_mode = -1;             // single-row streaming kernel: -1 built-in rule, 0 off, 1 forced shape
    int row_shape[2] = {0, 0};     // wavefronts per workgroup, tiles per wavefront and pass
    int rows_mode = -1;            // multi-row streaming kernel (stream_rows_kernel.h): -1 built-in rule, 0 off, 1 forced shape
    int rows_shape[3] = {0, 0, 0}; // wavefronts per workgroup, strips per workgroup, tile rows per wavefront and pass
    bool slots_off = false;        // no group-slot variants of the streaming kernel
    int gemm_kernel = 0;           // 0 any, 1 exact-dequantize, 2 deferred-scale
    int gemm_rt = 0;               // row tiles per wavefront of the exact-dequantize / fp8 kernel
    int gemm_cols = 0;             // columns of a 256-row tile of the exact-dequantize kernel (192 needs n % 192 == 0)
    int gemm_splits = 0;           // K split of the GEMM regime
    int stream_splits = 0;         // K slices of the streaming kernel (0 = built-in rule)
    bool persist_off = false;      // WOQ_GEMM_PERSIST=0: no persistent prefill kernels
};
EnvOverrides const& env_overrides();

// rows of K covered by one 1 KiB weight tile (16 columns wide)
inline int tile_k_of_bits(int bits)
{
    return bits == 4 ? 128 : 64;
}

constexpr int kTileN = 16;

// Arguments every device launcher receives; validated by the caller.
struct MatmulProblem
{
    void const* act;
    void const* pre_quant_scale;
    void const* weight;
    void const* scales;
    void const* zeros;
    void const* bias;
    void* out;
    float alpha;
    int m, n, k;
    int group_size; // 0 = one scale per column
    int bits;       // 4 or 8
    int out_dtype;  // WOQ_FP16 / WOQ_BF16
    int act_dtype;  // WOQ_FP16 / WOQ_BF16 / WOQ_FP8_E4M3
    bool w4a8;
    void* workspace;
    size_t workspace_bytes;
    // grouped (mixture-of-experts) problems: rows sorted by expert, expert_rows[e] = rows of experts
    // 0..e (device memory); m is then the total row count and the strides are bytes per expert
    int64_t const* expert_rows = nullptr;
    int num_experts = 0;
    size_t weight_stride = 0, scale_stride = 0;
    int activation = 5;             // WOQ_ACT_IDENTITY; see woq_grouped_matmul
    void const* residual = nullptr; // [m, n_out] in the output type, added after the activation
};

// kernel launchers (each returns a woq_status)
int launch_stream(MatmulProblem const& p, void* stream);
int launch_gemm(MatmulProblem const& p, void* stream);
int launch_prequant(void* out, void const* act, void const* scale, int m, int k, int in_dtype, int out_dtype,
    void* stream);
int launch_rmsnorm_prequant(void* out, void const* x, void const* gamma, void const* beta, void const* scale, float eps,
    int m, int k, int dtype, int out_dtype, void* stream);
int launch_activation(void* out, void const* in, void const* residual, long m, int n_in, int act, int dtype,
    void* stream);
int launch_dequant(void* out, void const* weight, void const* scales, void const* zeros, int k, int n, int group_size,
    int bits, int dtype, void* stream);

// How the GEMM regime runs a problem: which kernel, rows per output tile and the number of
// workgroups that split K for one tile (each with its own float32 slab of the ws_bytes when > 1).
struct GemmPlan
{
    bool skinny;  // deferred-scale 64-row kernel instead of the exact-dequantize prefill kernel
    int rt;       // row tiles per wavefront (tile rows = 16 * rt)
    int k_splits;
    size_t ws_bytes;
    double cost_us; // the cost model's estimate (plan_gemm only)
};

// float32 partial sums of a K split: one [m, n] slab per slice of K
inline size_t split_partial_bytes(int m, int n, int k_splits)
{
    return k_splits > 1 ? (size_t) m * (size_t) n * 4 * (size_t) k_splits : 0;
}

// Output tiles (of 16*rt rows x 256 columns) a problem has.
inline long gemm_tiles(int m, int n, int rt)
{
    return (long) ((m + rt * 16 - 1) / (rt * 16)) * ((n + 255) / 256);
}

// Estimated time (microseconds) of a 16-bit GEMM-regime problem on one kernel, tile height and K
// split, from a model fitted to sweeps over the Llama-3-8B / 70B layer shapes (M = 32 .. 1024, int4
// g128 and int8 per-channel, every kernel / tile height / split count from 1 to 20: picking by it
// stays within 1.6 % of the best measured choice on average, 15 % at worst):
//   * a workgroup spends c microseconds per tile row of K (c = a + b * rt for the exact-dequantize
//     kernel: the dequantize is paid once per workgroup, the MFMAs per row; a constant for the
//     deferred-scale kernel's 64- or 32-row tile) plus a prologue / epilogue of 1.7 - 3 us per tile;
//   * one workgroup per CU: ceil(workgroups / 256) rounds of tiles one after another (counted on the
//     fullest XCD), and a last round of more than 224 workgroups runs ~10 % longer (measured: 256
//     workgroups are no faster than 192, and 257 take two rounds);
//   * splitting K costs the reduction launch and the float32 partial slabs (written once, read once).
// `tiles` is the output tile count of that tile height (for a grouped problem: over all experts).
inline double gemm_cost_us(bool skinny, int rt, long tiles, int m, int n, int k, int bits, int splits, int group = -1)
{
    int const tk = tile_k_of_bits(bits);
    int const k_tiles = (k + tk - 1) / tk;
    double c;
    if (skinny)
        // (two row tiles: 0.79 before the A fragments were read a step ahead; four row tiles at group size 128:
        // 1.19 before the fragments were read just in time and placed free of LDS bank conflicts, re-measured
        // against the exact-dequantize kernel at 48 ... 128 rows since - `group` is -1 where the caller does not
        // know it)
        c = bits == 4 ? (rt == 2 ? 0.73 : (group == 128 ? 1.03 : 1.29)) : 0.565;
    else
        c = bits == 4 ? 0.807 + 0.108 * rt : 0.642 + 0.0404 * rt;
    // the tiles are dealt to the 8 XCDs (32 CUs each) in equal contiguous runs: the fullest XCD
    // sets the number of rounds
    long const wgs = (tiles + 7) / 8 * splits;
    long const rounds = (wgs + 31) / 32;
    int const steps = (k_tiles + splits - 1) / splits;
    double const last_round = wgs - (rounds - 1) * 32 > 28 ? 0.10 : 0.0;
    double const per_tile = skinny ? 3.15 : 1.34 + 0.081 * rt; // prologue and epilogue
    double t = ((double) rounds + last_round) * (steps * c + per_tile) + 2.25;
    if (splits > 1)
        t += 2.9 + (double) m * n * 4.0 * splits * 3.3e-7;
    return t;
}

// The K split (1 = none) that gemm_cost_us estimates cheapest for this kernel and tile height, and
// its cost.  A split leaves every workgroup at least four tile rows of K.
inline double gemm_best_split(bool skinny, int rt, long tiles, int m, int n, int k, int bits, bool allow_split, int& splits,
    int group = -1)
{
    int const tk = tile_k_of_bits(bits);
    int const k_tiles = (k + tk - 1) / tk;
    splits = 1;
    double best = gemm_cost_us(skinny, rt, tiles, m, n, k, bits, 1, group);
    if (!allow_split || k_tiles < 8)
        return best;
    for (int s = 2; s <= k_tiles / 4 && tiles * s <= 512; ++s)
    {
        double const t = gemm_cost_us(skinny, rt, tiles, m, n, k, bits, s, group);
        if (t < best)
        {
            best = t;
            splits = s;
        }
    }
    return best;
}

// Kernel, tile height and K split of a 16-bit GEMM-regime problem: the cheapest by gemm_cost_us of
//   * the deferred-scale kernel (32-row tiles for int4 up to 32 rows, else 64-row tiles);
//   * the exact-dequantize kernel with 64-, 128- or 256-row tiles.
// Environment overrides for experiments: WOQ_GEMM_KERNEL=exact|skinny, WOQ_GEMM_RT=4|8|16 (exact
// kernel), WOQ_GEMM_SPLITS=<n>
inline GemmPlan plan_gemm(int m, int n, int k, int bits, bool allow_split = true, int num_experts = 1, int group = -1)
{
    // rows per expert of a grouped problem (its tiles do not straddle experts)
    int const rows = num_experts > 1 ? (m + num_experts - 1) / num_experts : m;
    int const skinny_rt = (rows <= 32 && bits == 4) ? 2 : 4;
    EnvOverrides const& env = env_overrides();
    int const forced_rt = env.gemm_rt;
    GemmPlan pl{};
    double best = 0;
    bool have = false;
    for (int cand = 0; cand < 4; ++cand)
    {
        bool const skinny = cand == 0;
        int const rt = skinny ? skinny_rt : (cand == 1 ? 4 : (cand == 2 ? 8 : 16));
        if (env.gemm_kernel && skinny != (env.gemm_kernel == 2))
            continue;
        if (!skinny && forced_rt && rt != forced_rt)
            continue;
        int splits;
        double const cost = gemm_best_split(
            skinny, rt, (long) num_experts * gemm_tiles(rows, n, rt), m, n, k, bits, allow_split, splits, group);
        if (!have || cost < best)
        {
            have = true;
            best = cost;
            pl.skinny = skinny;
            pl.rt = rt;
            pl.k_splits = splits;
        }
    }
    int const tk = tile_k_of_bits(bits);
    int const k_tiles = (k + tk - 1) / tk;
    if (allow_split && env.gemm_splits >= 1 && env.gemm_splits <= k_tiles)
        pl.k_splits = env.gemm_splits;
    pl.ws_bytes = split_partial_bytes(m, n, pl.k_splits);
    pl.cost_us = best;
    return pl;
}

// Strips (16 output columns) per workgroup of the streaming kernel for 17..64 rows: one up to 256
// column strips, else two (257..511 workgroups, a partly filled second round over the 256 CUs,
// measured 40-60 % slower than half as many workgroups of twice the width).
inline int stream_mid_ns(int strips)
{
    return strips > 256 ? 2 : 1;
}

// Estimated time (microseconds) of the streaming kernel on 17..64 rows, fitted to the Llama-3-8B / 70B
// layer shapes and N = 2048 / 5120 (int4 and int8 read at the same rate here): every workgroup walks
// all of K, at a rate that falls with the rows it carries, in ceil(workgroups / 256) rounds.
inline double stream_cost_us(int m, int n, int k)
{
    int const strips = (n + 15) / 16;
    int const ns = stream_mid_ns(strips);
    long const groups = (strips + ns - 1) / ns;
    long const rounds = (groups + 255) / 256;
    int const rows = m > 32 ? m + 6 : m; // the step from two to four row tiles per wavefront
    double const per_1024 = ns == 1 ? 0.7 + 0.045 * rows : 0.6 + 0.06 * rows;
    return 3.0 + (double) rounds * k / 1024.0 * per_1024;
}

// W4A8 runs on one kernel (exact dequantize to e4m3, 64/128/256-row tiles, optional split-K).
// Estimated time (microseconds) of one tile height and K split: the same model as gemm_cost_us,
// fitted to a sweep of the fp8 kernel over the Llama-3-8B / 70B shapes (M = 32 .. 4096, every tile
// height, splits 1 .. 20): picking by it stays within 0.4 % of the best measured choice on average.
inline double w4a8_cost_us(int rt, long tiles, int m, int n, int k, int splits)
{
    int const k_tiles = (k + 127) / 128;
    long const wgs = (tiles + 7) / 8 * splits; // on the fullest XCD
    long const rounds = (wgs + 31) / 32;
    int const steps = (k_tiles + splits - 1) / splits;
    double const last_round = wgs - (rounds - 1) * 32 > 28 ? 0.04 : 0.0;
    double t = ((double) rounds + last_round) * (steps * (1.13 + 0.044 * rt) + 2.09) + 4.6;
    if (splits > 1)
        t += 2.5 + (double) m * n * 4.0 * (2 + 2 * splits) * 1.29e-7;
    return t;
}

inline GemmPlan plan_gemm_w4a8(int m, int n, int k)
{
    GemmPlan pl{};
    pl.skinny = false;
    int const k_tiles = (k + 127) / 128;
    EnvOverrides const& env = env_overrides();
    int const forced_rt = env.gemm_rt;
    int const forced_splits = env.gemm_splits >= 1 && env.gemm_splits <= k_tiles ? env.gemm_splits : 0;
    bool have = false;
    for (int rt = 4; rt <= 16; rt *= 2)
    {
        if (forced_rt ? rt != forced_rt : ((rt == 8 && m <= 64) || (rt == 16 && m <= 128)))
            continue;
        long const tiles = gemm_tiles(m, n, rt);
        int const max_s = forced_splits ? forced_splits : (k_tiles >= 8 ? k_tiles / 4 : 1);
        for (int s = forced_splits ? forced_splits : 1; s <= max_s && (s == 1 || forced_splits || tiles * s <= 512); ++s)
        {
            double const t = w4a8_cost_us(rt, tiles, m, n, k, s);
            if (!have || t < pl.cost_us)
            {
                have = true;
                pl.cost_us = t;
                pl.rt = rt;
                pl.k_splits = s;
            }
        }
    }
    pl.ws_bytes = split_partial_bytes(m, n, pl.k_splits);
    return pl;
}

// One way to run a 16-bit problem: the regime and, inside it, the streaming kernel's launch shape
// (for problems of `mt` 16-row tiles) or the GEMM kernel, tile height and K split.  Counterpart of
// the reference's CutlassGemmConfig with its enableCudaKernel pseudo-tactic
// (cutlass_heuristic.cpp:393-441).
struct Tactic
{
    int regime;               // WOQ_REGIME_STREAM or WOQ_REGIME_GEMM
    int mt, ns, waves, pf, lds; // streaming launch shape
    int skinny, rt, k_splits; // GEMM plan
};

// The tactic in force for the call running on this thread (set while profiling, or from the tuned
// table by woq_matmul); nullptr: every choice is the heuristics'.
Tactic const* current_tactic();
struct TacticScope
{
    explicit TacticScope(Tactic const* t);
    ~TacticScope();
    Tactic const* prev;
};
// Tuned table (filled by woq_profile_tactics / woq_import_tactics): the entry of exactly m rows,
// else of the smallest profiled row count above m.
bool find_tactic(woq_matmul_args const& a, Tactic& out);
// float32 split-K bytes the tuned entries of this n, k, quant_algo may use for at most m rows
size_t tuned_split_bytes(int m, int n, int k, int quant_algo);

// Raises a kernel's dynamic-LDS limit to `bytes` (hipFuncSetAttribute) on the current device, once per
// device: `raised` holds one bit per device ordinal below 64 (for ordinals from 64 on the idempotent
// call is simply repeated at every launch).  The sticky HIP error of a failed call is cleared.
int raise_lds_once(std::atomic<uint64_t>& raised, void const* kernel, int bytes);

// largest M the streaming kernels are instantiated for (16-bit activations; W4A8)
constexpr int kStreamMaxM = 128;
constexpr int kStreamW4a8MaxM = 32;     // rows the W4A8 streaming kernel covers (two 16-row tiles per wavefront above 16)
constexpr int kStreamW4a8AutoMaxM = 16; // rows up to which the built-in rule takes it
// most LDS a streaming workgroup stages its operands in (activations, group scales and zeros, row
// sums): what the CU's 160 KiB leave next to the static reduction buffer of the epilogue
// (`slots` = strips per wavefront x 16-row tiles, 256 floats per slot and wavefront)
constexpr size_t stream_max_staged_lds(int slots, int waves)
{
    return (size_t) 160 * 1024 - (size_t) waves * slots * 1024 - 2048;
}

} // namespace woq
