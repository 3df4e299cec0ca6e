// Internal declarations shared by the host code and the kernel launchers of libwoq.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/woq.h"

namespace woq
{

// records a message for woq_last_error() on this thread and returns `code`
int fail(int code, char const* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int bits_of(int quant_type)
{
    return quant_type == WOQ_W8_A16 ? 8 : 4;
}

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
};

// kernel launchers (each returns a woq_status)
int launch_stream(MatmulProblem const& p, void* stream);
int launch_gemm(MatmulProblem const& p, void* stream);
int launch_prequant(void* out, void const* act, void const* scale, int m, int k, int in_dtype, int out_dtype,
    void* stream);
int launch_dequant(void* out, void const* weight, void const* scales, void const* zeros, int k, int n, int group_size,
    int bits, int dtype, void* stream);

// How the GEMM regime runs a problem: which kernel, rows per output tile and the number of
// workgroups that split K for one tile (with a float32 partial buffer of ws_bytes when > 1).
struct GemmPlan
{
    bool skinny;  // deferred-scale 64-row kernel instead of the exact-dequantize prefill kernel
    int rt;       // row tiles per wavefront (tile rows = 16 * rt)
    int k_splits;
    size_t ws_bytes;
};

// The deferred-scale 64-row kernel is preferred up to 256 rows, and up to 512 rows when N is narrow
// (few column panels: the 256-row tiles of the prefill kernel would leave most CUs idle).
inline bool prefer_skinny(int m, int n)
{
    return m <= 256 || (m <= 512 && n <= 8192);
}

// Environment overrides for experiments: WOQ_GEMM_KERNEL=exact|skinny, WOQ_GEMM_SPLITS=<n>
inline GemmPlan plan_gemm(int m, int n, int k, int bits)
{
    GemmPlan pl;
    char const* e = std::getenv("WOQ_GEMM_KERNEL");
    pl.skinny = e ? !std::strcmp(e, "skinny") : prefer_skinny(m, n);
    if (pl.skinny)
        pl.rt = (m <= 32 && bits == 4) ? 2 : 4; // 32- or 64-row tiles
    else
        pl.rt = m <= 64 ? 4 : (m <= 128 ? 8 : 16);
    int const tile_rows = pl.rt * 16;
    int const tk = tile_k_of_bits(bits);
    int const k_tiles = (k + tk - 1) / tk;
    long const tiles = (long) ((m + tile_rows - 1) / tile_rows) * ((n + 255) / 256);
    pl.k_splits = 1;
    if (tiles < 160 && k_tiles >= 8)
    {
        long splits = 320 / tiles;
        if (splits > k_tiles / 4)
            splits = k_tiles / 4;
        if (splits > 1)
            pl.k_splits = (int) splits;
    }
    if (char const* f = std::getenv("WOQ_GEMM_SPLITS"))
    {
        int const v = std::atoi(f);
        if (v >= 1 && v <= k_tiles)
            pl.k_splits = v;
    }
    pl.ws_bytes = pl.k_splits > 1 ? (size_t) m * (size_t) n * 4 : 0;
    return pl;
}

// W4A8 runs on one kernel (exact dequantize to e4m3, 64/128/256-row tiles, optional split-K)
inline GemmPlan plan_gemm_w4a8(int m, int n, int k)
{
    GemmPlan pl;
    pl.skinny = false;
    pl.rt = m <= 64 ? 4 : (m <= 128 ? 8 : 16);
    int const k_tiles = (k + 127) / 128;
    long const tiles = (long) ((m + pl.rt * 16 - 1) / (pl.rt * 16)) * ((n + 255) / 256);
    pl.k_splits = 1;
    if (tiles < 160 && k_tiles >= 8)
    {
        long splits = 320 / tiles;
        if (splits > k_tiles / 4)
            splits = k_tiles / 4;
        if (splits > 1)
            pl.k_splits = (int) splits;
    }
    if (char const* f = std::getenv("WOQ_GEMM_SPLITS"))
    {
        int const v = std::atoi(f);
        if (v >= 1 && v <= k_tiles)
            pl.k_splits = v;
    }
    pl.ws_bytes = pl.k_splits > 1 ? (size_t) m * (size_t) n * 4 : 0;
    return pl;
}

// largest M the streaming kernel is instantiated for
constexpr int kStreamMaxM = 128;

} // namespace woq
