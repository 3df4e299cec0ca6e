// Internal declarations shared by the host code and the kernel launchers of libwoq.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <cstdio>

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

// largest M the streaming kernel is instantiated for
constexpr int kStreamMaxM = 128;

} // namespace woq
