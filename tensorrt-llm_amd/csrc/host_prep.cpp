// Host-side weight preparation of libwoq: int4 pack/unpack, the per-column symmetric quantizer,
// the gfx950 tile layout (and its inverse), and a decoder for weights that were laid out by the
// reference's preprocess_weights_for_mixed_gemm.
//
// Reference behaviour reproduced (not its code): cpp/tensorrt_llm/thop/weightOnlyQuantOp.cpp:284-353
// (pack/unpack), cpp/tensorrt_llm/kernels/cutlass_kernels/cutlass_preprocessors.cpp:652-762
// (quantizer) and :163-615 (the layout that woq_import_reference_weights inverts).
//
// The gfx950 tile layout
// ----------------------
// The logical weight is W[K, N] (K = input features).  It is cut into tiles of 16 columns by
// TILE_K rows (128 rows for int4, 64 for int8); a tile is exactly 1 KiB and tiles are stored
// [n_tile][k_tile], so a wavefront that walks K for one 16-column strip reads contiguous memory.
// Inside a tile, byte offset lane*16 belongs to lane = kg*16 + c of a 64-wide wavefront, where
// c is the column inside the tile and kg = 0..3.  The lane's 16 bytes are the B operands of the
// 16x16x32 MFMA for slabs j = 0..TILE_K/32-1: slab j, element e (0..7) is row
//     k = k_tile*TILE_K + j*32 + kg*8 + e.
// One global_load_dwordx4 per lane therefore yields, with no cross-lane traffic, everything
// that lane feeds to the matrix core for 128 (64) rows of K.  Values are stored biased
// (q + 8 / q + 128).  For int4, dword j holds element e at nibble position (e even ? e/2 :
// 4 + e/2), so that ((w >> 4*i) & 0x000F000F) isolates elements 2i (low half) and 2i+1 (high half)
// in the position of a packed pair of 16-bit floats.  For int8, element e of slab j is byte j*8 + e.
// K that is not a multiple of TILE_K is padded with q = 0.

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "woq_internal.h"

namespace woq
{

static thread_local char g_last_error[512] = "";

int fail(int code, char const* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

namespace
{

template <typename F>
void parallel_for(int64_t count, F&& body)
{
    unsigned hw = std::thread::hardware_concurrency();
    int64_t workers = std::max<int64_t>(1, std::min<int64_t>({(int64_t) (hw ? hw : 1), (int64_t) 16, count}));
    if (workers == 1)
    {
        for (int64_t i = 0; i < count; ++i)
            body(i);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (int64_t w = 0; w < workers; ++w)
        pool.emplace_back(
            [=, &body]()
            {
                for (int64_t i = w; i < count; i += workers)
                    body(i);
            });
    for (auto& t : pool)
        t.join();
}

// ---- 16-bit float conversions on the host (round to nearest even) --------------------------

float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t) (h & 0x8000) << 16;
    uint32_t exp = (h >> 10) & 0x1F;
    uint32_t man = h & 0x3FF;
    uint32_t bits;
    if (exp == 0)
    {
        if (man == 0)
            bits = sign;
        else
        {
            int shift = 0;
            while (!(man & 0x400))
            {
                man <<= 1;
                ++shift;
            }
            man &= 0x3FF;
            bits = sign | ((uint32_t) (127 - 15 - shift + 1) << 23) | (man << 13);
        }
    }
    else if (exp == 31)
        bits = sign | 0x7F800000u | (man << 13);
    else
        bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

uint16_t float_to_half(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000;
    uint32_t absx = x & 0x7FFFFFFF;
    if (absx > 0x7F800000)
        return (uint16_t) (sign | 0x7E00);
    if (absx >= 0x47800000) // >= 65536 -> inf (65520 and above round to inf, handled below too)
        return (uint16_t) (sign | 0x7C00);
    if (absx < 0x33000000) // < 2^-25 -> 0
        return (uint16_t) sign;
    int exp = (int) (absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFF) | 0x800000;
    int shift;
    uint32_t base;
    if (exp < -14)
    {
        shift = 13 + (-14 - exp);
        base = 0;
    }
    else
    {
        shift = 13;
        base = (uint32_t) (exp + 15) << 10;
        man &= 0x7FFFFF;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t half_ulp = 1u << (shift - 1);
    if (rem > half_ulp || (rem == half_ulp && (q & 1)))
        ++q;
    return (uint16_t) (sign | (base + q)); // a mantissa carry correctly bumps the exponent
}

float bf16_to_float(uint16_t b)
{
    uint32_t bits = (uint32_t) b << 16;
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

uint16_t float_to_bf16(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFF) > 0x7F800000)
        return (uint16_t) ((x >> 16) | 0x40);
    x += 0x7FFF + ((x >> 16) & 1);
    return (uint16_t) (x >> 16);
}

float load_as_float(void const* p, int64_t i, int dtype)
{
    switch (dtype)
    {
    case WOQ_FP32: return static_cast<float const*>(p)[i];
    case WOQ_FP16: return half_to_float(static_cast<uint16_t const*>(p)[i]);
    default: return bf16_to_float(static_cast<uint16_t const*>(p)[i]);
    }
}

void store_from_float(void* p, int64_t i, int dtype, float v)
{
    switch (dtype)
    {
    case WOQ_FP32: static_cast<float*>(p)[i] = v; break;
    case WOQ_FP16: static_cast<uint16_t*>(p)[i] = float_to_half(v); break;
    default: static_cast<uint16_t*>(p)[i] = float_to_bf16(v); break;
    }
}

// signed element (k, n) of a row-major matrix with `bits`-wide elements packed along n
inline int read_signed(uint8_t const* src, int64_t k, int64_t n, int64_t N, int bits)
{
    if (bits == 8)
        return (int8_t) src[k * N + n];
    uint8_t byte = src[(k * N + n) >> 1];
    int u = (n & 1) ? (byte >> 4) : (byte & 0xF);
    return u >= 8 ? u - 16 : u;
}

inline void write_signed(uint8_t* dst, int64_t k, int64_t n, int64_t N, int bits, int v)
{
    if (bits == 8)
    {
        dst[k * N + n] = (uint8_t) (int8_t) v;
        return;
    }
    uint8_t& byte = dst[(k * N + n) >> 1];
    if (n & 1)
        byte = (uint8_t) ((byte & 0x0F) | ((v & 0xF) << 4));
    else
        byte = (uint8_t) ((byte & 0xF0) | (v & 0xF));
}

inline int nibble_slot(int e)
{
    return (e & 1) ? 4 + (e >> 1) : (e >> 1);
}

int check_prep_shape(int64_t experts, int64_t k, int64_t n, int quant_type)
{
    if (quant_type != WOQ_W8_A16 && quant_type != WOQ_W4_A16 && quant_type != WOQ_W4_AFP8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_type %d", quant_type);
    if (experts < 1 || k < 1 || n < 1)
        return fail(WOQ_ERR_BAD_SHAPE, "experts, k and n must be positive (got %lld, %lld, %lld)", (long long) experts,
            (long long) k, (long long) n);
    if (n % kTileN)
        return fail(WOQ_ERR_BAD_SHAPE, "n must be a multiple of %d (got %lld)", kTileN, (long long) n);
    if (k % 32)
        return fail(WOQ_ERR_BAD_SHAPE, "k must be a multiple of 32 (got %lld)", (long long) k);
    return WOQ_OK;
}

constexpr int kPermW8[16] = {0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15};
constexpr int kPermW4[32] = {0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27, 4, 5, 12, 13, 20, 21, 28, 29, 6,
    7, 14, 15, 22, 23, 30, 31};
constexpr int kPermW4A8[32] = {0, 1, 2, 3, 16, 17, 18, 19, 4, 5, 6, 7, 20, 21, 22, 23, 8, 9, 10, 11, 24, 25, 26, 27,
    12, 13, 14, 15, 28, 29, 30, 31};

} // namespace
} // namespace woq

using namespace woq;

namespace
{
struct LaunchNote
{
    char const* fmt = nullptr;
    int v[6] = {};
};
thread_local LaunchNote g_launch_note;
thread_local char g_launch_text[160] = "";
} // namespace

void woq::note_launch(char const* fmt, int a, int b, int c, int d, int e, int f)
{
    g_launch_note = LaunchNote{fmt, {a, b, c, d, e, f}};
}

extern "C" const char* woq_last_launch(void)
{
    LaunchNote const& n = g_launch_note;
    g_launch_text[0] = 0;
    if (n.fmt)
    {
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Wformat-nonliteral"
        std::snprintf(g_launch_text, sizeof g_launch_text, n.fmt, n.v[0], n.v[1], n.v[2], n.v[3], n.v[4], n.v[5]);
#pragma GCC diagnostic pop
    }
    return g_launch_text;
}

extern "C" const char* woq_last_error(void)
{
    return g_last_error;
}

extern "C" int woq_abi_version(void)
{
    return WOQ_ABI_VERSION;
}

extern "C" int woq_layout_version(void)
{
    return WOQ_LAYOUT_VERSION;
}

extern "C" int woq_pack_int4(void* packed, const void* unpacked_int8, size_t n_unpacked)
{
    if (!packed || !unpacked_int8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_pack_int4: null pointer");
    if (n_unpacked == 0)
        return fail(WOQ_ERR_BAD_SHAPE, "weight should not be empty tensor");
    if (n_unpacked % 2)
        return fail(WOQ_ERR_BAD_SHAPE, "woq_pack_int4: element count must be even (got %zu)", n_unpacked);
    auto const* in = static_cast<int8_t const*>(unpacked_int8);
    auto* out = static_cast<uint8_t*>(packed);
    for (size_t i = 0; i < n_unpacked / 2; ++i)
    {
        int lo = in[2 * i], hi = in[2 * i + 1];
        if (lo < -8 || lo > 7 || hi < -8 || hi > 7)
            return fail(WOQ_ERR_VALUE, "Value in unpacked tensor not in int4 range");
        out[i] = (uint8_t) ((lo & 0xF) | ((hi & 0xF) << 4));
    }
    return WOQ_OK;
}

extern "C" int woq_unpack_int4(void* unpacked_int8, const void* packed, size_t n_packed)
{
    if (!packed || !unpacked_int8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_unpack_int4: null pointer");
    if (n_packed == 0)
        return fail(WOQ_ERR_BAD_SHAPE, "weight should not be empty tensor");
    auto const* in = static_cast<uint8_t const*>(packed);
    auto* out = static_cast<int8_t*>(unpacked_int8);
    for (size_t i = 0; i < n_packed; ++i)
    {
        out[2 * i] = (int8_t) ((int8_t) (in[i] << 4) >> 4);
        out[2 * i + 1] = (int8_t) ((int8_t) in[i] >> 4);
    }
    return WOQ_OK;
}

extern "C" size_t woq_preprocessed_bytes(int64_t k, int64_t n, int32_t quant_type)
{
    int bits = bits_of(quant_type);
    int64_t tk = tile_k_of_bits(bits);
    int64_t kp = (k + tk - 1) / tk * tk;
    return (size_t) (kp * n * bits / 8);
}

extern "C" int woq_preprocess_weights(
    void* dst, const void* src, int64_t experts, int64_t k, int64_t n, int32_t quant_type)
{
    if (!dst || !src)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_preprocess_weights: null pointer");
    if (int rc = check_prep_shape(experts, k, n, quant_type))
        return rc;
    int const bits = bits_of(quant_type);
    int const tk = tile_k_of_bits(bits);
    int const slabs = tk / 32;
    int64_t const k_tiles = (k + tk - 1) / tk;
    int64_t const n_tiles = n / kTileN;
    size_t const src_bytes = (size_t) (k * n * bits / 8);
    size_t const dst_bytes = woq_preprocessed_bytes(k, n, quant_type);
    int const bias = 1 << (bits - 1);

    for (int64_t ex = 0; ex < experts; ++ex)
    {
        auto const* s = static_cast<uint8_t const*>(src) + ex * src_bytes;
        auto* d = static_cast<uint8_t*>(dst) + ex * dst_bytes;
        parallel_for(k_tiles,
            [&](int64_t kt)
            {
                for (int64_t nt = 0; nt < n_tiles; ++nt)
                {
                    uint8_t* tile = d + (nt * k_tiles + kt) * 1024;
                    for (int kg = 0; kg < 4; ++kg)
                        for (int c = 0; c < kTileN; ++c)
                        {
                            uint8_t* lane = tile + (kg * 16 + c) * 16;
                            int64_t const col = nt * kTileN + c;
                            for (int j = 0; j < slabs; ++j)
                            {
                                int64_t const k0 = kt * tk + j * 32 + kg * 8;
                                if (bits == 4)
                                {
                                    uint32_t word = 0;
                                    for (int e = 0; e < 8; ++e)
                                    {
                                        int v = (k0 + e < k) ? read_signed(s, k0 + e, col, n, 4) : 0;
                                        word |= (uint32_t) (v + bias) << (4 * nibble_slot(e));
                                    }
                                    std::memcpy(lane + j * 4, &word, 4);
                                }
                                else
                                {
                                    for (int e = 0; e < 8; ++e)
                                    {
                                        int v = (k0 + e < k) ? read_signed(s, k0 + e, col, n, 8) : 0;
                                        lane[j * 8 + e] = (uint8_t) (v + bias);
                                    }
                                }
                            }
                        }
                }
            });
    }
    return WOQ_OK;
}

extern "C" int woq_unpreprocess_weights(
    void* dst_row_major, const void* src, int64_t experts, int64_t k, int64_t n, int32_t quant_type)
{
    if (!dst_row_major || !src)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_unpreprocess_weights: null pointer");
    if (int rc = check_prep_shape(experts, k, n, quant_type))
        return rc;
    int const bits = bits_of(quant_type);
    int const tk = tile_k_of_bits(bits);
    int const slabs = tk / 32;
    int64_t const k_tiles = (k + tk - 1) / tk;
    int64_t const n_tiles = n / kTileN;
    size_t const row_bytes = (size_t) (k * n * bits / 8);
    size_t const prep_bytes = woq_preprocessed_bytes(k, n, quant_type);
    int const bias = 1 << (bits - 1);

    for (int64_t ex = 0; ex < experts; ++ex)
    {
        auto const* s = static_cast<uint8_t const*>(src) + ex * prep_bytes;
        auto* d = static_cast<uint8_t*>(dst_row_major) + ex * row_bytes;
        // threads own disjoint k-tiles, hence disjoint rows of the output
        parallel_for(k_tiles,
            [&](int64_t kt)
            {
                for (int64_t nt = 0; nt < n_tiles; ++nt)
                {
                    uint8_t const* tile = s + (nt * k_tiles + kt) * 1024;
                    for (int kg = 0; kg < 4; ++kg)
                        for (int c = 0; c < kTileN; ++c)
                        {
                            uint8_t const* lane = tile + (kg * 16 + c) * 16;
                            int64_t const col = nt * kTileN + c;
                            for (int j = 0; j < slabs; ++j)
                            {
                                int64_t const k0 = kt * tk + j * 32 + kg * 8;
                                uint32_t word = 0;
                                if (bits == 4)
                                    std::memcpy(&word, lane + j * 4, 4);
                                for (int e = 0; e < 8 && k0 + e < k; ++e)
                                {
                                    int u = bits == 4 ? (int) ((word >> (4 * nibble_slot(e))) & 0xF)
                                                      : (int) lane[j * 8 + e];
                                    write_signed(d, k0 + e, col, n, bits, u - bias);
                                }
                            }
                        }
                }
            });
    }
    return WOQ_OK;
}

extern "C" int woq_import_reference_weights(void* dst_row_major, const void* src_reference_layout, int64_t experts,
    int64_t k, int64_t n, int32_t quant_type, int32_t arch)
{
    if (!dst_row_major || !src_reference_layout)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_import_reference_weights: null pointer");
    if (quant_type != WOQ_W8_A16 && quant_type != WOQ_W4_A16 && quant_type != WOQ_W4_AFP8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_type %d", quant_type);
    if (arch < 75)
        return fail(WOQ_ERR_UNSUPPORTED, "reference layouts exist for SM >= 75 only (got %d)", arch);
    int const bits = bits_of(quant_type);
    int const per_word = 32 / bits;
    int const plen = quant_type == WOQ_W8_A16 ? 16 : 32;
    int const* perm = quant_type == WOQ_W8_A16 ? kPermW8 : (quant_type == WOQ_W4_A16 ? kPermW4 : kPermW4A8);
    int64_t const tile_k = quant_type == WOQ_W4_AFP8 ? 128 : 64;
    int64_t const interleave = (128 * 8 / bits) / tile_k;
    bool const interleaved = !(arch >= 90 && arch < 100);
    if (experts < 1 || k % plen || n % 8 || (k * bits / 8) % 32 || (n * bits / 8) % 32 || (interleaved && k % tile_k)
        || (interleaved && n % interleave))
        return fail(WOQ_ERR_BAD_SHAPE, "shape [%lld, %lld] is not one the reference preprocess accepts", (long long) k,
            (long long) n);
    int inv_perm[32];
    for (int i = 0; i < plen; ++i)
        inv_perm[perm[i]] = i;
    int const bias = 1 << (bits - 1);
    size_t const mat_bytes = (size_t) (k * n * bits / 8);
    for (int64_t ex = 0; ex < experts; ++ex)
    {
        auto const* s = static_cast<uint8_t const*>(src_reference_layout) + ex * mat_bytes;
        auto* d = static_cast<uint8_t*>(dst_row_major) + ex * mat_bytes;
        // int4 rows are written by nibble: two neighbouring columns share a byte, so parallelise over rows
        parallel_for(k,
            [&](int64_t row)
            {
                int64_t const prow = row - row % plen + inv_perm[row % plen];
                for (int64_t col = 0; col < n; ++col)
                {
                    int64_t flat = interleaved ? (col / interleave) * (interleave * k)
                            + (prow / tile_k) * (interleave * tile_k) + (col % interleave) * tile_k + prow % tile_k
                                               : col * k + prow;
                    int64_t const word = flat / per_word;
                    int const within = (int) (flat % per_word);
                    int const slot = (within & 1) ? per_word / 2 + within / 2 : within / 2;
                    int64_t const phys = word * per_word + slot;
                    int u = bits == 8 ? (int) s[phys] : (int) ((s[phys >> 1] >> ((phys & 1) * 4)) & 0xF);
                    write_signed(d, row, col, n, bits, u - bias);
                }
            });
    }
    return WOQ_OK;
}

extern "C" int woq_reference_layout_step(void* dst, const void* src, int64_t experts, int64_t k, int64_t n,
    int32_t quant_type, int32_t step)
{
    if (!dst || !src)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "woq_reference_layout_step: null pointer");
    if (quant_type != WOQ_W8_A16 && quant_type != WOQ_W4_A16 && quant_type != WOQ_W4_AFP8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_type %d", quant_type);
    int const bits = bits_of(quant_type);
    if (experts < 1 || k < 1 || n < 1 || (k * n * bits) % 32)
        return fail(WOQ_ERR_BAD_SHAPE, "shape [%lld, %lld] does not fill whole 32-bit words", (long long) k, (long long) n);
    size_t const mat_bytes = (size_t) (k * n * bits / 8);
    auto const* s8 = static_cast<uint8_t const*>(src);
    auto* d8 = static_cast<uint8_t*>(dst);
    if (step == WOQ_REF_STEP_PERMUTE_ROWS)
    {
        // rows move inside blocks of 16 (int8) / 32 (int4) rows: written row i of a block is read row perm[i]
        int const plen = quant_type == WOQ_W8_A16 ? 16 : 32;
        int const* perm = quant_type == WOQ_W8_A16 ? kPermW8 : (quant_type == WOQ_W4_A16 ? kPermW4 : kPermW4A8);
        if (k % plen)
            return fail(WOQ_ERR_BAD_SHAPE,
                "Invalid shape for quantized tensor. Number of rows of quantized matrix must be a multiple of %d", plen);
        if (n % 8)
            return fail(WOQ_ERR_BAD_SHAPE,
                "Invalid shape for quantized tensor. On turing/Ampere, the number of cols must be a multiple of 8.");
        size_t const row_bytes = (size_t) (n * bits / 8);
        for (int64_t ex = 0; ex < experts; ++ex)
            parallel_for(k,
                [&](int64_t row)
                {
                    int64_t const from = row - row % plen + perm[row % plen];
                    std::memcpy(d8 + ex * mat_bytes + row * row_bytes, s8 + ex * mat_bytes + from * row_bytes, row_bytes);
                });
        return WOQ_OK;
    }
    if (step == WOQ_REF_STEP_SUBBYTE_TRANSPOSE)
    {
        // [k][n] -> [n][k] element by element (two int4 elements share a byte on both sides)
        if ((n * bits) % 8 || (k * bits) % 8)
            return fail(WOQ_ERR_BAD_SHAPE, "rows and columns must fill whole bytes");
        for (int64_t ex = 0; ex < experts; ++ex)
        {
            std::memset(d8 + ex * mat_bytes, 0, mat_bytes);
            // output rows (= input columns) are disjoint between threads
            parallel_for(n,
                [&](int64_t col)
                {
                    for (int64_t row = 0; row < k; ++row)
                        write_signed(d8 + ex * mat_bytes, col, row, k, bits,
                            read_signed(s8 + ex * mat_bytes, row, col, n, bits));
                });
        }
        return WOQ_OK;
    }
    if (step == WOQ_REF_STEP_ADD_BIAS_AND_INTERLEAVE)
    {
        // every element becomes unsigned (+128 / +8); inside each 32-bit word the elements are then
        // reordered: int8 [0, 2, 1, 3], int4 [0, 2, 4, 6, 1, 3, 5, 7] (written position <- element)
        int const per_word = 32 / bits;
        int const bias = 1 << (bits - 1);
        size_t const words = (size_t) experts * mat_bytes / 4;
        parallel_for((int64_t) words,
            [&](int64_t w)
            {
                uint8_t const* in = s8 + w * 4;
                uint32_t out = 0;
                for (int pos = 0; pos < per_word; ++pos)
                {
                    int const elt = pos < per_word / 2 ? 2 * pos : 2 * (pos - per_word / 2) + 1;
                    int const nib = (in[elt >> 1] >> ((elt & 1) * 4)) & 0xF;
                    int const v = bits == 8 ? (int) (int8_t) in[elt] : (nib >= 8 ? nib - 16 : nib);
                    out |= (uint32_t) ((v + bias) & ((1 << bits) - 1)) << (pos * bits);
                }
                std::memcpy(d8 + w * 4, &out, 4);
            });
        return WOQ_OK;
    }
    return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown step %d", step);
}

extern "C" int woq_symmetric_quantize(void* processed, void* unprocessed, void* scales, const void* weight,
    int64_t experts, int64_t k, int64_t n, int32_t quant_type, int32_t weight_dtype, int32_t scale_dtype)
{
    if (!scales)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "Scale output pointer is NULL");
    if (!weight)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "Input weight pointer is NULL");
    if (!processed && !unprocessed)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "Processed quantized tensor is NULL");
    if (quant_type != WOQ_W8_A16 && quant_type != WOQ_W4_A16 && quant_type != WOQ_W4_AFP8)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "unknown quant_type %d", quant_type);
    for (int dt : {weight_dtype, scale_dtype})
        if (dt != WOQ_FP32 && dt != WOQ_FP16 && dt != WOQ_BF16)
            return fail(WOQ_ERR_INVALID_ARGUMENT, "weight/scale dtype must be fp32, fp16 or bf16");
    if (experts < 1 || k < 1 || n < 1 || n % 2)
        return fail(WOQ_ERR_BAD_SHAPE, "bad shape [%lld, %lld, %lld]", (long long) experts, (long long) k,
            (long long) n);
    if (processed)
        if (int rc = check_prep_shape(experts, k, n, quant_type))
            return rc;

    int const bits = bits_of(quant_type);
    float const range = 1.f / (float) (1 << (bits - 1));
    float const lo = -(float) (1 << (bits - 1)), hi = (float) ((1 << (bits - 1)) - 1);
    size_t const q_bytes = (size_t) (k * n * bits / 8);
    std::vector<uint8_t> local;
    uint8_t* q_all = static_cast<uint8_t*>(unprocessed);
    if (!q_all)
    {
        local.resize(q_bytes * experts);
        q_all = local.data();
    }
    for (int64_t ex = 0; ex < experts; ++ex)
    {
        int64_t const w_off = ex * k * n;
        std::vector<float> col_scale(n, 0.f);
        // column maxima: threads own disjoint column ranges
        int64_t const chunks = std::min<int64_t>(n, 64);
        parallel_for(chunks,
            [&](int64_t ch)
            {
                int64_t c0 = ch * n / chunks, c1 = (ch + 1) * n / chunks;
                for (int64_t r = 0; r < k; ++r)
                    for (int64_t c = c0; c < c1; ++c)
                        col_scale[c] = std::max(col_scale[c], std::fabs(load_as_float(weight, w_off + r * n + c, weight_dtype)));
            });
        for (int64_t c = 0; c < n; ++c)
        {
            col_scale[c] *= range;
            store_from_float(scales, ex * n + c, scale_dtype, col_scale[c]);
        }
        uint8_t* q = q_all + ex * q_bytes;
        parallel_for(k,
            [&](int64_t r)
            {
                for (int64_t c = 0; c < n; ++c)
                {
                    float const s = col_scale[c];
                    float v = s != 0.f ? std::round(load_as_float(weight, w_off + r * n + c, weight_dtype) / s) : 0.f;
                    v = std::max(lo, std::min(hi, v));
                    write_signed(q, r, c, n, bits, (int) v);
                }
            });
    }
    if (processed)
        return woq_preprocess_weights(processed, q_all, experts, k, n, quant_type);
    return WOQ_OK;
}
