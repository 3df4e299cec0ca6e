/* CPU oracle, loop form.  TEST INFRASTRUCTURE ONLY: nothing in the product links or loads this.
 *
 * A plain-C restatement of the reference's host-side weight preparation, written as the
 * element-by-element loops the reference describes (the numpy oracle states the same steps as
 * whole-array index maps; the two are compared position by position in the tests):
 *
 *   oracle_pack_int4 / oracle_unpack_int4 ... cpp/tensorrt_llm/thop/weightOnlyQuantOp.cpp:284-353
 *   oracle_permute_rows ..................... cpp/tensorrt_llm/kernels/cutlass_kernels/cutlass_preprocessors.cpp:163-244
 *   oracle_subbyte_transpose ................ cutlass_preprocessors.cpp:250-410
 *   oracle_interleave_columns ............... cutlass_preprocessors.cpp:512-562
 *   oracle_bias_interleave .................. cutlass_preprocessors.cpp:412-510
 *   oracle_ref_preprocess ................... cutlass_preprocessors.cpp:564-615
 *   oracle_symmetric_quantize ............... cutlass_preprocessors.cpp:652-762
 *   oracle_dequant_matmul_f32 ............... tensorrt_llm/quantization/functional.py:269-290 (the
 *                                             dequantize-then-matmul fallback), float32 throughout
 *
 * quant_type: 0 = W8_A16, 1 = W4_A16, 2 = W4_AFP8 (cutlass_preprocessors.h:32-37).
 * All matrices are single (no expert dimension); callers loop over experts.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int bits_of(int quant_type) { return quant_type == 0 ? 8 : 4; }

/* nibble / byte accessors on a packed buffer of `bits`-wide elements, low nibble first */
static unsigned get_elt(const uint8_t* buf, size_t idx, int bits)
{
    if (bits == 8) return buf[idx];
    return (buf[idx >> 1] >> ((idx & 1) * 4)) & 0xF;
}

static void set_elt(uint8_t* buf, size_t idx, int bits, unsigned v)
{
    if (bits == 8) { buf[idx] = (uint8_t) v; return; }
    unsigned shift = (unsigned) (idx & 1) * 4;
    buf[idx >> 1] = (uint8_t) ((buf[idx >> 1] & ~(0xF << shift)) | ((v & 0xF) << shift));
}

int oracle_pack_int4(uint8_t* packed, const int8_t* unpacked, size_t n_unpacked)
{
    for (size_t i = 0; i < n_unpacked / 2; ++i)
    {
        int a = unpacked[2 * i], b = unpacked[2 * i + 1];
        if (a < -8 || a > 7 || b < -8 || b > 7) return -1;
        packed[i] = (uint8_t) ((a & 0xF) | ((b & 0xF) << 4));
    }
    return 0;
}

void oracle_unpack_int4(int8_t* unpacked, const uint8_t* packed, size_t n_packed)
{
    for (size_t i = 0; i < n_packed; ++i)
    {
        int lo = packed[i] & 0xF, hi = packed[i] >> 4;
        unpacked[2 * i] = (int8_t) (lo >= 8 ? lo - 16 : lo);
        unpacked[2 * i + 1] = (int8_t) (hi >= 8 ? hi - 16 : hi);
    }
}

static const int PERM_W8[16] = {0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15};
static const int PERM_W4[32] = {0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27, 4, 5, 12, 13, 20, 21, 28, 29,
    6, 7, 14, 15, 22, 23, 30, 31};
static const int PERM_W4A8[32] = {0, 1, 2, 3, 16, 17, 18, 19, 4, 5, 6, 7, 20, 21, 22, 23, 8, 9, 10, 11, 24, 25, 26, 27,
    12, 13, 14, 15, 28, 29, 30, 31};

/* row r of every block of P rows is taken from row perm[r] of that block; whole rows move */
int oracle_permute_rows(uint8_t* dst, const uint8_t* src, size_t rows, size_t cols, int quant_type)
{
    int bits = bits_of(quant_type);
    int P = quant_type == 0 ? 16 : 32;
    const int* perm = quant_type == 0 ? PERM_W8 : (quant_type == 1 ? PERM_W4 : PERM_W4A8);
    if (rows % (size_t) P || cols % 8) return -1;
    size_t row_bytes = cols * (size_t) bits / 8;
    for (size_t r = 0; r < rows; ++r)
    {
        size_t from = r - r % P + (size_t) perm[r % P];
        memcpy(dst + r * row_bytes, src + from * row_bytes, row_bytes);
    }
    return 0;
}

/* [rows][cols] -> [cols][rows] at element granularity */
int oracle_subbyte_transpose(uint8_t* dst, const uint8_t* src, size_t rows, size_t cols, int quant_type)
{
    int bits = bits_of(quant_type);
    if ((rows * (size_t) bits / 8) % 32 || (cols * (size_t) bits / 8) % 32) return -1;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c)
            set_elt(dst, c * rows + r, bits, get_elt(src, r * cols + c, bits));
    return 0;
}

/* column-major [cols][rows] -> groups of `interleave` columns whose `tile_k`-row tiles alternate */
int oracle_interleave_columns(uint8_t* dst, const uint8_t* src, size_t rows, size_t cols, int quant_type)
{
    int bits = bits_of(quant_type);
    size_t tile_k = quant_type == 2 ? 128 : 64;              /* 128*8 / bits(activation) */
    size_t interleave = (size_t) (128 * 8 / bits) / tile_k;  /* elements per 128-byte line / tile_k */
    if (rows % tile_k || cols % interleave) return -1;
    for (size_t c = 0; c < cols; ++c)
        for (size_t r = 0; r < rows; ++r)
        {
            size_t group = c / interleave, within = c % interleave;
            size_t out = group * interleave * rows + (r / tile_k) * interleave * tile_k + within * tile_k + r % tile_k;
            set_elt(dst, out, bits, get_elt(src, c * rows + r, bits));
        }
    return 0;
}

/* signed -> unsigned (+2^(bits-1)), then inside each 32-bit word the even-indexed elements go
 * to the low half and the odd-indexed ones to the high half */
int oracle_bias_interleave(uint8_t* buf, size_t num_elts, int quant_type)
{
    int bits = bits_of(quant_type);
    int per_word = 32 / bits;
    if (num_elts % (size_t) per_word) return -1;
    unsigned tmp[8];
    for (size_t base = 0; base < num_elts; base += (size_t) per_word)
    {
        for (int e = 0; e < per_word; ++e)
        {
            unsigned raw = get_elt(buf, base + (size_t) e, bits);
            int sv = bits == 8 ? (int) (int8_t) raw : (raw >= 8 ? (int) raw - 16 : (int) raw);
            tmp[e] = (unsigned) (sv + (1 << (bits - 1)));
        }
        for (int d = 0; d < per_word; ++d)
        {
            int from = d < per_word / 2 ? 2 * d : 2 * (d - per_word / 2) + 1;
            set_elt(buf, base + (size_t) d, bits, tmp[from]);
        }
    }
    return 0;
}

/* composition for one [rows][cols] matrix; arch 90 leaves out the column interleave */
int oracle_ref_preprocess(uint8_t* dst, const uint8_t* src, size_t rows, size_t cols, int quant_type, int arch)
{
    int bits = bits_of(quant_type);
    size_t nbytes = rows * cols * (size_t) bits / 8;
    uint8_t* a = (uint8_t*) malloc(nbytes);
    uint8_t* b = (uint8_t*) malloc(nbytes);
    if (!a || !b) { free(a); free(b); return -2; }
    int rc = oracle_permute_rows(a, src, rows, cols, quant_type);
    if (!rc) rc = oracle_subbyte_transpose(b, a, rows, cols, quant_type);
    if (!rc && arch != 90)
    {
        rc = oracle_interleave_columns(a, b, rows, cols, quant_type);
        uint8_t* t = a; a = b; b = t;
    }
    if (!rc) rc = oracle_bias_interleave(b, rows * cols, quant_type);
    if (!rc) memcpy(dst, b, nbytes);
    free(a);
    free(b);
    return rc;
}

/* per-column symmetric quantizer on float32 input [rows][cols]; q is UNPACKED int8;
 * `scales` receives the float32 scale (the caller rounds it to fp16/bf16 for storage) */
void oracle_symmetric_quantize(int8_t* q, float* scales, const float* w, size_t rows, size_t cols, int bits)
{
    float range = 1.0f / (float) (1 << (bits - 1));
    for (size_t c = 0; c < cols; ++c) scales[c] = 0.f;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c)
        {
            float a = fabsf(w[r * cols + c]);
            if (a > scales[c]) scales[c] = a;
        }
    for (size_t c = 0; c < cols; ++c) scales[c] *= range;
    float lo = -(float) (1 << (bits - 1)), hi = (float) ((1 << (bits - 1)) - 1);
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c)
        {
            float s = scales[c];
            float v = s != 0.f ? roundf(w[r * cols + c] / s) : 0.f; /* roundf: halves away from zero */
            if (v < lo) v = lo;
            if (v > hi) v = hi;
            q[r * cols + c] = (int8_t) v;
        }
}

/* out[m][n] = sum_k act[m][k] * (q[k][n] * scale[g][n] + zero[g][n]); group == 0: one scale per column */
void oracle_dequant_matmul_f32(float* out, const float* act, const int8_t* q, const float* scales, const float* zeros,
    size_t m, size_t n, size_t k, size_t group)
{
    float* wrow = (float*) malloc(n * sizeof(float));
    memset(out, 0, m * n * sizeof(float));
    for (size_t kk = 0; kk < k; ++kk)
    {
        size_t g = group ? kk / group : 0;
        for (size_t c = 0; c < n; ++c)
            wrow[c] = (float) q[kk * n + c] * scales[g * n + c] + (zeros ? zeros[g * n + c] : 0.f);
        for (size_t r = 0; r < m; ++r)
        {
            float a = act[r * k + kk];
            float* o = out + r * n;
            for (size_t c = 0; c < n; ++c) o[c] += a * wrow[c];
        }
    }
    free(wrow);
}
