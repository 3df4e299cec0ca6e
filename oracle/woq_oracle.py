"""CPU oracle for the weight-only quantized matmul path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product (the `tensorrt-llm_amd` package, `libwoq.so`) imports or calls this
file; only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` do,
and only as the checker.

It restates, in numpy, the algorithm of the reference's weight-only path.  Every function
cites the reference source it follows (paths relative to the reference checkout):

  pack/unpack int4 ............ cpp/tensorrt_llm/thop/weightOnlyQuantOp.cpp:284-353
  symmetric_quantize .......... cpp/tensorrt_llm/kernels/cutlass_kernels/cutlass_preprocessors.cpp:652-762
  reference weight layout ..... cutlass_preprocessors.cpp:163-244 (row permutation), :250-410 (sub-byte
                                transpose), :512-562 (column interleave), :412-510 (bias + register
                                interleave), :564-615 (composition)
  reference GEMV addressing ... cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/kernel.h:57-79,
                                details.h:100-125 (Mapper), converter.h:30-59 +
                                cutlass_extensions/.../interleaved_numeric_conversion.h (element order)
  dequantize .................. weightOnlyBatchedGemv/utility.h:122-163 (w = fma(cvt(q), scale, zero))
  pre-quant scale ............. cpp/tensorrt_llm/kernels/preQuantScaleKernel.cu:42-133
  matmul + epilogue ........... utility.h:217-269 (out = alpha * acc + bias); python fallback
                                tensorrt_llm/quantization/functional.py:223-234,269-290
  checkpoint-side folding ..... tensorrt_llm/quantization/functional.py:1010-1014 (zeros),
                                tensorrt_llm/models/modeling_utils.py:1661-1682 (W4A8 alpha)

Pinning status (what fixes each function besides its own formula):
  pack/unpack ............ brute force over all 256 byte values + inverse property.
  symmetric_quantize ..... explicit ties (half away from zero), /2^(bits-1) scale, zero-column guard.
  reference layout ....... three independently written pieces agree on every element position:
                           this file's array-op form, the loop-form C restatement in
                           oracle/ref_layout.c, and the emulation of the reference GEMV's thread
                           addressing (`ref_gemv_decode`) that must read back every (k, n).
                           The exact output BYTES of the reference's preprocess on a real SM are
                           stored nowhere in the reference tree: that byte-level parity is
                           "parity unpinned" beyond these source-derived cross checks.
  dequantize ............. exact integer recovery + one float formula; special cases (zero=0,
                           scale=1, identity activation recovers the weight).
  matmul ................. numpy float64 matmul of the dequantized weight (a library routine).
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------------------
# quantization types (cutlass_preprocessors.h:32-48)
# --------------------------------------------------------------------------------------
W8_A16 = "W8_A16"
W4_A16 = "W4_A16"
W4_AFP8 = "W4_AFP8"


def weight_bits(quant_type: str) -> int:
    return {W8_A16: 8, W4_A16: 4, W4_AFP8: 4}[quant_type]


# quant_algo bit flags of the groupwise plugin
# (plugins/weightOnlyGroupwiseQuantMatmulPlugin/weightOnlyGroupwiseQuantMatmulPlugin.cpp:29-37)
BIAS = 1
ZERO = 2
PRE_QUANT_SCALE = 4
FP8_ALPHA = 8
INT8_WEIGHT = 16

# --------------------------------------------------------------------------------------
# small-float helpers (values are carried as float32 arrays that are exactly representable
# in the narrow type; bit patterns are available through *_bits helpers)
# --------------------------------------------------------------------------------------


def f32_to_bf16_bits(x) -> np.ndarray:
    """float32 -> bfloat16 bit pattern, round to nearest even (NaN kept quiet)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    is_nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(is_nan, (u >> 16) | 0x40, rounded)
    return (rounded & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(x) -> np.ndarray:
    """Round float values to bfloat16 (through float32 first), return as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(x).astype(np.float32)))


def round_f16(x) -> np.ndarray:
    """Round to float16 with ONE rounding from the given precision, return as float32."""
    return np.asarray(x).astype(np.float16).astype(np.float32)


def round_e4m3(x) -> np.ndarray:
    """float -> OCP float8 e4m3fn value (returned as float32): round to nearest even,
    saturating to +-448 (the reference casts with `__nv_fp8_e4m3`, which is satfinite:
    preQuantScaleKernel.cu:42-90)."""
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    ax = np.abs(x)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
    e = np.clip(e, -6, 8)  # below 2^-6 the format is subnormal with quantum 2^-9
    quantum = np.exp2(e - 3)
    r = np.rint(ax / quantum) * quantum  # np.rint is half-to-even
    r = np.minimum(r, 448.0)
    out = np.where(np.isnan(x), np.nan, np.sign(x) * r)
    return out.astype(np.float32)


def e4m3_bits(x) -> np.ndarray:
    """Bit pattern (uint8) of values already representable in e4m3fn."""
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    ax = np.abs(x)
    out = np.zeros(x.shape, dtype=np.uint8)
    normal = ax >= 2.0 ** -6
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(normal, ax, 1.0)))
    mant = np.where(normal, ax / np.exp2(e) - 1.0, 0.0) * 8
    out = np.where(normal, ((e + 7).astype(np.int64) << 3) | np.rint(mant).astype(np.int64), 0).astype(np.uint8)
    sub = np.rint(ax / 2.0 ** -9).astype(np.int64)
    out = np.where(normal, out, sub.astype(np.uint8))
    out = np.where(np.isnan(x), 0x7F, out)
    return (out | sign).astype(np.uint8)


def round_to(x, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return round_bf16(x)
    if dtype == "fp16":
        return round_f16(x)
    if dtype == "fp8":
        return round_e4m3(x)
    if dtype == "fp32":
        return np.asarray(x).astype(np.float32)
    raise ValueError(dtype)


# --------------------------------------------------------------------------------------
# a2: pack / unpack (thop/weightOnlyQuantOp.cpp:284-353)
# --------------------------------------------------------------------------------------


def pack_int8_tensor_to_packed_int4(w: np.ndarray) -> np.ndarray:
    """[..., N] int8 in [-8, 7] -> [..., ceil(N/2)] int8; element 2j is the LOW nibble."""
    w = np.asarray(w)
    if w.dtype != np.int8:
        raise TypeError("Weight must be a int8 tensor")
    if w.size == 0:
        raise ValueError("weight should not be empty tensor")
    if (w < -8).any() or (w > 7).any():
        raise ValueError("Value in unpacked tensor not in int4 range")
    if w.shape[-1] % 2:
        w = np.concatenate([w, np.zeros(w.shape[:-1] + (1,), np.int8)], axis=-1)
    lo = w[..., 0::2].astype(np.uint8) & 0x0F
    hi = (w[..., 1::2].astype(np.uint8) & 0x0F) << 4
    return (lo | hi).astype(np.uint8).view(np.int8)


def unpack_int4_packed_tensor_to_int8(w: np.ndarray) -> np.ndarray:
    """[..., N/2] int8 -> [..., N] int8, sign-extending both nibbles."""
    w = np.asarray(w)
    if w.dtype != np.int8:
        raise TypeError("Weight must be a packed int8 tensor")
    if w.size == 0:
        raise ValueError("weight should not be empty tensor")
    u = w.view(np.uint8)
    lo = ((u & 0x0F).astype(np.int16) ^ 8) - 8
    hi = ((u >> 4).astype(np.int16) ^ 8) - 8
    out = np.empty(w.shape[:-1] + (w.shape[-1] * 2,), dtype=np.int8)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


# --------------------------------------------------------------------------------------
# a3: symmetric per-column quantizer (cutlass_preprocessors.cpp:652-762)
# --------------------------------------------------------------------------------------


def _round_half_away(x: np.ndarray) -> np.ndarray:
    """C `round()`: halfway cases away from zero (cutlass_preprocessors.cpp:718,735)."""
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def symmetric_quantize(w: np.ndarray, bits: int, scale_dtype: str = "fp16"):
    """w: [K, N] or [E, K, N] float (already transposed to in x out).
    Returns (q_signed int8 [.., K, N] UNPACKED, scales float32 [.., N] rounded to scale_dtype).

    scale_n = max_k |w[k, n]| * 2^-(bits-1) in float32 (so /128 or /8), stored in scale_dtype;
    the division uses the float32 (unrounded) scale; q = clamp(round_half_away(w / scale));
    a zero column quantizes to 0."""
    w = np.asarray(w, dtype=np.float32)
    if w.ndim not in (2, 3):
        raise ValueError("Shape must be 2-D or 3-D")
    amax = np.abs(w).max(axis=-2)
    col_scale = (amax * np.float32(1.0 / (1 << (bits - 1)))).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        scaled = (w / col_scale[..., None, :]).astype(np.float32)
    scaled = np.where(col_scale[..., None, :] != 0, _round_half_away(scaled), 0.0)
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    q = np.clip(scaled, lo, hi).astype(np.int8)
    return q, round_to(col_scale, scale_dtype)


# --------------------------------------------------------------------------------------
# a4-a8: the REFERENCE's preprocessed layout, array-op form
# --------------------------------------------------------------------------------------

_PERM = {
    # cutlass_preprocessors.cpp:163-184
    W8_A16: [0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15],
    W4_A16: [0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27,
             4, 5, 12, 13, 20, 21, 28, 29, 6, 7, 14, 15, 22, 23, 30, 31],
    W4_AFP8: [0, 1, 2, 3, 16, 17, 18, 19, 4, 5, 6, 7, 20, 21, 22, 23,
              8, 9, 10, 11, 24, 25, 26, 27, 12, 13, 14, 15, 28, 29, 30, 31],
}


def ref_layout_constants(quant_type: str):
    """(ThreadblockK, ColumnsInterleaved) from
    cutlass_extensions/include/cutlass_extensions/gemm/kernel/mixed_gemm_B_layout.h:89-117:
    ThreadblockK = 128*8/bits(A); ColumnsInterleaved = (128*8/bits(B)) / ThreadblockK."""
    a_bits = 8 if quant_type == W4_AFP8 else 16
    tile_k = 128 * 8 // a_bits
    interleave = (128 * 8 // weight_bits(quant_type)) // tile_k
    return tile_k, interleave


# element held at physical position p of a 32-bit word after the register interleave
# (cutlass_preprocessors.cpp:436-439 for int8, :470-489 for int4)
_WORD_ORDER = {8: [0, 2, 1, 3], 4: [0, 2, 4, 6, 1, 3, 5, 7]}


def _pack_unsigned(flat_u: np.ndarray, bits: int) -> np.ndarray:
    if bits == 8:
        return flat_u.astype(np.uint8)
    return (flat_u[0::2].astype(np.uint8) | (flat_u[1::2].astype(np.uint8) << 4)).astype(np.uint8)


def _unpack_unsigned(raw: np.ndarray, bits: int) -> np.ndarray:
    raw = np.asarray(raw).view(np.uint8).reshape(-1)
    if bits == 8:
        return raw.astype(np.int32)
    out = np.empty(raw.size * 2, np.int32)
    out[0::2] = raw & 0x0F
    out[1::2] = raw >> 4
    return out


def ref_preprocess(q: np.ndarray, quant_type: str, arch: int = 80) -> np.ndarray:
    """preprocess_weights_for_mixed_gemm (cutlass_preprocessors.cpp:564-615) on ONE matrix.
    q: [K, N] signed integers (unpacked).  Returns uint8 bytes, K*N*bits/8 of them.
    arch 90 skips the column interleave (:607); every other supported arch uses all four steps."""
    bits = weight_bits(quant_type)
    q = np.asarray(q).astype(np.int32)
    K, N = q.shape
    perm = _PERM[quant_type]
    tile_k, interleave = ref_layout_constants(quant_type)
    if K % len(perm) or N % 8:
        raise ValueError("rows must be a multiple of %d and cols of 8" % len(perm))
    if (K * bits // 8) % 32 or (N * bits // 8) % 32:
        raise ValueError("Number of bytes for rows and cols must be a multiple of 32")
    # a4: rows permuted inside blocks of len(perm): out_row[i] = in_row[perm[i]]
    x = q.reshape(K // len(perm), len(perm), N)[:, perm, :].reshape(K, N)
    # a5: element-granular transpose -> [N][K], K contiguous
    x = np.ascontiguousarray(x.T)
    # a6: [N/I][K/T][I][T]
    if arch != 90:
        if K % tile_k:
            raise ValueError("rows must be a multiple of %d" % tile_k)
        x = x.reshape(N // interleave, interleave, K // tile_k, tile_k).transpose(0, 2, 1, 3)
    flat = np.ascontiguousarray(x).reshape(-1)
    # a7: bias to unsigned, then reorder inside every 32-bit word
    flat = flat + (1 << (bits - 1))
    epw = 32 // bits
    flat = flat.reshape(-1, epw)[:, _WORD_ORDER[bits]].reshape(-1)
    return _pack_unsigned(flat, bits)


def ref_layout_decode(raw: np.ndarray, K: int, N: int, quant_type: str, arch: int = 80) -> np.ndarray:
    """Inverse of `ref_preprocess` (array-op form): bytes -> [K, N] signed integers."""
    bits = weight_bits(quant_type)
    perm = _PERM[quant_type]
    tile_k, interleave = ref_layout_constants(quant_type)
    flat = _unpack_unsigned(raw, bits)
    epw = 32 // bits
    inv_word = np.argsort(_WORD_ORDER[bits])
    flat = flat.reshape(-1, epw)[:, inv_word].reshape(-1) - (1 << (bits - 1))
    if arch != 90:
        x = flat.reshape(N // interleave, K // tile_k, interleave, tile_k).transpose(0, 2, 1, 3).reshape(N, K)
    else:
        x = flat.reshape(N, K)
    x = x.T
    inv_perm = np.argsort(perm)
    x = x.reshape(K // len(perm), len(perm), N)[:, inv_perm, :].reshape(K, N)
    return np.ascontiguousarray(x).astype(np.int8)


def ref_gemv_decode(raw: np.ndarray, K: int, N: int, quant_type: str, cta_n: int = 4) -> np.ndarray:
    """Emulates how the reference's small-M kernel ADDRESSES preprocessed weights
    (weightOnlyBatchedGemv/kernel.h:57-79 for the offsets, details.h:100-125 for `Mapper`,
    the interleaved converter for the order inside a 32-bit word) and returns the [K, N]
    signed matrix those threads would multiply with.  Written from the kernel side, so it is
    independent of `ref_preprocess`; the two must invert each other."""
    bits = weight_bits(quant_type)
    tile = 128 if quant_type == W4_AFP8 else 64          # kernelLauncher.h:31-47 (KTile)
    interleave = 128 * 8 // (tile * bits)                # details.h:104
    step_k = 128 // bits                                 # details.h:102
    threads = 128
    cta_k = step_k * threads
    ga = tile // 32                                      # kElementGroupSizeA
    gw = interleave * ga                                 # kElementGroupSizeW
    go = 4 * ga                                          # kGroupOffsetA
    elems = _unpack_unsigned(raw, bits)
    epw = 32 // bits
    # converter: natural element j of a word sits at physical sub-position pos[j]
    pos = np.argsort(_WORD_ORDER[bits])
    interleaved_k = K * interleave
    out = np.full((K, N), 127, dtype=np.int32)
    seen = np.zeros((K, N), dtype=np.int32)
    if N % (cta_n * interleave):
        raise ValueError("launch failed")  # kernel.h:127-130
    for bn in range(N // (cta_n * interleave)):
        for tid in range(threads):
            real_n0 = bn * cta_n * interleave + (tid * step_k // tile) % interleave
            real_k0 = (tid * step_k // (interleave * tile)) * tile + (tid * step_k) % tile
            it = 0
            idx_k = tid * step_k
            while idx_k < interleaved_k:
                for i in range(cta_n):
                    n = real_n0 + i * interleave
                    base = (bn * cta_n + i) * interleaved_k + tid * step_k + it * cta_k
                    chunk = elems[base: base + step_k]
                    # converter output order
                    conv = chunk.reshape(-1, epw)[:, pos].reshape(-1) - (1 << (bits - 1))
                    for kk in range(step_k):
                        phys = kk % ga + (kk % go) // ga * gw + kk // go * ga
                        k = real_k0 + it * cta_k // interleave + kk
                        out[k, n] = conv[phys]
                        seen[k, n] += 1
                idx_k += cta_k
                it += 1
    if not (seen == 1).all():
        raise AssertionError("reference GEMV addressing did not visit every (k, n) exactly once")
    return out.astype(np.int8)


# --------------------------------------------------------------------------------------
# the gfx950 layout this build defines (independent numpy restatement, used to check the
# C++ preprocess in the product)
# --------------------------------------------------------------------------------------

GFX950_TILE_N = 16


def gfx950_tile_k(bits: int) -> int:
    return 128 if bits == 4 else 64


def gfx950_preprocessed_bytes(K: int, N: int, bits: int) -> int:
    tk = gfx950_tile_k(bits)
    return N * (-(-K // tk) * tk) * bits // 8


def gfx950_preprocess(q: np.ndarray, bits: int) -> np.ndarray:
    """[K, N] signed -> bytes in the gfx950 tile layout.

    A tile is 16 columns x tile_k rows (128 for int4, 64 for int8) = 1024 bytes, tiles ordered
    [n_tile][k_tile].  Inside a tile, lane = kg*16 + c (c = column in tile, kg = 0..3) owns 16
    consecutive bytes holding its MFMA B-operand slices: slab j (32 rows each) / element e (0..7)
    is row  k = k_tile*tile_k + j*32 + kg*8 + e.  Values are stored biased (q + 2^(bits-1)).
    int4: dword j of the lane, nibble position p holds e = [0,2,4,6,1,3,5,7][p].
    int8: byte j*8 + e.  K is zero-padded (q = 0) up to a multiple of tile_k."""
    q = np.asarray(q).astype(np.int32)
    K, N = q.shape
    if N % GFX950_TILE_N:
        raise ValueError("N must be a multiple of 16")
    tk = gfx950_tile_k(bits)
    Kp = -(-K // tk) * tk
    if Kp != K:
        q = np.concatenate([q, np.zeros((Kp - K, N), np.int32)], axis=0)
    u = q + (1 << (bits - 1))
    slabs = tk // 32
    x = u.reshape(Kp // tk, slabs, 4, 8, N // 16, 16)          # [kt, j, kg, e, nt, c]
    x = x.transpose(4, 0, 2, 5, 1, 3)                          # [nt, kt, kg, c, j, e]
    if bits == 4:
        x = x[..., _WORD_ORDER[4]]
    return _pack_unsigned(np.ascontiguousarray(x).reshape(-1), bits)


def gfx950_decode(raw: np.ndarray, K: int, N: int, bits: int) -> np.ndarray:
    tk = gfx950_tile_k(bits)
    Kp = -(-K // tk) * tk
    slabs = tk // 32
    flat = _unpack_unsigned(raw, bits)
    x = flat.reshape(N // 16, Kp // tk, 4, 16, slabs, 8)
    if bits == 4:
        x = x[..., np.argsort(_WORD_ORDER[4])]
    x = x.transpose(1, 4, 2, 5, 0, 3).reshape(Kp, N) - (1 << (bits - 1))
    return np.ascontiguousarray(x[:K]).astype(np.int8)


# --------------------------------------------------------------------------------------
# dequantize / pre-quant scale / matmul
# --------------------------------------------------------------------------------------


def expand_groups(t: np.ndarray, K: int, group_size: int) -> np.ndarray:
    """[K/g, N] (or [N] / [1, N] when group_size == 0: one scale per column) -> [K, N]."""
    t = np.asarray(t)
    if group_size == 0:
        return np.broadcast_to(t.reshape(1, -1), (K, t.size))
    return np.repeat(t, group_size, axis=0)[:K]


def dequantize(q, scales, zeros, group_size: int, dtype: str) -> np.ndarray:
    """w[k, n] = T(q[k, n] * scale[g(k), n] + zero[g(k), n]) with ONE defined rounding sequence
    (the reference computes `fma2(cvt(q), scale, zero)` in the activation type:
    weightOnlyBatchedGemv/utility.h:157-162; cvt(q) is exact):
      fp16: the exact value rounded once to fp16 (= a half-precision fused multiply-add);
      bf16: the exact value rounded to float32, then to bf16 (= a float32 fused multiply-add
            followed by a bf16 conversion; identical to a bf16 FMA whenever q*s+z fits float32
            exactly, i.e. whenever scale and zero are within 2^12 of each other);
      fp8 (W4A8): float32 FMA of q with the (fp16-valued) scale/zero, rounded once to e4m3fn
            (mma_tensorop_dequantizer.h + dq_mma_multistage_finegrained.h:595-609 round the
            dequantized weight to e4m3 before the MMA).
    Inputs are float32 arrays holding values representable in the scale type."""
    q = np.asarray(q).astype(np.float64)
    K = q.shape[0]
    s = expand_groups(scales, K, group_size).astype(np.float64)
    exact = q * s
    if zeros is not None:
        exact = exact + expand_groups(zeros, K, group_size).astype(np.float64)
    if dtype == "fp16":
        return round_f16(exact)
    if dtype == "bf16":
        return round_bf16(exact.astype(np.float32))
    if dtype == "fp8":
        return round_e4m3(exact.astype(np.float32))
    raise ValueError(dtype)


def apply_per_channel_scale(act, pre_quant_scale, in_dtype: str, out_dtype: str | None = None) -> np.ndarray:
    """smoothed[m, k] = T_out(T_in(act[m, k] * pqs[k])) (preQuantScaleKernel.cu:42-90: one multiply in
    the input type (`__hmul2`), then for W4A8 a cast of that T_in value to e4m3).  The product of
    two fp16/bf16 numbers is exact in float64, so one rounding to T_in is the type's own multiply."""
    prod = np.asarray(act, np.float32).astype(np.float64) * np.asarray(pre_quant_scale, np.float32).astype(np.float64)
    t = round_f16(prod) if in_dtype == "fp16" else round_to(prod.astype(np.float32), in_dtype)
    if out_dtype is None or out_dtype == in_dtype:
        return t
    return round_to(t, out_dtype)


def rmsnorm_ref(x, gamma, eps: float, dtype: str, beta=None) -> np.ndarray:
    """T(x * rsqrt(mean(x^2) + eps) * gamma [+ beta]) with the reference kernel's float32 steps
    (kernels/rmsnormKernels.cu:29-38 compute_rmsnorm: val * s_variance * gamma, then + beta, each a
    float32 operation; :106-107 variance / hidden_dim, rsqrtf(variance + eps); :124 cast to T).  The
    sum of squares is taken in float64 here: its float32 summation order is the kernel's own."""
    x = np.asarray(x, np.float32)
    var = (x.astype(np.float64) ** 2).sum(-1, keepdims=True) / x.shape[-1]
    inv = (1.0 / np.sqrt(var.astype(np.float32) + np.float32(eps))).astype(np.float32)
    y = (x * inv).astype(np.float32) * np.asarray(gamma, np.float32)
    if beta is not None:
        y = y.astype(np.float32) + np.asarray(beta, np.float32)
    return round_to(y.astype(np.float32), dtype)


def woq_matmul_ref(act, q, scales, zeros=None, bias=None, pre_quant_scale=None, alpha: float = 1.0,
                   group_size: int = 0, act_dtype: str = "bf16", w4a8: bool = False) -> np.ndarray:
    """The dequantize-then-matmul path with float64 accumulation (well inside "fp32 accumulated"):
    out = alpha * (smooth(act) @ dequant(q)) + bias, NOT rounded to the output type.
    With w4a8, `act` already holds e4m3 values when pre_quant_scale is None; otherwise the
    product act*pqs is rounded to e4m3 (the reference's apply_per_channel_scale<T, fp8>)."""
    a = np.asarray(act, np.float32)
    if pre_quant_scale is not None:
        a = apply_per_channel_scale(a, pre_quant_scale, act_dtype, "fp8" if w4a8 else None)
    w = dequantize(q, scales, zeros, group_size, "fp8" if w4a8 else act_dtype)
    out = a.astype(np.float64) @ w.astype(np.float64)
    out = out * float(alpha)
    if bias is not None:
        out = out + np.asarray(bias, np.float32).reshape(1, -1).astype(np.float64)
    return out


def activation_ref(x, name: str) -> np.ndarray:
    """The MoE activations in float64 (tests/functional/test_moe.py:173-190: torch gelu is the erf
    form; a gated activation takes value = first half, gate = second half of the last axis and
    returns value * f(gate), functional.py:804-821)."""
    from scipy.special import erf
    x = np.asarray(x, np.float64)
    f = {"gelu": lambda v: 0.5 * v * (1.0 + erf(v / np.sqrt(2.0))), "relu": lambda v: np.maximum(v, 0.0),
         "silu": lambda v: v / (1.0 + np.exp(-v)), "identity": lambda v: v}
    if name in ("swiglu", "geglu"):
        half = x.shape[-1] // 2
        return x[..., :half] * f["silu" if name == "swiglu" else "gelu"](x[..., half:])
    return f[name](x)


def grouped_matmul_ref(act, q, scales, zeros, bias, total_rows_before_expert, group_size: int = 0,
                       act_dtype: str = "bf16", activation: str = "identity", residual=None) -> np.ndarray:
    """The MoE expert GEMM (MoeGemmRunner::moeGemm / moeGemmBiasAct,
    kernels/internal_cutlass_kernels/include/moe_gemm_kernels.h:235-244; the CUTLASS problem visitor
    gives expert e the rows [total[e-1], total[e]), cutlass_extensions/gemm/kernel/moe_problem_visitor.h:163-176):
    rows of expert e times ITS dequantized weight, plus its bias row, then the activation on the
    unrounded sums (the fused epilogue's order, fused_moe_kernel_routine.cuh:380-400).  q [E, K, N],
    scales / zeros [E, N] or [E, K/g, N], bias [E, N]; float64 accumulation, not rounded.  `residual`
    (an extension of this library, the skip connection) is added last."""
    act = np.asarray(act, np.float32)
    total = np.asarray(total_rows_before_expert, np.int64)
    out = np.zeros((act.shape[0], np.asarray(q).shape[2]), np.float64)
    begin = 0
    for e, end in enumerate(total):
        end = int(end)
        if end > begin:
            out[begin:end] = woq_matmul_ref(act[begin:end], q[e], scales[e], None if zeros is None else zeros[e],
                                            None if bias is None else bias[e], None, 1.0, group_size, act_dtype)
        begin = end
    out = activation_ref(out, activation)
    return out if residual is None else out + np.asarray(residual, np.float64)


def max_rel_err(out, ref) -> float:
    """The parity norm used by every output test: max|out - ref| / max|ref|."""
    ref = np.asarray(ref, np.float64)
    denom = np.abs(ref).max()
    return float(np.abs(np.asarray(out, np.float64) - ref).max() / (denom if denom > 0 else 1.0))


def column_magnitude(act, w, alpha: float = 1.0) -> np.ndarray:
    """Expected magnitude of one output of column n when the signs of its K products are random:
    sqrt(mean_m sum_k (alpha * a[m, k] * w[k, n])^2).  The floor of the per-column norm below."""
    a2 = np.asarray(act, np.float64) ** 2
    w2 = np.asarray(w, np.float64) ** 2
    return abs(float(alpha)) * np.sqrt((a2 @ w2).mean(axis=0))


def max_col_rel_err(out, ref, col_floor=None) -> float:
    """Per-output-column parity norm: max_n ( max_m |out - ref|[m, n] / max(max_m |ref|[m, n], floor[n]) ).
    A wrong strip or column shows here whatever the magnitude of the other columns.  `col_floor`
    (column_magnitude of the same operands) keeps the norm meaningful when a column's few outputs all
    happen to lie near zero (M = 1: the elementwise relative error is ill-defined there)."""
    ref = np.asarray(ref, np.float64)
    ref = ref.reshape(-1, ref.shape[-1])
    err = np.abs(np.asarray(out, np.float64).reshape(ref.shape) - ref).max(axis=0)
    denom = np.abs(ref).max(axis=0)
    if col_floor is not None:
        denom = np.maximum(denom, np.asarray(col_floor, np.float64))
    return float((err / np.where(denom > 0, denom, 1.0)).max())


# --------------------------------------------------------------------------------------
# checkpoint-side folding rules (callers of the op)
# --------------------------------------------------------------------------------------


def fold_zero_points(zero_points, scales, bits: int = 4, gptq_minus_one: bool = False, dtype: str = "bf16"):
    """zeros = (2^(bits-1) - zp - [GPTQ ? 1 : 0]) * scale, in the scale dtype
    (tensorrt_llm/quantization/functional.py:1010-1014)."""
    z = (float(1 << (bits - 1)) - np.asarray(zero_points, np.float32) - (1.0 if gptq_minus_one else 0.0))
    return round_to((z.astype(np.float64) * np.asarray(scales, np.float32).astype(np.float64)).astype(np.float32), dtype)


# --------------------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations (seeded)
# --------------------------------------------------------------------------------------


def make_w8_per_channel(K: int, N: int, seed: int, dtype: str = "fp16"):
    """W ~ N(0, 0.02); scale_n = absmax_n / 127 in `dtype`; q = clamp(rint(W / scale), -127, 127)."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    scale = round_to(np.abs(w).max(axis=0) / np.float32(127.0), dtype)
    q = np.clip(np.rint(w / np.where(scale == 0, 1, scale)), -127, 127).astype(np.int8)
    return q, scale


def make_w4_groupwise_asym(K: int, N: int, group: int, seed: int, dtype: str = "bf16"):
    """W ~ N(0, 0.02); per (group, column): scale = (max - min)/15, zp = rint(-min/scale) in [0, 15],
    q_u4 = clamp(rint(W/scale) + zp, 0, 15).  Returns (q_signed = q_u4 - 8, scales, zeros) with
    zeros = (8 - zp) * scale, the pre-scaled additive form the op takes."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    wg = w.reshape(K // group, group, N)
    mx, mn = wg.max(axis=1), wg.min(axis=1)
    scale = round_to(np.maximum(mx - mn, 1e-8) / np.float32(15.0), dtype)
    zp = np.clip(np.rint(-mn / scale), 0, 15)
    qu = np.clip(np.rint(wg / scale[:, None, :]) + zp[:, None, :], 0, 15)
    q = (qu - 8).reshape(K, N).astype(np.int8)
    zeros = fold_zero_points(zp, scale, 4, False, dtype)
    return q, scale, zeros


def make_w4_groupwise_sym(K: int, N: int, group: int, seed: int, dtype: str = "bf16"):
    """Symmetric int4: scale = absmax_group / 8 (documented choice), q = clamp(rint(W/scale), -8, 7)."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    wg = w.reshape(K // group, group, N)
    scale = round_to(np.maximum(np.abs(wg).max(axis=1), 1e-8) / np.float32(8.0), dtype)
    q = np.clip(np.rint(wg / scale[:, None, :]), -8, 7).reshape(K, N).astype(np.int8)
    return q, scale


def make_activations(M: int, K: int, seed: int, dtype: str = "bf16"):
    rng = np.random.default_rng(seed)
    return round_to(rng.standard_normal((M, K), dtype=np.float32), dtype)


def make_w4a8_problem(M: int, K: int, N: int, seed: int, out_dtype: str = "bf16"):
    """The W4A8 AWQ-style configuration: int4 symmetric g128, smoothing vector ~ U(0.5, 2),
    activations bf16 ~ N(0,1).  Applies the loader's folding
    (tensorrt_llm/models/modeling_utils.py:1661-1682): the per-tensor weight scale wsf2 is
    divided out of the group scales (stored as fp16), the activation scale out of the smoothing
    vector, and alpha = act_sf * wsf2."""
    q, scale = make_w4_groupwise_sym(K, N, 128, seed, "fp32")
    rng = np.random.default_rng(seed + 7)
    smooth = round_to(rng.uniform(0.5, 2.0, size=(K,)).astype(np.float32), out_dtype)
    act = make_activations(M, K, seed + 13, out_dtype)
    amax_act = np.abs(act * smooth).max()
    act_sf = np.float32(amax_act / 448.0)
    wsf2 = np.float32(np.abs(q.astype(np.float32).reshape(K // 128, 128, N) * scale[:, None, :]).max() / 448.0)
    scales_h = round_f16(scale / wsf2)
    pqs = round_to(smooth / act_sf, out_dtype)
    alpha = float(act_sf * wsf2)
    return dict(act=act, q=q, scales=scales_h, pre_quant_scale=pqs, alpha=alpha)


# --------------------------------------------------------------------------------------
# the reference's CPU path, timed by bench.py as `cpu_baseline` (kind "port"):
# torch dequant + float32 matmul (tensorrt_llm/quantization/functional.py:223-234,269-290)
# --------------------------------------------------------------------------------------


def torch_cpu_dequant_matmul(act_f32, q_i8, scales_f32, zeros_f32, group_size: int):
    """act [M,K] float32 torch tensor, q [K,N] int8, scales/zeros [K/g, N] float32 -> [M,N] float32."""
    import torch

    K = q_i8.shape[0]
    if group_size:
        s = scales_f32.repeat_interleave(group_size, dim=0)[:K]
        w = q_i8.to(torch.float32) * s
        if zeros_f32 is not None:
            w = w + zeros_f32.repeat_interleave(group_size, dim=0)[:K]
    else:
        w = q_i8.to(torch.float32) * scales_f32.reshape(1, -1)
    return act_f32 @ w
