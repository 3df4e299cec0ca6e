"""Checkpoint front-end: GPTQ / AutoAWQ tensors -> the operands of the groupwise matmul.

Counterpart of `postprocess_weight_only_groupwise` and its helpers
(tensorrt_llm/quantization/functional.py:832-868, 903-1037), which the reference's weights loader
calls per tensor.  Same arithmetic, same argument conventions:

  * GPTQ (AutoGPTQ): `qweight` int32 [K/8, N] (8 rows per word, row i in bits 4*(i%8)),
    `scales` [K/g, N], `qzeros` int32 [K/g, N/8] (8 columns per word, storing zero_point - 1);
    int8 GPTQ: `qweight` int32 [K/4, N] (4 rows per word), `qzeros` int32 [K/g, N/4].
  * AutoAWQ: `qweight` int32 [K, N/8] and `qzeros` int32 [K/g, N/8], 8 columns per word in the
    order 0,2,4,6,1,3,5,7 (undone by the gather [0,4,1,5,2,6,3,7], functional.py:843-845).
  * the op takes signed weights q = u - 8 (u - 128) and ADDITIVE, pre-scaled zeros
    `zero = (8 - qzero - [GPTQ]) * scale` (128 for int8), functional.py:1010-1014.

Returned tensors are what `weight_only_groupwise_quant_matmul` takes: `weight` in this library's
gfx950 layout (opaque bytes), `weights_scaling_factor` [K/g, N] and `zero` [K/g, N] in `dtype`.
All tensors are CPU tensors, as in the reference's loader.
"""
from __future__ import annotations

import torch

from . import ops

AWQ_UNPACK_ORDER = [0, 4, 1, 5, 2, 6, 3, 7]


def unpack_int32_into_int8(w_packed: torch.Tensor, autoawq_reorder: bool = False) -> torch.Tensor:
    """[R, C] int32 (or any 4-byte type) -> [R, 8*C] int8 holding the unsigned nibbles, low nibble
    first (functional.py:834-846)."""
    b = w_packed.contiguous().view(torch.uint8)
    out = torch.empty(b.shape[0], b.shape[1] * 2, dtype=torch.int8)
    out[:, ::2] = (b % 16).to(torch.int8)
    out[:, 1::2] = (b // 16).to(torch.int8)
    if autoawq_reorder:
        out = out.view(-1, 8)[:, AWQ_UNPACK_ORDER].reshape(out.shape)
    return out.contiguous()


def change_qkv_leading_dim(w: torch.Tensor, num_heads: int) -> torch.Tensor:
    """[.., heads*3*d] stored head-major (h, qkv, d) -> (qkv, h, d) (functional.py:849-858)."""
    if w.dim() == 1:
        return w.reshape(num_heads, 3, -1).transpose(0, 1).reshape(-1)
    shape = w.shape
    head_dim = shape[1] // (3 * num_heads)
    return w.reshape(-1, num_heads, 3, head_dim).transpose(1, 2).reshape(shape[0], -1)


def pad_like(w: torch.Tensor, target_shape, value=0) -> torch.Tensor:
    """Pads every dimension at its end up to target_shape (functional.py:861-872)."""
    if tuple(w.shape) == tuple(target_shape):
        return w
    pad = []
    for dim in range(len(target_shape)):
        cur = -1 - dim
        pad += [0, max(0, target_shape[cur] - w.shape[cur])]
    return torch.nn.functional.pad(w, pad, value=value)


def padded_features(in_features: int, out_features: int, group_size: int, tp_size: int = 1, w4a8: bool = False):
    """The layers' padding rule (quantization/layers.py:719-726, 965-972): per-channel layers round
    both feature counts up to 64*tp, groupwise layers to max(64 | 128 for W4A8, group_size)*tp."""
    mult = (64 if group_size == 0 else max(128 if w4a8 else 64, group_size)) * tp_size
    up = lambda v: (v + mult - 1) // mult * mult
    return up(in_features), up(out_features)


def _signed_to_packed(q_signed: torch.Tensor) -> torch.Tensor:
    """[K, N] int8 in [-8, 7] -> [K, N/2] int8, two's-complement nibbles, even column low
    (functional.py:956-957, 975-976)."""
    u = q_signed.clone()
    u[u < 0] += 16
    u = u.view(torch.uint8)
    return (u[:, 1::2] * 16 + u[:, ::2]).view(torch.int8).contiguous()


def _finish(q_signed, scales, qzeros, bits, use_gptq, dtype, tp_split, padded_shape, num_heads):
    half = 1 << (bits - 1)
    if num_heads:
        q_signed = change_qkv_leading_dim(q_signed, num_heads)
        scales = change_qkv_leading_dim(scales, num_heads)
        qzeros = change_qkv_leading_dim(qzeros, num_heads)
    if tp_split is not None:
        tp_dim, tp_size, tp_rank = tp_split
        q_signed = q_signed.chunk(tp_size, tp_dim)[tp_rank]
        # groups follow rows, columns follow columns
        scales = scales.chunk(tp_size, tp_dim)[tp_rank]
        qzeros = qzeros.chunk(tp_size, tp_dim)[tp_rank]
    if padded_shape is not None:
        k_pad, n_pad = padded_shape
        group = q_signed.shape[0] // scales.shape[0]
        q_signed = pad_like(q_signed, (k_pad, n_pad))
        scales = pad_like(scales, (k_pad // group, n_pad), 1)
        qzeros = pad_like(qzeros, (k_pad // group, n_pad), half - 1)  # 7 for int4, as the reference pads
    q_signed = q_signed.contiguous()
    if bits == 4:
        weight = ops.preprocess_weights_for_mixed_gemm(_signed_to_packed(q_signed), torch.quint4x2, dtype)
    else:
        weight = ops.preprocess_weights_for_mixed_gemm(q_signed, torch.int8, dtype)
    scales = scales.to(dtype).contiguous()
    # same operation order and types as the reference: integer offset, times the scale in `dtype`
    zeros = ((-qzeros.to(torch.int32) + half - (1 if use_gptq else 0)).to(dtype) * scales).to(dtype).contiguous()
    return {"weight": weight, "weights_scaling_factor": scales, "zero": zeros}


def postprocess_gptq(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor, dtype=torch.float16, *,
                     bits: int = 4, tp_split=None, padded_shape=None, num_heads: int = 0):
    """AutoGPTQ tensors of one linear layer -> {"weight", "weights_scaling_factor", "zero"}.
    `tp_split` = (dim, size, rank) cuts the logical [K, N] weight like the reference's loader
    (dim 1 for column-parallel, 0 for row-parallel); `padded_shape` = (K, N) to pad up to;
    `num_heads` != 0 applies the fused-QKV head reordering (`using_head_as_leading_dim`)."""
    if bits == 4:
        q_signed = unpack_int32_into_int8(qweight.T).T - 8  # functional.py:946-947
        qz = unpack_int32_into_int8(qzeros, False)
    elif bits == 8:
        # 4 rows per int32 word, low byte first (functional.py:958-962)
        q_signed = (qweight.T.contiguous().view(torch.uint8).T.contiguous().to(torch.int16) - 128).to(torch.int8)
        qz = qzeros.contiguous().view(torch.uint8)
    else:
        raise ValueError("bits must be 4 or 8")
    return _finish(q_signed.contiguous(), scales, qz, bits, True, dtype, tp_split, padded_shape, num_heads)


def postprocess_autoawq(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor, dtype=torch.float16, *,
                        tp_split=None, padded_shape=None, num_heads: int = 0):
    """AutoAWQ (HF AWQ) int4 tensors of one linear layer -> {"weight", "weights_scaling_factor", "zero"}."""
    q_signed = unpack_int32_into_int8(qweight, True) - 8  # functional.py:948-949
    qz = unpack_int32_into_int8(qzeros, True)
    return _finish(q_signed.contiguous(), scales, qz, 4, False, dtype, tp_split, padded_shape, num_heads)
