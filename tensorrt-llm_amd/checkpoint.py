"""Checkpoint front-end: float / GPTQ / AutoAWQ / ModelOpt tensors -> the operands of the two matmul ops.

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

  * ModelOpt AWQ (the reference's own quantizer): `weight` int8 [N/2, K] (two output channels per
    byte, signed nibbles), `weight_scale` [N, K/g], `input_quantizer._pre_quant_scale` [K]; for W4A8
    also the per-tensor `activation_scaling_factor` and `weights_scaling_factor_2`, folded by the
    loader (tensorrt_llm/models/modeling_utils.py:1626-1682): `postprocess_modelopt_awq`, `fold_w4a8`.
  * float weights of per-channel layers (W8A16 / W4A16): `postprocess_weight_only`
    (functional.py:875-901: transpose, TP split, padding, symmetric quantization, bias).
  * q / k / v (or gate / up) tensors that arrive separately are concatenated along N first
    (functional.py:932-944): `concat_gptq_parts`, and list arguments of `postprocess_modelopt_awq`.

Returned tensors are what `weight_only_groupwise_quant_matmul` takes: `weight` in this library's
gfx950 layout (opaque bytes), `weights_scaling_factor` [K/g, N] and `zero` [K/g, N] in `dtype`.
All tensors are CPU tensors, as in the reference's loader.

`load_trtllm_linear` reads one linear layer of a TensorRT-LLM checkpoint (`rank<r>.safetensors` +
`config.json`, docs/source/architecture/checkpoint.md:94-176; tensor names of
quantization/layers.py:744-751, 998-1037) whose `weight` was already laid out by the reference's
preprocess for some SM, decodes that layout and re-lays it out for gfx950.

The three small helpers `unpack_int32_into_int8`, `change_qkv_leading_dim` and `pad_like` follow the
reference's helpers of the same names closely (functional.py:833-872): each has one obvious
implementation, and the loaders above call them with the reference's argument conventions.
"""
from __future__ import annotations

import json
import os

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


def concat_gptq_parts(parts):
    """[(qweight, scales, qzeros), ...] of layers that share their input (q, k, v or gate, up) -> one
    (qweight, scales, qzeros) with the output columns side by side.  All three GPTQ / AutoAWQ tensors
    keep N (or N/8) in their last dimension, so this is a concatenation along it
    (functional.py:939-943: `torch.cat(weights[i::len(weights) // 3], dim=1)`)."""
    return tuple(torch.cat([p[i] for p in parts], dim=1) for i in range(3))


def fold_w4a8(weights_scaling_factor: torch.Tensor, prequant_scaling_factor: torch.Tensor,
              activation_scaling_factor: torch.Tensor, weights_scaling_factor_2: torch.Tensor):
    """The W4A8 loader fold (tensorrt_llm/models/modeling_utils.py:1661-1682), in its order of
    operations: the group scales are divided by the per-tensor weight scale in their own type and then
    stored as float16 (the fp8 kernels read half scales whatever the activation type:
    weightOnlyGroupwiseQuantMatmulPlugin.cpp:254); the smoothing vector is divided by the per-tensor
    activation scale (so that smoothed activations land in the e4m3 range); alpha = their product
    restores the magnitude in the epilogue.  Returns the four tensors under the reference's names."""
    act_sf = torch.as_tensor(activation_scaling_factor)
    wsf2 = torch.as_tensor(weights_scaling_factor_2)
    # the reference divides IN PLACE (`weights[name] /= ...`): whatever the type and shape of the per-tensor
    # factors (the layers declare them float32 of shape (1,), quantization/layers.py), the quotient is
    # formed in the promoted type and rounded back to the tensor's own dtype, which the tensor keeps
    scales = weights_scaling_factor.clone()
    scales /= wsf2
    pqs = prequant_scaling_factor.clone()
    pqs /= act_sf
    return {
        "weights_scaling_factor": scales.to(torch.float16).contiguous(),
        "prequant_scaling_factor": pqs.contiguous(),
        "alpha": (act_sf.to(torch.float32) * wsf2.to(torch.float32)).reshape(1),
        "activation_scaling_factor": act_sf,
    }


def postprocess_weight_only(weight: torch.Tensor, quant_type: torch.dtype = torch.int8, *, bias: torch.Tensor | None = None,
                            tp_split=None, padded_shape=None):
    """Per-channel loader hook: a float weight of one linear layer -> {"weight", "per_channel_scale"}
    (+ "bias"), the operands of `weight_only_quant_matmul` (W8A16 with quant_type torch.int8, W4A16 with
    torch.quint4x2).  Counterpart of `postprocess_weight_only`
    (tensorrt_llm/quantization/functional.py:875-901), in its order of operations:

      * `weight` [out_features, in_features] (or [E, out, in]) as checkpoints store it is transposed to the
        op's [K, N];
      * `tp_split` = (dim, size, rank) cuts the logical [K, N] weight (dim 1: column-parallel, 0:
        row-parallel).  With `padded_shape` = the layer's (in_features, out_features) AFTER padding
        (see padded_features) the cut is the reference's `torch.split(v, padded size, dim)[rank]`: ranks
        own runs of the padded per-rank size, the last one what is left, and each piece is padded with
        zeros up to the padded shape; without it the weight is cut into `size` equal parts;
      * `symmetric_quantize_last_axis_of_batched_matrix` (one scale per output column: amax / 2^(bits-1),
        round half away from zero) quantizes the piece and lays it out for the kernels;
      * the bias follows the columns of a column-parallel layer (split and padded the same way) and is
        passed through otherwise."""
    if quant_type not in (torch.int8, torch.quint4x2):
        raise ValueError("quant_type must be torch.int8 or torch.quint4x2")
    if weight.dim() not in (2, 3) or not weight.is_floating_point():
        raise ValueError("a float weight [out_features, in_features] (or [E, out, in]) is required")
    v = weight.transpose(-1, -2)
    tp_dim = None
    if tp_split is not None:
        tp_dim, tp_size, tp_rank = tp_split
        if tp_dim not in (0, 1) or not 0 <= tp_rank < tp_size:
            raise ValueError("tp_split is (dim 0 | 1, size, rank)")
        axis = tp_dim + (v.dim() - 2)
        if padded_shape is not None:
            pieces = torch.split(v, padded_shape[tp_dim], axis)
            if tp_rank >= len(pieces):
                raise ValueError("rank %d owns nothing: %d pieces of %d" % (tp_rank, len(pieces), padded_shape[tp_dim]))
            v = pieces[tp_rank]
        else:
            v = v.chunk(tp_size, axis)[tp_rank]
    if padded_shape is not None:
        v = pad_like(v, tuple(v.shape[:-2]) + tuple(padded_shape))
    processed, scales = ops.symmetric_quantize_last_axis_of_batched_matrix(v.contiguous(), quant_type)
    out = {"weight": processed, "per_channel_scale": scales}
    if bias is not None:
        if tp_dim == 1:
            if padded_shape is not None:
                bias = torch.split(bias, padded_shape[1], -1)[tp_rank]
            else:
                bias = bias.chunk(tp_size, -1)[tp_rank]
        if padded_shape is not None:
            bias = pad_like(bias, tuple(bias.shape[:-1]) + (padded_shape[1],))
        out["bias"] = bias.contiguous()
    return out


def postprocess_modelopt_awq(weight, weight_scale, pre_quant_scale, dtype=torch.float16, *, group_size: int = 128,
                             activation_scaling_factor=None, weights_scaling_factor_2=None, tp_split=None):
    """ModelOpt AWQ tensors of one linear layer -> {"weight", "weights_scaling_factor",
    "prequant_scaling_factor"} (+ "alpha", "activation_scaling_factor" for W4A8, when the two
    per-tensor factors are given).

    `weight` int8 [N/2, K]: byte (j, k) holds output channels 2j (low nibble) and 2j + 1 of input k as
    signed 4-bit values; its transpose is the row-major packed [K, N/2] tensor the preprocess takes
    (modeling_utils.py:1645-1648; functional.py:950-957 unpacks and re-packs the same nibbles).
    `weight_scale` [N, K/g] (any shape with that many elements in that order: functional.py:918-931
    reshapes what ModelOpt exports) becomes [K/g, N]; `pre_quant_scale` [K] becomes [1, K].
    Lists of tensors (q, k, v that arrive separately) are concatenated along N; the smoothing vector is
    shared, the first one is taken (functional.py:932-937).  `tp_split` = (dim, size, rank) as in
    postprocess_gptq, applied to each part before the concatenation as the reference does."""
    w4a8 = activation_scaling_factor is not None
    weights = list(weight) if isinstance(weight, (list, tuple)) else [weight]
    scales = list(weight_scale) if isinstance(weight_scale, (list, tuple)) else [weight_scale]
    pqs = pre_quant_scale[0] if isinstance(pre_quant_scale, (list, tuple)) else pre_quant_scale
    if len(weights) != len(scales):
        raise ValueError("as many weight_scale tensors as weight tensors are required")
    packed, scale_parts = [], []
    for w, sc in zip(weights, scales):
        if w.dtype != torch.int8 or w.dim() != 2:
            raise ValueError("ModelOpt AWQ weights are int8 [N/2, K]")
        k = w.shape[1]
        if k % group_size:
            raise ValueError("in_features must be a multiple of the group size")
        wt = w.T.contiguous()  # [K, N/2], row-major, even column in the low nibble
        st = sc.reshape(w.shape[0] * 2, k // group_size).T  # [K/g, N]
        if tp_split is not None:
            tp_dim, tp_size, tp_rank = tp_split
            wt = wt.chunk(tp_size, tp_dim)[tp_rank]
            st = st.chunk(tp_size, tp_dim)[tp_rank]
        packed.append(wt)
        scale_parts.append(st)
    wt = torch.cat(packed, dim=1).contiguous()
    st = torch.cat(scale_parts, dim=1).to(dtype).contiguous()
    pqs = pqs.to(dtype).reshape(1, -1)
    if tp_split is not None and tp_split[0] == 0:  # row-parallel: the smoothing vector follows the rows of K
        pqs = pqs.chunk(tp_split[1], 1)[tp_split[2]]
    act_type = torch.float8_e4m3fn if w4a8 else dtype
    out = {"weight": ops.preprocess_weights_for_mixed_gemm(wt, torch.quint4x2, act_type),
           "weights_scaling_factor": st, "prequant_scaling_factor": pqs.contiguous()}
    if w4a8:
        if weights_scaling_factor_2 is None:
            raise ValueError("W4A8 needs weights_scaling_factor_2 next to activation_scaling_factor")
        out.update(fold_w4a8(st, out["prequant_scaling_factor"], activation_scaling_factor, weights_scaling_factor_2))
    return out


# quant_algo strings of a checkpoint's config.json (tensorrt_llm/quantization/mode.py QuantAlgo) that
# name a weight-only linear layer: (weight bits, groupwise?, fp8 activations?)
_QUANT_ALGOS = {"W8A16": (8, False, False), "W4A16": (4, False, False), "W4A16_AWQ": (4, True, False),
                "W4A8_AWQ": (4, True, True), "W4A16_GPTQ": (4, True, False), "W8A16_GPTQ": (8, True, False)}


def load_trtllm_linear(checkpoint, prefix: str, *, sm_arch: int, quant_algo: str | None = None,
                       group_size: int | None = None, rank: int = 0):
    """One weight-only linear layer of a TensorRT-LLM checkpoint -> the operands of this library's matmul.

    `checkpoint`: a checkpoint directory (`config.json` + `rank<rank>.safetensors`) or a dict of
    tensors.  `prefix`: the layer's name, e.g. "transformer.layers.0.mlp.fc".  `sm_arch`: the SM the
    checkpoint's weights were preprocessed for (the byte layout differs: 90 has no column
    interleave; the checkpoint does not record it).  `quant_algo` / `group_size` default to
    config.json's `quantization` section.

    Tensors read (quantization/layers.py:744-751 per-channel, :998-1037 groupwise):
      <prefix>.weight                   int8 [K, N*bits/8], or typed as the activation dtype
                                        ([K, N/4] halfs for int4, [K, N/2] for int8)
      <prefix>.per_channel_scale        [N]                 (W8A16 / W4A16)
      <prefix>.weights_scaling_factor   [K/g, N]            (groupwise; float16 bits for W4A8)
      <prefix>.zero                     [K/g, N]            optional
      <prefix>.prequant_scaling_factor  [1, K]              optional (AWQ)
      <prefix>.alpha                    [1] float32         W4A8
      <prefix>.bias                     [N]                 optional
    Returns a dict: weight (gfx950 layout), scales, zeros, pre_quant_scale, bias (None where absent),
    alpha, n, k, group_size, quant_algo (the op's bit flags), bits, w4a8."""
    if isinstance(checkpoint, (str, os.PathLike)):
        from safetensors import safe_open
        cfg_path = os.path.join(checkpoint, "config.json")
        if os.path.exists(cfg_path):
            with open(cfg_path) as f:
                q = json.load(f).get("quantization", {})
            quant_algo = quant_algo or q.get("quant_algo")
            group_size = group_size if group_size is not None else q.get("group_size")
        tensors = {}
        with safe_open(os.path.join(checkpoint, "rank%d.safetensors" % rank), framework="pt", device="cpu") as f:
            for key in f.keys():
                if key.startswith(prefix + "."):
                    tensors[key] = f.get_tensor(key)
    else:
        tensors = {k: v for k, v in checkpoint.items() if k.startswith(prefix + ".")}
    if quant_algo not in _QUANT_ALGOS:
        raise ValueError("quant_algo %r is not a weight-only algorithm this loader knows (%s)"
                         % (quant_algo, ", ".join(sorted(_QUANT_ALGOS))))
    bits, groupwise, w4a8 = _QUANT_ALGOS[quant_algo]
    get = lambda name: tensors.get(prefix + "." + name)
    weight = get("weight")
    if weight is None:
        raise KeyError(prefix + ".weight")
    weight = weight.contiguous().view(torch.int8)  # groupwise layers type the bytes as the activation dtype
    k, n = weight.shape[0], weight.shape[1] * 8 // bits
    quant_type = torch.int8 if bits == 8 else torch.quint4x2
    act_type = torch.float8_e4m3fn if w4a8 else torch.float16
    row_major = ops.import_reference_weights(weight, quant_type, act_type, sm_arch)
    out = {"weight": ops.preprocess_weights_for_mixed_gemm(row_major, quant_type, act_type), "n": n, "k": k,
           "bits": bits, "w4a8": w4a8, "zeros": None, "pre_quant_scale": None, "alpha": 1.0, "bias": get("bias")}
    from .functional import BIAS, ZERO, PRE_QUANT_SCALE, FP8_ALPHA, INT8_WEIGHT
    algo = (INT8_WEIGHT if bits == 8 and groupwise else 0) | (BIAS if out["bias"] is not None else 0)
    if not groupwise:
        scales = get("per_channel_scale")
        if scales is None:
            raise KeyError(prefix + ".per_channel_scale")
        out.update(scales=scales.reshape(-1).contiguous(), group_size=0)
    else:
        scales = get("weights_scaling_factor")
        if scales is None:
            raise KeyError(prefix + ".weights_scaling_factor")
        if not group_size:
            group_size = k // scales.shape[0]
        if w4a8:  # float16 values stored under the activation dtype's name
            scales = scales.contiguous().view(torch.float16)
        out.update(scales=scales.contiguous(), group_size=int(group_size))
        zero, pqs = get("zero"), get("prequant_scaling_factor")
        if zero is not None:
            out["zeros"] = (zero.contiguous().view(torch.float16) if w4a8 else zero).contiguous()
            algo |= ZERO
        if pqs is not None:
            out["pre_quant_scale"] = pqs.reshape(-1).contiguous()
            algo |= PRE_QUANT_SCALE
        if w4a8:
            alpha = get("alpha")
            if alpha is None:
                raise KeyError(prefix + ".alpha")
            out["alpha"] = float(alpha.reshape(-1)[0])
            algo |= FP8_ALPHA
    out["quant_algo"] = algo
    return out


def linear_forward(layer: dict, x: torch.Tensor, device=None) -> torch.Tensor:
    """Runs a layer returned by load_trtllm_linear on the GPU: moves its tensors there on first use and
    calls the matching op (per-channel: weight_only_quant_matmul's kernel, groupwise: the groupwise one;
    the bias of a per-channel layer, which that plugin does not take, is added afterwards as the
    reference's layer does, quantization/layers.py:769-776)."""
    from . import functional as F
    device = device or x.device
    if "_dev" not in layer:
        layer["_dev"] = {key: (v.to(device) if isinstance(v, torch.Tensor) else v) for key, v in layer.items()
                         if key in ("weight", "scales", "zeros", "pre_quant_scale", "bias")}
    d = layer["_dev"]
    if layer["group_size"] == 0:
        algo = F.INT8_WEIGHT if layer["bits"] == 8 else 0
        out = F.woq_matmul_raw(x, None, d["weight"], d["scales"], None, None, n=layer["n"], k=layer["k"], group_size=0,
                               quant_algo=algo, out_dtype=x.dtype)
        return out if d["bias"] is None else out + d["bias"]
    out_dtype = x.dtype if x.dtype != torch.float8_e4m3fn else (d["bias"].dtype if d["bias"] is not None
                                                                 else torch.float16)
    algo = layer["quant_algo"]
    pqs = d["pre_quant_scale"]
    if x.dtype == torch.float8_e4m3fn:  # activations already smoothed and cast
        algo &= ~F.PRE_QUANT_SCALE
        pqs = None
    return F.woq_matmul_raw(x, pqs, d["weight"], d["scales"], d["zeros"], d["bias"], n=layer["n"], k=layer["k"],
                            group_size=layer["group_size"], quant_algo=algo, alpha=layer["alpha"], out_dtype=out_dtype)
