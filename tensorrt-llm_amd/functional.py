"""The two matmul ops of the reference's quantization front end, run eagerly on torch device
tensors through libwoq's C ABI.

Mirrors tensorrt_llm/quantization/functional.py:216-347 (`weight_only_quant_matmul`,
`weight_only_groupwise_quant_matmul`): same argument order and meaning; the plugin path of the
reference is the semantic (zeros AND pre-quant scale both apply).  Weights are the opaque
tensors made by ops.preprocess_weights_for_mixed_gemm, moved to the GPU.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import lib, check, MatmulArgs, GroupedMatmulArgs

_DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, torch.float16: torch.float16,
           torch.bfloat16: torch.bfloat16}
_WOQ_DT = {torch.float16: _lib.FP16, torch.bfloat16: _lib.BF16, torch.float8_e4m3fn: _lib.FP8_E4M3}

# WeightOnlyQuantMatmulPlugin::WeightTypeId
# (cpp/tensorrt_llm/plugins/weightOnlyQuantMatmulPlugin/weightOnlyQuantMatmulPlugin.h:38-42)
INT8, INT4 = 1, 2
# quant_algo flags (plugins/weightOnlyGroupwiseQuantMatmulPlugin/weightOnlyGroupwiseQuantMatmulPlugin.cpp:29-37)
BIAS, ZERO, PRE_QUANT_SCALE, FP8_ALPHA, INT8_WEIGHT = 1, 2, 4, 8, 16


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream_handle(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise RuntimeError("weight-only matmul runs on the GPU only (got a %s tensor); "
                               "there is no CPU path" % t.device.type)
        if t is not None and not t.is_contiguous():
            raise RuntimeError("tensors must be contiguous")


def woq_matmul_raw(act, pre_quant_scale, weight, scales, zeros, bias, *, n: int, k: int, group_size: int,
                   quant_algo: int, alpha: float = 1.0, out_dtype=None, regime: int = 0, workspace=None,
                   out=None, static_scratch: bool = False) -> torch.Tensor:
    """One call of woq_matmul.  `act` is [..., k]; returns [..., n].  With `static_scratch` the call goes
    through woq_matmul_static: no workspace is allocated or passed, the library's own device array is
    used (pass `out` as well and the call allocates nothing at all)."""
    _require_gpu(act, pre_quant_scale, weight, scales, zeros, bias, workspace, out)
    out_dtype = out_dtype or (act.dtype if act.dtype != torch.float8_e4m3fn else scales.dtype)
    if act.shape[-1] != k:
        raise RuntimeError("activation has %d input features, weight expects %d" % (act.shape[-1], k))
    m = act.numel() // k if k else 0
    # the C ABI receives untyped pointers: a tensor of another element type would be read as the expected
    # one without any error.  16-bit activations and the smoothing vector are of the output type; scales
    # and zeros too, except for W4A8, whose kernels read float16 values whatever the output type (the
    # reference stores those bits under the activation type's name: a 2-byte tensor of either type passes)
    w4a8 = bool(quant_algo & FP8_ALPHA)
    if act.dtype != torch.float8_e4m3fn and act.dtype != out_dtype:
        raise RuntimeError("activation dtype %s does not match the output dtype %s" % (act.dtype, out_dtype))
    scale_types = (torch.float16, out_dtype) if w4a8 else (out_dtype,)
    for name, t, allowed in (("pre_quant_scale", pre_quant_scale, (out_dtype,)), ("scales", scales, scale_types),
                             ("zeros", zeros, scale_types), ("bias", bias, (out_dtype,))):
        if t is not None and t.dtype not in allowed:
            raise RuntimeError("%s has dtype %s, the op expects %s" % (name, t.dtype, " or ".join(map(str, allowed))))
    if out is None:
        out = torch.empty(act.shape[:-1] + (n,), dtype=out_dtype, device=act.device)
    elif out.dtype != out_dtype:
        raise RuntimeError("out has dtype %s, expected %s" % (out.dtype, out_dtype))
    need = 0 if static_scratch else lib.woq_workspace_bytes(m, n, k, quant_algo, _WOQ_DT[act.dtype])
    if need and workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=act.device)
    args = MatmulArgs(
        act=_ptr(act), pre_quant_scale=_ptr(pre_quant_scale), weight=_ptr(weight), scales=_ptr(scales),
        zeros=_ptr(zeros), bias=_ptr(bias), out=_ptr(out), alpha=float(alpha), m=m, n=n, k=k,
        group_size=group_size, quant_algo=quant_algo, act_dtype=_WOQ_DT[act.dtype], out_dtype=_WOQ_DT[out_dtype],
        regime=regime, workspace=_ptr(workspace),
        workspace_bytes=0 if workspace is None else workspace.numel() * workspace.element_size())
    entry = lib.woq_matmul_static if static_scratch else lib.woq_matmul
    check(entry(ctypes.byref(args), _stream_handle(act.device)))
    return out


def profile_tactics(pre_quant_scale, weight, scales, zeros, bias, *, n: int, k: int, group_size: int,
                    quant_algo: int, dtype: torch.dtype, min_m: int = 1, max_m: int = 4096, alpha: float = 1.0) -> int:
    """Times this library's candidate kernels for the layer on the current stream and records the
    fastest per row count (woq_profile_tactics; the reference does this in the plugins' initialize
    through GemmPluginProfiler::profileTactics, gemmPluginProfiler.cpp:118-216).  Allocates the
    activations, output and workspace of max_m rows itself, as the reference's profiler allocates its
    temporary buffers (gemmPluginProfiler.cpp:252-270).  Returns the number of table entries."""
    _require_gpu(pre_quant_scale, weight, scales, zeros, bias)
    dev = weight.device
    act = torch.randn((max_m, k), device=dev).to(dtype)
    out = torch.empty((max_m, n), dtype=dtype, device=dev)
    need = lib.woq_workspace_bytes(max_m, n, k, quant_algo, _WOQ_DT[dtype])
    # room for every split-K candidate, not only the heuristics' own
    need = max(need, max_m * k * 2 + 256 + min(max_m * n * 4 * 20, 160 << 20))
    workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    args = MatmulArgs(
        act=_ptr(act), pre_quant_scale=_ptr(pre_quant_scale), weight=_ptr(weight), scales=_ptr(scales),
        zeros=_ptr(zeros), bias=_ptr(bias), out=_ptr(out), alpha=float(alpha), m=max_m, n=n, k=k,
        group_size=group_size, quant_algo=quant_algo, act_dtype=_WOQ_DT[dtype], out_dtype=_WOQ_DT[dtype],
        regime=0, workspace=_ptr(workspace), workspace_bytes=workspace.numel())
    check(lib.woq_profile_tactics(ctypes.byref(args), min_m, max_m, _stream_handle(dev)))
    return lib.woq_tactic_count()


def describe_tactic(m: int, n: int, k: int, group_size: int, quant_algo: int, dtype: torch.dtype) -> str:
    """What a matmul call of this shape goes by: "heuristic" or the tuned table's entry."""
    args = MatmulArgs(m=m, n=n, k=k, group_size=group_size, quant_algo=quant_algo, act_dtype=_WOQ_DT[dtype],
                      out_dtype=_WOQ_DT[dtype], regime=0)
    buf = ctypes.create_string_buffer(128)
    check(lib.woq_describe_tactic(ctypes.byref(args), buf, len(buf)))
    return buf.value.decode()


def export_tactics() -> str:
    """The tuned table as text (store it next to the model; import_tactics loads it again)."""
    need = lib.woq_export_tactics(None, 0)
    buf = ctypes.create_string_buffer(need)
    lib.woq_export_tactics(buf, need)
    return buf.value.decode()


def import_tactics(text: str) -> None:
    check(lib.woq_import_tactics(text.encode()))


def clear_tactics() -> None:
    lib.woq_clear_tactics()


def tactic_count() -> int:
    return lib.woq_tactic_count()


def woq_grouped_matmul_raw(act, weight, scales, zeros, bias, total_rows_before_expert, *, n: int, k: int,
                           group_size: int, quant_algo: int, activation: str = "identity", residual=None,
                           regime: int = 0, out=None) -> torch.Tensor:
    """One call of woq_grouped_matmul (the MoE expert GEMM: moe_gemm_kernels.h:235-244 with weight-only
    scales).  `act` is [total_rows, k] sorted by expert, `weight` the preprocessed [E, ...] tensor,
    `scales` / `zeros` [E, n] or [E, k/group, n], `bias` [E, n], `total_rows_before_expert` an int64
    device tensor [E] of inclusive prefix sums (None: one expert owns every row).  `activation` is one
    of gelu / relu / silu / swiglu / geglu / identity (tensorrt_llm/layers/moe.py activation names);
    the gated ones return [total_rows, n/2].  `residual` [total_rows, n_out] is added after the activation."""
    _require_gpu(act, weight, scales, zeros, bias, total_rows_before_expert, residual, out)
    if total_rows_before_expert is not None and total_rows_before_expert.dtype != torch.int64:
        raise RuntimeError("total_rows_before_expert must be int64")
    if act.dim() != 2 or act.shape[1] != k:
        raise RuntimeError("activation must be [total_rows, %d]" % k)
    if activation not in _lib.ACTIVATIONS:
        raise RuntimeError("unknown activation %r" % (activation,))
    act_id = _lib.ACTIVATIONS[activation]
    n_out = n // 2 if activation in ("swiglu", "geglu") else n
    if out is None:
        out = torch.empty((act.shape[0], n_out), dtype=act.dtype, device=act.device)
    if residual is not None and (tuple(residual.shape) != (act.shape[0], n_out) or residual.dtype != act.dtype):
        raise RuntimeError("residual must be [%d, %d] of the activation dtype" % (act.shape[0], n_out))
    base = MatmulArgs(
        act=_ptr(act), pre_quant_scale=None, weight=_ptr(weight), scales=_ptr(scales), zeros=_ptr(zeros),
        bias=_ptr(bias), out=_ptr(out), alpha=1.0, m=act.shape[0], n=n, k=k, group_size=group_size,
        quant_algo=quant_algo, act_dtype=_WOQ_DT[act.dtype], out_dtype=_WOQ_DT[act.dtype], regime=regime,
        workspace=None, workspace_bytes=0)
    experts = 1 if total_rows_before_expert is None else total_rows_before_expert.numel()
    args = GroupedMatmulArgs(base=base, total_rows_before_expert=_ptr(total_rows_before_expert), num_experts=experts,
                             activation=act_id, residual=_ptr(residual))
    check(lib.woq_grouped_matmul(ctypes.byref(args), _stream_handle(act.device)))
    return out


def weight_only_quant_matmul(input: torch.Tensor, weights: torch.Tensor, scales: torch.Tensor, weightTypeId: int,
                             dtype="float16", transa: bool = False, transb: bool = False) -> torch.Tensor:
    """Per-channel W8A16 / W4A16: input [.., K] x weights [K, N or N/2] (int8 storage, preprocessed),
    scales [N].  Mirrors functional.py:216-256 + weightOnlyQuantMatmulPlugin.cpp:283-339."""
    if transa or transb:
        raise RuntimeError("transa/transb are not supported by the weight-only matmul plugin path")
    if weightTypeId not in (INT8, INT4):
        raise RuntimeError("weightTypeId must be 1 (int8) or 2 (int4)")
    k = input.shape[-1]
    n = weights.shape[-1] * (2 if weightTypeId == INT4 else 1)  # `real_n`
    algo = INT8_WEIGHT if weightTypeId == INT8 else 0
    return woq_matmul_raw(input, None, weights, scales, None, None, n=n, k=k, group_size=0, quant_algo=algo,
                          out_dtype=_DTYPES[dtype])


def weight_only_groupwise_quant_matmul(input: torch.Tensor, pre_quant_scale, weights: torch.Tensor,
                                       scales: torch.Tensor, zeros, biases, alpha, quant_algo: int, group_size: int,
                                       dtype="float16") -> torch.Tensor:
    """Groupwise W4A16 / W8A16 / W4A8.  Mirrors functional.py:259-347 +
    weightOnlyGroupwiseQuantMatmulPlugin.cpp:407-495.  `weights` is the preprocessed tensor; the
    reference types it as the activation dtype ([K, N/4] halfs for int4, [K, N/2] for int8), a
    plain int8 [K, N/2] / [K, N] tensor is accepted as well."""
    out_dtype = _DTYPES[dtype]
    k = input.shape[-1]
    bits = 8 if quant_algo & INT8_WEIGHT else 4
    n = weights.shape[-1] * weights.element_size() * 8 // bits
    a = 1.0
    if quant_algo & FP8_ALPHA:
        a = float(alpha) if not hasattr(alpha, "raw_value") else float(alpha.raw_value[0])
    return woq_matmul_raw(
        input, pre_quant_scale if quant_algo & PRE_QUANT_SCALE else None, weights, scales,
        zeros if quant_algo & ZERO else None, biases if quant_algo & BIAS else None,
        n=n, k=k, group_size=group_size, quant_algo=quant_algo, alpha=a, out_dtype=out_dtype)


def apply_per_channel_scale(act: torch.Tensor, per_channel_scale: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """kernels/preQuantScaleKernel.cu:42-149: act * scale, optionally cast to fp8 e4m3."""
    _require_gpu(act, per_channel_scale)
    out_dtype = out_dtype or act.dtype
    k = act.shape[-1]
    out = torch.empty(act.shape, dtype=out_dtype, device=act.device)
    check(lib.woq_apply_per_channel_scale(_ptr(out), _ptr(act), _ptr(per_channel_scale), act.numel() // k, k,
                                          _WOQ_DT[act.dtype], _WOQ_DT[out_dtype], _stream_handle(act.device)))
    return out


def rmsnorm_prequant(x: torch.Tensor, gamma: torch.Tensor, pre_quant_scale=None, eps: float = 1e-6, beta=None,
                     out_dtype=None) -> torch.Tensor:
    """RMSNorm (kernels/rmsnormKernels.cu:29-124) fused with the smoothing pass
    (kernels/preQuantScaleKernel.cu:42-149): T_out(T(T(rmsnorm(x)) * pre_quant_scale)), T_out = x.dtype or
    fp8 e4m3.  `pre_quant_scale` and `beta` may be None."""
    _require_gpu(x, gamma, pre_quant_scale, beta)
    out_dtype = out_dtype or x.dtype
    k = x.shape[-1]
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    check(lib.woq_rmsnorm_prequant(_ptr(out), _ptr(x), _ptr(gamma), _ptr(beta), _ptr(pre_quant_scale), float(eps),
                                   x.numel() // k, k, _WOQ_DT[x.dtype], _WOQ_DT[out_dtype], _stream_handle(x.device)))
    return out


def dequantize_weights(weights: torch.Tensor, scales: torch.Tensor, zeros, *, k: int, n: int, group_size: int,
                       quant_type: int, dtype: torch.dtype) -> torch.Tensor:
    """W[k, n] = dtype(q * scale + zero) from preprocessed weights (woq_dequantize)."""
    _require_gpu(weights, scales, zeros)
    out = torch.empty((k, n), dtype=dtype, device=weights.device)
    check(lib.woq_dequantize(_ptr(out), _ptr(weights), _ptr(scales), _ptr(zeros), k, n, group_size, quant_type,
                             _WOQ_DT[dtype], _stream_handle(weights.device)))
    return out
