"""The weight-preparation torch ops of the reference, served by libwoq's host code.

Same names, argument order, checks and return shapes as
cpp/tensorrt_llm/thop/weightOnlyQuantOp.cpp:123-363 (`torch.ops.trtllm.*`):

    symmetric_quantize_last_axis_of_batched_matrix(weight, quant_type) -> [processed, scales]
    _symmetric_quantize_last_axis_of_batched_matrix(weight, quant_type) -> [unprocessed, processed, scales]
    preprocess_weights_for_mixed_gemm(weight, quant_type, activation_type) -> processed
    unpack_int4_packed_tensor_to_int8(weight) / pack_int8_tensor_to_packed_int4(weight)

    _permute_B_rows_for_mixed_gemm(weight, quant_type, arch) / _subbyte_transpose(weight, quant_type)
    _add_bias_and_interleave_int4s(weight) / _add_bias_and_interleave_int8s(weight)
        (the reference's test-only operators, :65-120, :252-281: single steps of ITS preprocess)

plus two that have no counterpart there: `unprocess_weights_for_mixed_gemm` (inverse of the
gfx950 layout) and `import_reference_weights` (decode a buffer the REFERENCE preprocessed).

`processed` tensors are opaque: only this library's kernels can read them (the reference's are
SM-specific in the same way).  All tensors here are CPU tensors, as in the reference.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import lib, check

_TORCH_TO_WOQ = {torch.float16: _lib.FP16, torch.bfloat16: _lib.BF16, torch.float32: _lib.FP32}


def _check_cpu_contiguous(t: torch.Tensor, what: str = "weight") -> None:
    if t.device.type != "cpu":
        raise RuntimeError("%s must be a CPU tensor" % what)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % what)


def _quant_type(quant_type: torch.dtype, activation_type: torch.dtype = torch.float16) -> int:
    """get_ft_quant_type (thop/weightOnlyQuantOp.cpp:41-62)."""
    if quant_type not in (torch.int8, torch.quint4x2):
        raise RuntimeError("Must be int4 or int8 quantization")
    if activation_type == torch.float8_e4m3fn:
        return _lib.W4_AFP8
    return _lib.W8_A16 if quant_type == torch.int8 else _lib.W4_A16


def _bits(qt: int) -> int:
    return 8 if qt == _lib.W8_A16 else 4


def pack_int8_tensor_to_packed_int4(weight: torch.Tensor) -> torch.Tensor:
    _check_cpu_contiguous(weight)
    if weight.numel() == 0:
        raise RuntimeError("weight should not be empty tensor")
    if weight.dtype != torch.int8:
        raise RuntimeError("Weight must be a int8 tensor")
    if weight.shape[-1] % 2:
        raise RuntimeError("last dimension must be even")
    out = torch.zeros(weight.shape[:-1] + (weight.shape[-1] // 2,), dtype=torch.int8)
    check(lib.woq_pack_int4(out.data_ptr(), weight.data_ptr(), weight.numel()))
    return out


def unpack_int4_packed_tensor_to_int8(weight: torch.Tensor) -> torch.Tensor:
    _check_cpu_contiguous(weight)
    if weight.numel() == 0:
        raise RuntimeError("weight should not be empty tensor")
    if weight.dtype != torch.int8:
        raise RuntimeError("Weight must be a packed int8 tensor")
    out = torch.zeros(weight.shape[:-1] + (weight.shape[-1] * 2,), dtype=torch.int8)
    check(lib.woq_unpack_int4(out.data_ptr(), weight.data_ptr(), weight.numel()))
    return out


def _dims(weight: torch.Tensor, bits: int):
    if weight.dim() not in (2, 3):
        raise RuntimeError("Invalid dim. The dim of weight should be 2 or 3")
    experts = 1 if weight.dim() == 2 else weight.shape[0]
    return experts, weight.shape[-2], weight.shape[-1] * (8 // bits)


def preprocess_weights_for_mixed_gemm(row_major_quantized_weight: torch.Tensor, quant_type: torch.dtype,
                                      activation_type: torch.dtype = torch.float16) -> torch.Tensor:
    """[K, N*bits/8] (or [E, K, N*bits/8]) int8, row-major signed, int4 packed along N ->
    same-size opaque int8 tensor in the gfx950 tile layout.  (Only when K is not a multiple of
    128 for int4 / 64 for int8 does the row count grow, to the next such multiple.)"""
    w = row_major_quantized_weight
    _check_cpu_contiguous(w)
    if w.dtype != torch.int8:
        raise RuntimeError("Quantized tensor must be int8 dtype")
    qt = _quant_type(quant_type, activation_type)
    experts, k, n = _dims(w, _bits(qt))
    per_matrix = lib.woq_preprocessed_bytes(k, n, qt)
    rows = per_matrix // w.shape[-1]
    out = torch.zeros(w.shape[:-2] + (rows, w.shape[-1]), dtype=torch.int8)
    check(lib.woq_preprocess_weights(out.data_ptr(), w.data_ptr(), experts, k, n, qt))
    return out


def unprocess_weights_for_mixed_gemm(processed: torch.Tensor, k: int, quant_type: torch.dtype,
                                     activation_type: torch.dtype = torch.float16) -> torch.Tensor:
    """Inverse of preprocess_weights_for_mixed_gemm: back to row-major [.., k, N*bits/8]."""
    _check_cpu_contiguous(processed)
    qt = _quant_type(quant_type, activation_type)
    experts = 1 if processed.dim() == 2 else processed.shape[0]
    n = processed.shape[-1] * (8 // _bits(qt))
    out = torch.zeros(processed.shape[:-2] + (k, processed.shape[-1]), dtype=torch.int8)
    check(lib.woq_unpreprocess_weights(out.data_ptr(), processed.data_ptr(), experts, k, n, qt))
    return out


def import_reference_weights(reference_processed: torch.Tensor, quant_type: torch.dtype,
                             activation_type: torch.dtype = torch.float16, arch: int = 80) -> torch.Tensor:
    """Decodes weights laid out by the reference's preprocess for SM `arch` to row-major signed."""
    w = reference_processed
    _check_cpu_contiguous(w)
    if w.dtype != torch.int8:
        raise RuntimeError("Quantized tensor must be int8 dtype")
    qt = _quant_type(quant_type, activation_type)
    experts, k, n = _dims(w, _bits(qt))
    out = torch.zeros_like(w)
    check(lib.woq_import_reference_weights(out.data_ptr(), w.data_ptr(), experts, k, n, qt, arch))
    return out


def _reference_step(weight: torch.Tensor, qt: int, step: int) -> torch.Tensor:
    _check_cpu_contiguous(weight, "Quantized tensor")
    if weight.dtype != torch.int8:
        raise RuntimeError("Quantized tensor must be int8 dtype")
    experts, k, n = _dims(weight, _bits(qt))
    out = torch.empty_like(weight)
    check(lib.woq_reference_layout_step(out.data_ptr(), weight.data_ptr(), experts, k, n, qt, step))
    return out


def _permute_B_rows_for_mixed_gemm(quantized_tensor: torch.Tensor, quant_type: torch.dtype,
                                   arch_version: int) -> torch.Tensor:
    """Row permutation of the reference's preprocess (blocks of 16 int8 / 32 int4 rows) on packed
    row-major weights; `arch_version` is accepted and, as in the reference's function, not consulted."""
    return _reference_step(quantized_tensor, _quant_type(quant_type), 0)


def _subbyte_transpose(quantized_tensor: torch.Tensor, quant_type: torch.dtype) -> torch.Tensor:
    """Element-granular transpose of packed weights: the result has the input's tensor shape (as in the
    reference) and holds [n][k] elements."""
    return _reference_step(quantized_tensor, _quant_type(quant_type), 1)


def _add_bias_and_interleave(weight: torch.Tensor, qt: int) -> torch.Tensor:
    _check_cpu_contiguous(weight)
    if weight.numel() == 0:
        raise RuntimeError("weight should not be empty tensor")
    if weight.dtype != torch.int8:
        raise RuntimeError("Weight must be a packed int8 tensor" if qt == _lib.W4_A16 else "Weight must be an int8 tensor")
    out = torch.empty_like(weight)
    elts = weight.numel() * (8 // _bits(qt))
    check(lib.woq_reference_layout_step(out.data_ptr(), weight.data_ptr(), 1, 1, elts, qt, 2))
    return out


def _add_bias_and_interleave_int4s(weight: torch.Tensor) -> torch.Tensor:
    return _add_bias_and_interleave(weight, _lib.W4_A16)


def _add_bias_and_interleave_int8s(weight: torch.Tensor) -> torch.Tensor:
    return _add_bias_and_interleave(weight, _lib.W8_A16)


def _symmetric_quantize_helper(weight: torch.Tensor, quant_type: torch.dtype, return_unprocessed: bool):
    _check_cpu_contiguous(weight)
    if weight.numel() == 0:
        raise RuntimeError("weight should not be empty tensor")
    if weight.dim() not in (2, 3):
        raise RuntimeError("Invalid dim. The dim of weight should be 2 or 3")
    if weight.dtype not in _TORCH_TO_WOQ:
        raise RuntimeError("Invalid datatype. Weight must be FP16 or BF16")
    qt = _quant_type(quant_type)
    bits = _bits(qt)
    experts = 1 if weight.dim() == 2 else weight.shape[0]
    k, n = weight.shape[-2], weight.shape[-1]
    qshape = weight.shape[:-1] + (n * bits // 8,)
    unprocessed = torch.empty(qshape, dtype=torch.int8)
    per_matrix = lib.woq_preprocessed_bytes(k, n, qt)
    processed = torch.zeros(weight.shape[:-2] + (per_matrix // qshape[-1], qshape[-1]), dtype=torch.int8)
    scales = torch.empty(weight.shape[:-2] + (n,), dtype=weight.dtype)
    dt = _TORCH_TO_WOQ[weight.dtype]
    check(lib.woq_symmetric_quantize(processed.data_ptr(), unprocessed.data_ptr(), scales.data_ptr(),
                                     weight.data_ptr(), experts, k, n, qt, dt, dt))
    if return_unprocessed:
        return [unprocessed, processed, scales]
    return [processed, scales]


def symmetric_quantize_last_axis_of_batched_matrix(weight: torch.Tensor, quant_type: torch.dtype):
    return _symmetric_quantize_helper(weight, quant_type, False)


def _symmetric_quantize_last_axis_of_batched_matrix(weight: torch.Tensor, quant_type: torch.dtype):
    return _symmetric_quantize_helper(weight, quant_type, True)


def _register_torch_ops() -> None:
    """Registers the ops as torch.ops.trtllm.* so that code written against the reference (its
    conversion scripts and tests call them by these names) finds them.  A failure here is an error:
    the promise that such code runs unchanged would otherwise break silently."""
    defs = {
        "symmetric_quantize_last_axis_of_batched_matrix":
            ("(Tensor weight, ScalarType quant_type) -> Tensor[]", symmetric_quantize_last_axis_of_batched_matrix),
        "_symmetric_quantize_last_axis_of_batched_matrix":
            ("(Tensor weight, ScalarType quant_type) -> Tensor[]", _symmetric_quantize_last_axis_of_batched_matrix),
        "preprocess_weights_for_mixed_gemm":
            ("(Tensor weight, ScalarType quant_type, ScalarType activation_type) -> Tensor",
             preprocess_weights_for_mixed_gemm),
        "unpack_int4_packed_tensor_to_int8": ("(Tensor weight) -> Tensor", unpack_int4_packed_tensor_to_int8),
        "pack_int8_tensor_to_packed_int4": ("(Tensor weight) -> Tensor", pack_int8_tensor_to_packed_int4),
        "_permute_B_rows_for_mixed_gemm":
            ("(Tensor quantized_tensor, ScalarType quant_type, int arch_version) -> Tensor", _permute_B_rows_for_mixed_gemm),
        "_subbyte_transpose": ("(Tensor quantized_tensor, ScalarType quant_type) -> Tensor", _subbyte_transpose),
        "_add_bias_and_interleave_int4s": ("(Tensor weight) -> Tensor", _add_bias_and_interleave_int4s),
        "_add_bias_and_interleave_int8s": ("(Tensor weight) -> Tensor", _add_bias_and_interleave_int8s),
    }
    for name, (schema, fn) in defs.items():
        qual = "trtllm::" + name
        if hasattr(torch.ops.trtllm, name):  # this module imported twice in one process
            continue
        torch.library.define(qual, schema)
        torch.library.impl(qual, "CPU")(fn)


REGISTERED_TORCH_OPS = ("symmetric_quantize_last_axis_of_batched_matrix", "_symmetric_quantize_last_axis_of_batched_matrix",
                        "preprocess_weights_for_mixed_gemm", "unpack_int4_packed_tensor_to_int8",
                        "pack_int8_tensor_to_packed_int4", "_permute_B_rows_for_mixed_gemm", "_subbyte_transpose",
                        "_add_bias_and_interleave_int4s", "_add_bias_and_interleave_int8s")

_register_torch_ops()
