"""MI355X-native weight-only quantized matmul (the computation behind TensorRT-LLM's
WeightOnlyQuantMatmulPlugin / WeightOnlyGroupwiseQuantMatmulPlugin).

The package is a thin Python mirror of the reference's interface over `libwoq.so` (HIP kernels
behind a C ABI, see include/woq.h):

  ops         the `torch.ops.trtllm.*` weight-preparation ops (also registered under that name)
  functional  weight_only_quant_matmul / weight_only_groupwise_quant_matmul
  plugin      WeightOnlyQuantMatmulPlugin / WeightOnlyGroupwiseQuantMatmulPlugin (enqueue semantics)
  checkpoint  GPTQ / AutoAWQ tensors -> the groupwise op's operands (postprocess_weight_only_groupwise)

There is no CPU or PyTorch fallback for the matmul: if libwoq.so is missing, importing fails.
"""
from . import _lib, ops, functional, plugin, checkpoint  # noqa: F401
from ._lib import WoqError, lib_path  # noqa: F401

__all__ = ["ops", "functional", "plugin", "checkpoint", "WoqError", "lib_path"]
