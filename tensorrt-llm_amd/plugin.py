"""Plugin-shaped wrappers: the state and `enqueue` contract of the reference's two TensorRT
plugins, without TensorRT.

  WeightOnlyQuantMatmulPlugin          cpp/tensorrt_llm/plugins/weightOnlyQuantMatmulPlugin/weightOnlyQuantMatmulPlugin.{h,cpp}
  WeightOnlyGroupwiseQuantMatmulPlugin cpp/tensorrt_llm/plugins/weightOnlyGroupwiseQuantMatmulPlugin/weightOnlyGroupwiseQuantMatmulPlugin.{h,cpp}

Fields are the plugin fields (`type_id`, `weight_type_id` / `type_id`, `quant_algo`, `group_size`,
`alpha`); `enqueue(inputs, outputs, workspace)` takes the inputs in the plugins' order and returns 0.
"""
from __future__ import annotations

import torch

from . import functional as F
from ._lib import lib
from . import _lib

PLUGIN_NAMESPACE = "tensorrt_llm"
PLUGIN_VERSION = "1"


def _profile_layer(n: int, k: int, group_size: int, quant_algo: int, dtype: torch.dtype, min_m: int, max_m: int,
                   alpha: float, device) -> int:
    """Tactic profiling of one layer shape on stand-in operands, as the reference's profiler does on
    its own temporary buffers (gemmPluginProfiler.cpp:252-270, called from the plugins' initialize
    through configGemm, weightOnlyQuantMatmulPlugin.cpp:255-275): kernel times do not depend on the
    values, so random packed weights and unit scales stand in for the layer's."""
    nbytes = int(lib.woq_preprocessed_bytes(k, n, _lib.W8_A16 if quant_algo & F.INT8_WEIGHT else _lib.W4_A16))
    weight = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=device)
    groups = (k // group_size, n) if group_size else (n,)
    scales = torch.full(groups, 0.01, dtype=dtype, device=device)
    zeros = torch.zeros(groups, dtype=dtype, device=device) if quant_algo & F.ZERO else None
    bias = torch.zeros((n,), dtype=dtype, device=device) if quant_algo & F.BIAS else None
    pqs = torch.ones((k,), dtype=dtype, device=device) if quant_algo & F.PRE_QUANT_SCALE else None
    return F.profile_tactics(pqs, weight, scales, zeros, bias, n=n, k=k, group_size=group_size,
                             quant_algo=quant_algo, dtype=dtype, min_m=min_m, max_m=max_m, alpha=alpha)


class WeightOnlyQuantMatmulPlugin:
    name = "WeightOnlyQuantMatmul"

    def __init__(self, type_id: torch.dtype, weight_type_id: int):
        if type_id not in (torch.float16, torch.bfloat16):
            raise RuntimeError("No valid weightOnlyQuantMatmul configuration")
        if weight_type_id not in (F.INT8, F.INT4):
            raise RuntimeError("weight_type_id must be 1 (INT8) or 2 (INT4)")
        self.type_id = type_id
        self.weight_type_id = weight_type_id

    def get_workspace_size(self, max_m: int, n: int, k: int) -> int:
        dt = _lib.BF16 if self.type_id == torch.bfloat16 else _lib.FP16
        algo = F.INT8_WEIGHT if self.weight_type_id == F.INT8 else 0
        return int(lib.woq_workspace_bytes(max_m, n, k, algo, dt))

    def initialize(self, min_m: int, max_m: int, n: int, k: int, device="cuda") -> int:
        """configurePlugin's dimensions + initialize's profiling in one call
        (weightOnlyQuantMatmulPlugin.cpp:233-275).  Returns the number of tuned entries; the table
        travels as text (functional.export_tactics / import_tactics), the counterpart of the tactic
        map the reference serialises with the plugin (:374-391)."""
        algo = F.INT8_WEIGHT if self.weight_type_id == F.INT8 else 0
        return _profile_layer(n, k, 0, algo, self.type_id, min_m, max_m, 1.0, device)

    def enqueue(self, inputs, outputs, workspace=None) -> int:
        """inputs: [act [.., K], weight [K, N or N/2], scales [N]]; outputs: [out [.., N]]."""
        act, weight, scales = inputs
        k = act.shape[-1]
        n = weight.shape[-1] * (2 if self.weight_type_id == F.INT4 else 1)
        algo = F.INT8_WEIGHT if self.weight_type_id == F.INT8 else 0
        F.woq_matmul_raw(act, None, weight, scales, None, None, n=n, k=k, group_size=0, quant_algo=algo,
                         out_dtype=self.type_id, out=outputs[0], workspace=workspace)
        return 0


class WeightOnlyGroupwiseQuantMatmulPlugin:
    name = "WeightOnlyGroupwiseQuantMatmul"

    def __init__(self, type_id: torch.dtype, quant_algo: int, group_size: int, alpha: float = 1.0):
        if type_id not in (torch.float16, torch.bfloat16):
            raise RuntimeError("Unsupported data type")
        self.type_id, self.quant_algo, self.group_size, self.alpha = type_id, quant_algo, group_size, alpha

    def get_workspace_size(self, max_m: int, n: int, k: int) -> int:
        dt = _lib.BF16 if self.type_id == torch.bfloat16 else _lib.FP16
        return int(lib.woq_workspace_bytes(max_m, n, k, self.quant_algo, dt))

    def initialize(self, min_m: int, max_m: int, n: int, k: int, device="cuda") -> int:
        """Profiles the layer shape for row counts min_m..max_m
        (weightOnlyGroupwiseQuantMatmulPlugin.cpp: configurePlugin + initialize → configGemm →
        profileTactics).  Returns the number of tuned entries."""
        return _profile_layer(n, k, self.group_size, self.quant_algo, self.type_id, min_m, max_m, self.alpha, device)

    def enqueue(self, inputs, outputs, workspace=None) -> int:
        """inputs in plugin order: act, [pre_quant_scale], weight, scales, [zeros], [bias]."""
        it = iter(inputs)
        act = next(it)
        pqs = next(it) if self.quant_algo & F.PRE_QUANT_SCALE else None
        weight = next(it)
        scales = next(it)
        zeros = next(it) if self.quant_algo & F.ZERO else None
        bias = next(it) if self.quant_algo & F.BIAS else None
        bits = 8 if self.quant_algo & F.INT8_WEIGHT else 4
        n = weight.shape[-1] * weight.element_size() * 8 // bits
        F.woq_matmul_raw(act, pqs, weight, scales, zeros, bias, n=n, k=act.shape[-1], group_size=self.group_size,
                         quant_algo=self.quant_algo, alpha=self.alpha, out_dtype=self.type_id, out=outputs[0],
                         workspace=workspace)
        return 0
