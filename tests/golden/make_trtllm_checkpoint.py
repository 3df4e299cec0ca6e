#!/usr/bin/env python3
"""Writes the tiny TensorRT-LLM checkpoints under tests/golden/trtllm_ckpt_*/ that pin
`checkpoint.load_trtllm_linear`.

    python tests/golden/make_trtllm_checkpoint.py

Each directory is a checkpoint as docs/source/architecture/checkpoint.md (of the reference) describes
it: `config.json` with a `quantization` section and `rank0.safetensors` with one linear layer under
the reference's tensor names (quantization/layers.py:744-751, 998-1037).  The `weight` tensor is in
the REFERENCE's preprocessed layout for the SM in the directory name, produced by the oracle's
restatement of preprocess_weights_for_mixed_gemm (`oracle/woq_oracle.py: ref_preprocess`; the
reference itself cannot be built or run here).  The row-major quantized weight the layout was made
from is stored next to it under `_expected.<layer>.q` for the byte-level check.  Seeded; running the
script again rewrites identical files."""
import json
import os
import sys

import numpy as np
import torch
from safetensors.torch import save_file

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, os.pardir, os.pardir, "oracle"))
import woq_oracle as o  # noqa: E402

CASES = [
    # directory, quant_algo, arch, layer, K, N, group, dtype, zeros, pre-quant scale, bias
    ("trtllm_ckpt_w4a16_awq_sm80", "W4A16_AWQ", 80, "transformer.layers.0.mlp.fc", 256, 128, 64, "float16", True, True, True),
    ("trtllm_ckpt_w4a16_gptq_sm90", "W4A16_GPTQ", 90, "transformer.layers.0.attention.qkv", 128, 192, 128, "bfloat16", True, False, False),
    ("trtllm_ckpt_w8a16_sm90", "W8A16", 90, "transformer.layers.0.attention.dense", 128, 64, 0, "float16", False, False, True),
    ("trtllm_ckpt_w4a16_sm80", "W4A16", 80, "transformer.layers.0.mlp.proj", 128, 128, 0, "bfloat16", False, False, False),
    ("trtllm_ckpt_w4a8_awq_sm89", "W4A8_AWQ", 89, "transformer.layers.0.mlp.gate", 256, 64, 128, "bfloat16", False, True, False),
]
TORCH = {"float16": torch.float16, "bfloat16": torch.bfloat16}
ORACLE = {"float16": "fp16", "bfloat16": "bf16"}


def t(x, dtype):
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(dtype).contiguous()


def main():
    for i, (name, algo, arch, layer, K, N, group, dtype, zero, pqs, bias) in enumerate(CASES):
        rng = np.random.default_rng(1000 + i)
        td, od = TORCH[dtype], ORACLE[dtype]
        bits = 8 if algo.startswith("W8") else 4
        w4a8 = algo == "W4A8_AWQ"
        q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
        qt = o.W8_A16 if bits == 8 else (o.W4_AFP8 if w4a8 else o.W4_A16)
        raw = o.ref_preprocess(q, qt, arch)  # int8 [K, N*bits/8], the reference's bytes
        tensors = {"_expected.%s.q" % layer: torch.from_numpy(q.copy())}
        w = torch.from_numpy(np.ascontiguousarray(raw).view(np.int8).reshape(K, N * bits // 8).copy())
        if group:
            w = w.view(td)  # groupwise layers declare the weight in the activation dtype
            gshape = (K // group, N)
            if w4a8:
                scales = o.round_f16(rng.uniform(0.5, 8.0, gshape).astype(np.float32))
                tensors[layer + ".weights_scaling_factor"] = t(scales, torch.float16).view(td)
                tensors[layer + ".alpha"] = torch.tensor([0.0123], dtype=torch.float32)
            else:
                scales = o.round_to(rng.uniform(0.002, 0.02, gshape).astype(np.float32), od)
                tensors[layer + ".weights_scaling_factor"] = t(scales, td)
            if zero:
                tensors[layer + ".zero"] = t(o.round_to((rng.standard_normal(gshape) * 0.02).astype(np.float32), od), td)
            if pqs:
                tensors[layer + ".prequant_scaling_factor"] = t(
                    o.round_to(rng.uniform(0.5, 2.0, (1, K)).astype(np.float32), od), td)
        else:
            tensors[layer + ".per_channel_scale"] = t(
                o.round_to(rng.uniform(0.002, 0.02, (N,)).astype(np.float32), od), td)
        tensors[layer + ".weight"] = w.contiguous()
        if bias:
            tensors[layer + ".bias"] = t(o.round_to(rng.standard_normal(N).astype(np.float32), od), td)
        out_dir = os.path.join(HERE, name)
        os.makedirs(out_dir, exist_ok=True)
        save_file(tensors, os.path.join(out_dir, "rank0.safetensors"))
        cfg = {"architecture": "LlamaForCausalLM", "dtype": dtype,
               "quantization": {"quant_algo": algo, "group_size": group or None, "has_zero_point": zero,
                                "pre_quant_scale": pqs},
               "mapping": {"world_size": 1, "tp_size": 1, "pp_size": 1},
               "_fixture": {"layer": layer, "sm_arch": arch, "k": K, "n": N}}
        with open(os.path.join(out_dir, "config.json"), "w") as f:
            json.dump(cfg, f, indent=1, sort_keys=True)
        print(name, sum(v.numel() * v.element_size() for v in tensors.values()), "bytes")


if __name__ == "__main__":
    main()
