"""Calls on two streams at once: the library keeps no device state between or across calls of woq_matmul
(partial sums and smoothed activations live in the caller's workspace), so launches that overlap on the GPU,
each with a workspace of its own, return the bits they return alone.  (woq_matmul_static is the exception by
design - one scratch array per GPU - and is tested in test_zz_no_alloc.py.)"""
import numpy as np
import pytest
import torch

from _util import TORCH_DT, parity_err, preprocess, random_problem, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-2
GEMM = 2


def _operands(pkg, oracle, dev, p):
    F = pkg.functional
    dt = p["dtype"]
    opt = lambda x: None if x is None else to_dev(x, dt, dev)
    algo = (F.INT8_WEIGHT if p["bits"] == 8 else 0) | (F.ZERO if p["zeros"] is not None else 0) \
        | (F.BIAS if p["bias"] is not None else 0) | (F.PRE_QUANT_SCALE if p["pqs"] is not None else 0)
    need = pkg._lib.lib.woq_workspace_bytes(p["M"], p["N"], p["K"], algo, pkg._lib.BF16 if dt == "bf16" else pkg._lib.FP16)
    return dict(act=to_dev(p["act"], dt, dev), pqs=opt(p["pqs"]), w=preprocess(pkg, oracle, p["q"], p["bits"]).to(dev),
                scales=to_dev(p["scales"], dt, dev), zeros=opt(p["zeros"]), bias=opt(p["bias"]), algo=algo,
                ws=torch.full((max(int(need), 256),), 0x5A, dtype=torch.uint8, device=dev),
                out=torch.empty((p["M"], p["N"]), dtype=TORCH_DT[dt], device=dev))


def _call(pkg, p, o, regime):
    pkg.functional.woq_matmul_raw(o["act"], o["pqs"], o["w"], o["scales"], o["zeros"], o["bias"], n=p["N"], k=p["K"],
                                  group_size=p["group"], quant_algo=o["algo"], out_dtype=o["out"].dtype, regime=regime,
                                  workspace=o["ws"], out=o["out"])


def test_two_streams_with_their_own_workspaces(pkg, oracle, dev):
    """A split-K GEMM with a smoothing pass, a multi-row decode call, a one-row decode call and a second split-K
    GEMM, issued in alternation on two streams for many rounds: every output equals the one the same call
    produced alone, bit for bit, and meets the parity bar."""
    cases = [(random_problem(oracle, 48, 4096, 512, 4, 128, "bf16", zero=True, bias=True, pqs=True, seed=1), GEMM),
             (random_problem(oracle, 8, 4096, 4096, 4, 128, "bf16", zero=True, seed=2), 0),
             (random_problem(oracle, 1, 4096, 272, 4, 64, "fp16", zero=True, bias=True, seed=3), 0),
             (random_problem(oracle, 96, 2048, 784, 8, 0, "fp16", bias=True, seed=4), GEMM)]
    ops = [_operands(pkg, oracle, dev, p) for p, _ in cases]
    alone = []
    for (p, regime), o in zip(cases, ops):
        _call(pkg, p, o, regime)
        torch.cuda.synchronize()
        alone.append(o["out"].clone())
        assert parity_err(oracle, alone[-1].float().cpu().numpy(), p) < TOL
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream(dev))
    for _ in range(25):
        # stream 0 runs cases 0, 1 while stream 1 runs cases 2, 3; then the pairs swap streams
        for first in (0, 1):
            for si, s in enumerate(streams):
                with torch.cuda.stream(s):
                    for ci in ((0, 1) if si == first else (2, 3)):
                        ops[ci]["out"].zero_()
                        _call(pkg, cases[ci][0], ops[ci], cases[ci][1])
            # a case must not run on both streams at once (one workspace, one output): join before the swap
            for s in streams:
                s.synchronize()
            for ci in range(4):
                assert torch.equal(ops[ci]["out"], alone[ci]), ci
