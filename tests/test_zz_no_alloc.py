"""woq_matmul_static, the entry point that allocates nothing: called through the C ABI on problems
whose kernels use scratch memory (split-K partial sums, smoothed activations, the W4A8 smoothing
pass), it must return what woq_matmul returns with a caller workspace, bit for bit - on two calls in
a row, the second with a smaller input (the static scratch keeps the first call's contents), and
reject a call whose scratch would not fit."""
import ctypes

import pytest
import torch

from _util import random_problem, preprocess, to_dev, TORCH_DT

pytestmark = pytest.mark.gpu


def _operands(pkg, oracle, dev, M, K, N, bits, group, dtype, seed, pqs):
    p = random_problem(oracle, M, K, N, bits, group, dtype, zero=group != 0, bias=True, pqs=pqs, seed=seed)
    F = pkg.functional
    algo = (F.INT8_WEIGHT if bits == 8 else 0) | (F.ZERO if group else 0) | F.BIAS | (F.PRE_QUANT_SCALE if pqs else 0)
    opt = lambda x: None if x is None else to_dev(x, dtype, dev)
    return dict(act=to_dev(p["act"], dtype, dev), pqs=opt(p["pqs"]), w=preprocess(pkg, oracle, p["q"], bits).to(dev),
                scales=to_dev(p["scales"], dtype, dev), zeros=opt(p["zeros"]), bias=opt(p["bias"]), algo=algo,
                n=N, k=K, group=group, dtype=TORCH_DT[dtype])


def _call(pkg, o, static, regime):
    out = torch.full((o["act"].shape[0], o["n"]), float("nan"), dtype=o["dtype"], device=o["act"].device)
    pkg.functional.woq_matmul_raw(o["act"], o["pqs"], o["w"], o["scales"], o["zeros"], o["bias"], n=o["n"], k=o["k"],
                                  group_size=o["group"], quant_algo=o["algo"], out_dtype=o["dtype"], regime=regime,
                                  out=out, static_scratch=static)
    torch.cuda.synchronize()
    return out


GEMM = 2


@pytest.mark.parametrize("bits,group,dtype,pqs", [(4, 128, "bf16", True), (4, 64, "fp16", False), (8, 0, "bf16", True)])
def test_static_scratch_matches_caller_workspace_twice(pkg, oracle, dev, bits, group, dtype, pqs):
    """GEMM regime on skinny problems with long K: the plan splits K (float32 slabs in the scratch)
    and, with a smoothing vector, the smoothed activations sit in front of them."""
    lib = pkg._lib.lib
    big = _operands(pkg, oracle, dev, 96, 4096, 512, bits, group, dtype, 1, pqs)
    small = _operands(pkg, oracle, dev, 40, 2048, 256, bits, group, dtype, 2, pqs)
    for o in (big, small):  # two calls in a row on the same scratch, the second smaller
        m = o["act"].shape[0]
        assert lib.woq_workspace_bytes(m, o["n"], o["k"], o["algo"], pkg._lib.BF16) > 0  # scratch is in use
        want = _call(pkg, o, False, GEMM)
        got = _call(pkg, o, True, GEMM)
        assert not torch.isnan(want.float()).any()
        assert torch.equal(got, want)
    # and the first problem again after the smaller one overwrote part of the scratch
    assert torch.equal(_call(pkg, big, True, GEMM), _call(pkg, big, False, GEMM))


def test_static_scratch_w4a8_and_auto_regime(pkg, oracle, dev):
    """W4A8 with 16-bit activations: the smoothing pass writes e4m3 activations to the scratch in both
    regimes (16 rows stream, 200 rows run the fp8 GEMM with a K split)."""
    F = pkg.functional
    for M, K, N in ((200, 2048, 512), (16, 1024, 384)):
        prob = oracle.make_w4a8_problem(M, K, N, seed=M, out_dtype="bf16")
        w = preprocess(pkg, oracle, prob["q"], 4, torch.float8_e4m3fn).to(dev)
        args = dict(n=N, k=K, group_size=128, quant_algo=F.FP8_ALPHA | F.PRE_QUANT_SCALE, alpha=prob["alpha"],
                    out_dtype=torch.bfloat16)
        ops = (to_dev(prob["act"], "bf16", dev), to_dev(prob["pre_quant_scale"], "bf16", dev), w,
               to_dev(prob["scales"], "fp16", dev), None, None)
        want = F.woq_matmul_raw(*ops, **args)
        got = F.woq_matmul_raw(*ops, static_scratch=True, **args)
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_static_scratch_rejects_what_does_not_fit(pkg, dev):
    """A smoothing buffer beyond the static scratch: a clear error, nothing launched (the check needs
    no valid device memory, only non-null pointers)."""
    lib, L = pkg._lib.lib, pkg._lib
    m, k, n = 8192, 8192, 4096  # smoothed activations alone: 128 MiB
    assert m * k * 2 > lib.woq_static_scratch_bytes()
    one = ctypes.c_void_p(256)
    args = L.MatmulArgs(act=one, pre_quant_scale=one, weight=one, scales=one, zeros=None, bias=None, out=one, alpha=1.0,
                        m=m, n=n, k=k, group_size=128, quant_algo=L.ALGO_PRE_QUANT_SCALE, act_dtype=L.BF16,
                        out_dtype=L.BF16, regime=L.REGIME_GEMM, workspace=None, workspace_bytes=0)
    assert lib.woq_matmul_static(ctypes.byref(args), None) == -4  # WOQ_ERR_WORKSPACE
    assert b"static scratch" in lib.woq_last_error()


def test_static_scratch_allocates_nothing_and_replays_from_a_graph(pkg, oracle, dev):
    """After woq_static_init() and one call outside capture, a static call with `out=` given leaves the
    device's free memory where it was, and the same call captured into a HIP graph replays to the eager
    bits every time (eager work of the library between the replays; the input changes between them)."""
    assert pkg._lib.lib.woq_static_init() == 0
    assert pkg._lib.lib.woq_static_init() == 0  # idempotent
    o = _operands(pkg, oracle, dev, 96, 4096, 512, 4, 128, "bf16", 5, True)
    other = _operands(pkg, oracle, dev, 40, 2048, 256, 4, 128, "bf16", 6, True)
    F = pkg.functional
    out = torch.empty((96, o["n"]), dtype=o["dtype"], device=dev)

    def static_call():
        F.woq_matmul_raw(o["act"], o["pqs"], o["w"], o["scales"], o["zeros"], o["bias"], n=o["n"], k=o["k"],
                         group_size=o["group"], quant_algo=o["algo"], out_dtype=o["dtype"], regime=GEMM, out=out,
                         static_scratch=True)

    static_call()  # first use of this kernel variant: outside capture
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    for _ in range(3):
        static_call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            static_call()
    torch.cuda.current_stream(dev).wait_stream(side)
    acts = [o["act"].clone(), (o["act"] * 0.5).contiguous(), o["act"].flip(0).contiguous()]
    for a in acts:
        o["act"].copy_(a)
        want = _call(pkg, o, False, GEMM)
        _call(pkg, other, True, GEMM)  # eager work on the same scratch between the replays
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
