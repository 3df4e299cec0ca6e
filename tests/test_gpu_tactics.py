"""Tactic profiler on the GPU: after profiling a layer the tuned choices (a kernel and launch shape,
or "heuristic" where nothing was clearly faster than the built-in choice) are in force for regime
AUTO and the results still match the oracle (same tolerance as the kernels' own parity tests);
an imported entry this build has no kernel for falls back to the heuristics."""
import pytest
import torch

from _util import parity_err, random_problem, reference, run_product, preprocess, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(autouse=True)
def _clean(pkg):
    pkg.functional.clear_tactics()
    yield
    pkg.functional.clear_tactics()


@pytest.mark.parametrize("bits,group,dtype", [(4, 128, "bf16"), (8, 0, "fp16")])
def test_profile_then_matmul(pkg, oracle, dev, bits, group, dtype):
    F = pkg.functional
    K, N, max_m = 1024, 2048, 192
    tdt = {"bf16": torch.bfloat16, "fp16": torch.float16}[dtype]
    p = random_problem(oracle, max_m, K, N, bits, group, dtype, zero=group != 0, seed=11)
    w = preprocess(pkg, oracle, p["q"], bits).to(dev)
    algo = (F.INT8_WEIGHT if bits == 8 else 0) | (F.ZERO if group else 0)
    zeros = to_dev(p["zeros"], dtype, dev) if group else None
    n = F.profile_tactics(None, w, to_dev(p["scales"], dtype, dev), zeros, None, n=N, k=K, group_size=group,
                          quant_algo=algo, dtype=tdt, min_m=1, max_m=max_m)
    # 1..15, 16, 32, 64, 128 and max_m
    assert n == 15 + 4 + 1
    text = F.export_tactics()
    for m in (1, 5, 16, 40, 100, max_m):
        assert F.describe_tactic(m, N, K, group, algo, tdt).split()[0] in ("heuristic", "stream", "gemm")
        q = dict(p, act=p["act"][:m], M=m)
        err = parity_err(oracle, run_product(pkg, oracle, dev, q, 0, w_dev=w), q)
        assert err < TOL, (m, F.describe_tactic(m, N, K, group, algo, tdt), err)
    assert F.describe_tactic(max_m + 1, N, K, group, algo, tdt) == "heuristic"
    # the exported text brings the same table back
    F.clear_tactics()
    F.import_tactics(text)
    assert F.export_tactics() == text


def test_unknown_shape_falls_back(pkg, oracle, dev):
    F = pkg.functional
    K, N, m = 512, 256, 4
    p = random_problem(oracle, m, K, N, 4, 128, "bf16", zero=True, seed=5)
    dt = F._WOQ_DT[torch.bfloat16]
    # a streaming launch shape that passes the range checks but is not instantiated
    F.import_tactics("woq-tactics 1\n%d %d %d 128 %d %d 1 1 3 5 7 0 0 0 0\n" % (N, K, F.ZERO, dt, m))
    assert F.describe_tactic(m, N, K, 128, F.ZERO, torch.bfloat16).startswith("stream")
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, 0), p)
    assert err < TOL, err


def test_plugin_initialize_profiles_the_layer(pkg, oracle, dev):
    """The plugin mirrors' initialize (configurePlugin dimensions + profiling on stand-in buffers):
    afterwards the real layer's calls go by the tuned table and match the oracle."""
    F, P = pkg.functional, pkg.plugin
    K, N, max_m = 512, 1024, 48
    plug = P.WeightOnlyGroupwiseQuantMatmulPlugin(torch.bfloat16, F.ZERO, 64)
    assert plug.initialize(1, max_m, N, K, device=dev) == 15 + 2 + 1
    assert "woq-tactics 1" in F.export_tactics()
    for m in (2, 20, max_m):
        p = random_problem(oracle, m, K, N, 4, 64, "bf16", zero=True, seed=m)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, 0), p)
        assert err < TOL, (m, err)
    per_channel = P.WeightOnlyQuantMatmulPlugin(torch.float16, F.INT8)
    assert per_channel.initialize(4, 4, N, K, device=dev) == 18 + 1
    assert per_channel.get_workspace_size(4, N, K) >= 0
