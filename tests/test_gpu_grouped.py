"""GPU parity of the grouped (mixture-of-experts) weight-only matmul against the oracle, through the
C ABI: expert e multiplies its rows with its own weights.  Same bar as the single-matrix kernels:
max|out - ref| / max|ref| <= 1e-2 against the float64-accumulated dequantize-then-matmul reference."""
import numpy as np
import pytest
import torch

from _util import TORCH_DT, preprocess, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-2
STREAM, GEMM = 1, 2


def grouped_problem(oracle, rows, K, N, bits, group, dtype, zero, bias, seed):
    rng = np.random.default_rng(seed)
    E, total = len(rows), int(sum(rows))
    lo = -(1 << (bits - 1))
    q = rng.integers(lo, -lo, size=(E, K, N)).astype(np.int8)
    gshape = (E, -(-K // group), N) if group else (E, N)  # a group size above 128 may leave a shorter last group
    p = dict(rows=rows, q=q, bits=bits, group=group, dtype=dtype, K=K, N=N,
             scales=oracle.round_to(rng.uniform(0.002, 0.02, gshape).astype(np.float32) * (16.0 / (1 << bits)), dtype),
             zeros=oracle.round_to((rng.standard_normal(gshape) * 0.02).astype(np.float32), dtype) if zero else None,
             bias=oracle.round_to(rng.standard_normal((E, N)).astype(np.float32), dtype) if bias else None,
             act=oracle.round_to(rng.standard_normal((total, K)).astype(np.float32), dtype),
             total=np.cumsum(np.asarray(rows, np.int64)))
    return p


def run_grouped(pkg, oracle, dev, p, regime=0, activation="identity", single=False, residual=None):
    F = pkg.functional
    dt = p["dtype"]
    w = torch.stack([preprocess(pkg, oracle, p["q"][e], p["bits"]) for e in range(len(p["rows"]))]).to(dev)
    algo = (F.INT8_WEIGHT if p["bits"] == 8 else 0) | (F.ZERO if p["zeros"] is not None else 0) \
        | (F.BIAS if p["bias"] is not None else 0)
    opt = lambda x: None if x is None else to_dev(x, dt, dev)
    total = None if single else torch.from_numpy(p["total"]).to(dev)
    # a recognisable fill: every row belongs to some expert and must be written
    n_out = p["N"] // 2 if activation in ("swiglu", "geglu") else p["N"]
    out = torch.full((p["act"].shape[0], n_out), float("nan"), dtype=TORCH_DT[dt], device=dev)
    F.woq_grouped_matmul_raw(to_dev(p["act"], dt, dev), w, to_dev(p["scales"], dt, dev), opt(p["zeros"]),
                             opt(p["bias"]), total, n=p["N"], k=p["K"], group_size=p["group"], quant_algo=algo,
                             activation=activation, residual=None if residual is None else to_dev(residual, dt, dev),
                             regime=regime, out=out)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def reference(oracle, p, activation="identity", residual=None):
    return oracle.grouped_matmul_ref(p["act"], p["q"], p["scales"], p["zeros"], p["bias"], p["total"], p["group"],
                                     p["dtype"], activation, residual)


@pytest.mark.parametrize("rows", [[3, 0, 16, 1], [40, 0, 5, 17], [0, 0, 7, 0], [1, 1, 1, 1, 1, 1, 1, 1]])
@pytest.mark.parametrize("bits,group,zero", [(4, 128, True), (4, 64, False), (8, 0, False)])
def test_grouped_decode_sizes_stream(pkg, oracle, dev, rows, bits, group, zero):
    """Few rows per expert (AUTO picks the streaming kernel): empty experts, one-row experts, and
    experts with more than 16 rows that take several passes."""
    p = grouped_problem(oracle, rows, 1024, 272, bits, group, "bf16", zero, True, seed=sum(rows) + bits)
    out = run_grouped(pkg, oracle, dev, p)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p)) < TOL


@pytest.mark.parametrize("rows", [[100, 0, 30, 70, 1], [64, 64, 64], [5, 129, 0, 63, 200]])
@pytest.mark.parametrize("bits,group,zero,dtype", [(4, 128, True, "bf16"), (4, 0, False, "fp16"), (8, 64, True, "bf16")])
def test_grouped_mid_sizes_tiles(pkg, oracle, dev, rows, bits, group, zero, dtype):
    """More than 16 rows per expert on average: 64-row tiles, a tile never spans two experts."""
    p = grouped_problem(oracle, rows, 512, 528, bits, group, dtype, zero, True, seed=sum(rows))
    out = run_grouped(pkg, oracle, dev, p)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p)) < TOL


def test_grouped_prefill_sizes(pkg, oracle, dev):
    """Hundreds of rows per expert: the exact-dequantize kernel with 256-row (or 128-row) tiles."""
    p = grouped_problem(oracle, [600, 300, 0, 700], 512, 512, 4, 128, "bf16", True, True, seed=9)
    out = run_grouped(pkg, oracle, dev, p)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p)) < TOL


@pytest.mark.parametrize("regime", [STREAM, GEMM])
@pytest.mark.parametrize("kernel", ["exact", "skinny"])
def test_grouped_forced_kernels_agree(pkg, oracle, dev, woq_env, regime, kernel):
    """The same problem on each kernel family, whatever AUTO would pick."""
    woq_env(WOQ_GEMM_KERNEL=kernel)
    p = grouped_problem(oracle, [20, 3, 0, 50, 33], 768, 272, 4, 128, "fp16", True, False, seed=12)
    out = run_grouped(pkg, oracle, dev, p, regime=regime)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p)) < TOL


def test_grouped_single_expert_equals_plain_matmul(pkg, oracle, dev):
    """One expert owning every row is the ordinary matmul: identical bits from the tiled kernels."""
    F = pkg.functional
    p = grouped_problem(oracle, [200], 512, 256, 4, 128, "bf16", True, True, seed=3)
    out = run_grouped(pkg, oracle, dev, p, regime=GEMM)
    w = preprocess(pkg, oracle, p["q"][0], 4).to(dev)
    plain = F.woq_matmul_raw(to_dev(p["act"], "bf16", dev), None, w, to_dev(p["scales"][0], "bf16", dev),
                             to_dev(p["zeros"][0], "bf16", dev), to_dev(p["bias"][0], "bf16", dev), n=256, k=512,
                             group_size=128, quant_algo=F.ZERO | F.BIAS, out_dtype=torch.bfloat16, regime=GEMM)
    torch.cuda.synchronize()
    # the plain call may split K (fewer tiles than CUs), the grouped one never does: same bar, not same bits
    assert oracle.max_rel_err(out, plain.float().cpu().numpy()) < 2e-3
    assert oracle.max_rel_err(out, reference(oracle, p)) < TOL


@pytest.mark.parametrize("activation", ["gelu", "relu", "silu", "swiglu", "geglu"])
@pytest.mark.parametrize("rows", [[3, 0, 16, 1], [40, 5], [90, 0, 70, 33]])
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_grouped_activations(pkg, oracle, dev, activation, rows, dtype):
    """moeGemmBiasAct's activations: fused into the streaming kernel's epilogue (few rows per expert,
    with strips paired for the gated ones) or applied by the activation pass behind the tiled
    kernels.  N = 544: a gated output of 272 columns, the last workgroup's strips only partly there."""
    p = grouped_problem(oracle, rows, 512, 544, 4, 128, dtype, True, True, seed=len(activation) + sum(rows))
    out = run_grouped(pkg, oracle, dev, p, activation=activation)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p, activation)) < TOL


@pytest.mark.parametrize("regime", [STREAM, GEMM])
@pytest.mark.parametrize("bits,group", [(8, 0), (4, 64)])
def test_grouped_swiglu_forced_regimes(pkg, oracle, dev, regime, bits, group):
    p = grouped_problem(oracle, [7, 20, 0, 9], 1024, 288, bits, group, "bf16", group != 0, True, seed=31)
    out = run_grouped(pkg, oracle, dev, p, regime=regime, activation="swiglu")
    assert oracle.max_rel_err(out, reference(oracle, p, "swiglu")) < TOL


@pytest.mark.parametrize("M", [1, 9, 300])
@pytest.mark.parametrize("activation", ["identity", "swiglu", "gelu"])
def test_single_expert_without_prefix_sums(pkg, oracle, dev, M, activation):
    """num_experts = 1 and no prefix sums: the plain matmul with a fused activation."""
    p = grouped_problem(oracle, [M], 512, 544, 4, 128, "bf16", True, True, seed=M)
    out = run_grouped(pkg, oracle, dev, p, activation=activation, single=True)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p, activation)) < TOL


@pytest.mark.parametrize("activation", ["identity", "swiglu", "gelu"])
@pytest.mark.parametrize("rows,single", [([9], True), ([300], True), ([700], True), ([3, 0, 16, 1], False),
                                         ([40, 5], False), ([90, 0, 70, 33], False), ([600, 300, 0, 700], False)])
def test_residual_is_added_after_the_activation(pkg, oracle, dev, activation, rows, single):
    """out = T(f(acc + bias) + residual) on every kernel: streaming, 64-row tiles, 256-row tiles, with
    the gated epilogue, and behind the separate activation pass."""
    p = grouped_problem(oracle, rows, 512, 288, 4, 128, "bf16", True, True, seed=sum(rows) + len(activation))
    n_out = 144 if activation == "swiglu" else 288
    rng = np.random.default_rng(77)
    residual = oracle.round_to(rng.standard_normal((sum(rows), n_out)).astype(np.float32) * 3.0, "bf16")
    out = run_grouped(pkg, oracle, dev, p, activation=activation, single=single, residual=residual)
    assert np.isfinite(out).all()
    assert oracle.max_rel_err(out, reference(oracle, p, activation, residual)) < TOL
    # and it is the residual that was added: the difference to a call without it is the residual itself
    plain = run_grouped(pkg, oracle, dev, p, activation=activation, single=single)
    assert np.abs((out - plain) - residual).max() <= 0.05 * np.abs(residual).max()


def test_grouped_rejections(pkg, oracle, dev):
    F = pkg.functional
    p = grouped_problem(oracle, [2, 2], 256, 64, 4, 128, "bf16", False, False, seed=1)
    w = torch.stack([preprocess(pkg, oracle, p["q"][e], 4) for e in range(2)]).to(dev)
    act, sc = to_dev(p["act"], "bf16", dev), to_dev(p["scales"], "bf16", dev)
    with pytest.raises(RuntimeError, match="int64"):
        F.woq_grouped_matmul_raw(act, w, sc, None, None, torch.tensor([2, 4], dtype=torch.int32, device=dev), n=64,
                                 k=256, group_size=128, quant_algo=0)
    with pytest.raises(RuntimeError, match="total_rows"):
        F.woq_grouped_matmul_raw(act.reshape(2, 2, 256), w, sc, None, None,
                                 torch.tensor([2, 4], dtype=torch.int64, device=dev), n=64, k=256, group_size=128,
                                 quant_algo=0)


@pytest.mark.parametrize("group,K", [(192, 1024), (256, 1024), (320, 768)])
@pytest.mark.parametrize("zero", [False, True])
@pytest.mark.parametrize("rows,regime", [([3, 0, 16, 1], STREAM), ([20, 3, 0, 50, 33], GEMM), ([300, 0, 270], GEMM)])
def test_grouped_flexible_group_sizes(pkg, oracle, dev, woq_env, group, K, zero, rows, regime):
    """Group sizes that are multiples of 64 above 128 through the grouped entry: every expert's table has
    ceil(k / group) rows (1024 / 192 and 768 / 320 leave a shorter last group), so the per-expert scale and
    zero offsets follow that row count.  Streaming passes, the deferred-scale and the exact-dequantize tiled
    kernels."""
    p = grouped_problem(oracle, rows, K, 272, 4, group, "bf16", zero, True, seed=group + sum(rows))
    ref = reference(oracle, p)
    for kernel in (("exact", "skinny") if regime == GEMM and sum(rows) < 200 else (None,)):
        woq_env(WOQ_GEMM_KERNEL=kernel)
        out = run_grouped(pkg, oracle, dev, p, regime=regime)
        assert np.isfinite(out).all()
        assert oracle.max_rel_err(out, ref) < TOL, kernel
