"""Shared helpers of the GPU parity tests: build one seeded problem with the oracle, move it to
the GPU in the library's formats, run the product through the C ABI wrappers."""
import numpy as np
import torch

TORCH_DT = {"bf16": torch.bfloat16, "fp16": torch.float16}


def to_dev(x, dtype, dev):
    """float32 numpy values (already representable in `dtype`) -> device tensor of that dtype."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(TORCH_DT[dtype]).to(dev)


def random_problem(oracle, M, K, N, bits, group, dtype, zero=False, bias=False, pqs=False, seed=0):
    """Random integer weights, scales ~ U, zeros ~ N, as the reference's op tests do
    (tests/quantization/test_weight_only_groupwise_quant_matmul.py:185-200)."""
    rng = np.random.default_rng(seed)
    lo = -(1 << (bits - 1))
    q = rng.integers(lo, -lo, size=(K, N)).astype(np.int8)
    gshape = (-(-K // group), N) if group else (N,)  # a group size above 128 may leave a shorter last group
    scales = oracle.round_to(rng.uniform(0.002, 0.02, gshape).astype(np.float32) * (16.0 / (1 << bits)), dtype)
    p = dict(q=q, scales=scales, zeros=None, bias=None, pqs=None, bits=bits, group=group, dtype=dtype, M=M, K=K, N=N)
    if zero:
        p["zeros"] = oracle.round_to((rng.standard_normal(gshape) * 0.02).astype(np.float32), dtype)
    if bias:
        p["bias"] = oracle.round_to(rng.standard_normal(N).astype(np.float32), dtype)
    if pqs:
        p["pqs"] = oracle.round_to(rng.uniform(0.5, 2.0, K).astype(np.float32), dtype)
    p["act"] = oracle.round_to(rng.standard_normal((M, K)).astype(np.float32), dtype)
    return p


def reference(oracle, p, alpha=1.0):
    return oracle.woq_matmul_ref(p["act"], p["q"], p["scales"], p["zeros"], p["bias"], p["pqs"], alpha,
                                 p["group"], p["dtype"])


def parity_err(oracle, out, p, alpha=1.0, w4a8=False):
    """The larger of the two parity norms of `out` against the float64 oracle: the global one,
    max|out - ref| / max|ref|, and the per-output-column one (oracle.max_col_rel_err, floored by the
    column's expected output magnitude)."""
    ref = reference(oracle, p, alpha)
    a = p["act"] if p["pqs"] is None else oracle.apply_per_channel_scale(p["act"], p["pqs"], p["dtype"])
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], p["group"], p["dtype"])
    floor = oracle.column_magnitude(a, w, alpha)
    return max(oracle.max_rel_err(out, ref), oracle.max_col_rel_err(out, ref, floor))


def preprocess(pkg, oracle, q, bits, act_dtype=torch.bfloat16):
    src = torch.from_numpy(q if bits == 8 else oracle.pack_int8_tensor_to_packed_int4(q))
    qt = torch.int8 if bits == 8 else torch.quint4x2
    return pkg.ops.preprocess_weights_for_mixed_gemm(src, qt, act_dtype)


def run_product(pkg, oracle, dev, p, regime=0, w_dev=None):
    F = pkg.functional
    dt = p["dtype"]
    w = w_dev if w_dev is not None else preprocess(pkg, oracle, p["q"], p["bits"]).to(dev)
    algo = (F.INT8_WEIGHT if p["bits"] == 8 else 0) | (F.ZERO if p["zeros"] is not None else 0) \
        | (F.BIAS if p["bias"] is not None else 0) | (F.PRE_QUANT_SCALE if p["pqs"] is not None else 0)
    opt = lambda x: None if x is None else to_dev(x, dt, dev)
    out = F.woq_matmul_raw(to_dev(p["act"], dt, dev), opt(p["pqs"]), w, to_dev(p["scales"], dt, dev),
                           opt(p["zeros"]), opt(p["bias"]), n=p["N"], k=p["K"], group_size=p["group"],
                           quant_algo=algo, out_dtype=TORCH_DT[dt], regime=regime)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()
