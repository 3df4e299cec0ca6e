"""GPU parity of the fused RMSNorm + smoothing pass against the oracle's restatement of the
reference's two kernels (rmsnormKernels.cu + preQuantScaleKernel.cu).  The kernel sums the squares in
float32 in its own order, so 1/rms can differ from the oracle's in the last bit and a few outputs
land on the neighbouring value of the 16-bit type; the smoothing multiply and its rounding can carry
that to a second step.  The bar: (a) at most two units in the last place of the output type
anywhere, (b) bit-identical on at least 98 % of the elements."""
import numpy as np
import pytest
import torch

from _util import TORCH_DT, to_dev

pytestmark = pytest.mark.gpu


def _case(oracle, m, k, dtype, scale, beta, seed):
    rng = np.random.default_rng(seed)
    x = oracle.round_to((rng.standard_normal((m, k)) * rng.uniform(0.1, 4.0, (m, 1))).astype(np.float32), dtype)
    gamma = oracle.round_to(rng.uniform(0.5, 1.5, k).astype(np.float32), dtype)
    b = oracle.round_to((rng.standard_normal(k) * 0.1).astype(np.float32), dtype) if beta else None
    s = oracle.round_to(rng.uniform(0.5, 2.0, k).astype(np.float32), dtype) if scale else None
    return x, gamma, b, s


def _ulp(ref, dtype):
    """Spacing of the output type at |ref| (normal range)."""
    bits = {"bf16": 7, "fp16": 10, "fp8": 3}[dtype]
    mag = np.maximum(np.abs(ref), {"bf16": 1e-30, "fp16": 6.2e-5, "fp8": 2.0 ** -6}[dtype])
    return 2.0 ** (np.floor(np.log2(mag)) - bits)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("m,k", [(1, 4096), (5, 64), (16, 8192), (300, 4096), (3, 28672), (2, 40), (7, 5128)])
@pytest.mark.parametrize("scale,beta,fp8", [(True, False, False), (True, False, True), (False, False, False),
                                            (True, True, False), (False, True, True)])
def test_rmsnorm_prequant(pkg, oracle, dev, dtype, m, k, scale, beta, fp8):
    F = pkg.functional
    x, gamma, b, s = _case(oracle, m, k, dtype, scale, beta, seed=m + k)
    eps = 1e-5
    opt = lambda v: None if v is None else to_dev(v, dtype, dev)
    out = F.rmsnorm_prequant(to_dev(x, dtype, dev), to_dev(gamma, dtype, dev), opt(s), eps, opt(b),
                             torch.float8_e4m3fn if fp8 else None)
    torch.cuda.synchronize()
    assert out.dtype == (torch.float8_e4m3fn if fp8 else TORCH_DT[dtype]) and tuple(out.shape) == (m, k)
    got = out.float().cpu().numpy()
    ref = oracle.rmsnorm_ref(x, gamma, eps, dtype, b)
    if s is not None:
        ref = oracle.apply_per_channel_scale(ref, s, dtype, "fp8" if fp8 else None)
    elif fp8:
        ref = oracle.round_to(ref, "fp8")
    assert np.isfinite(got).all()
    assert (np.abs(got - ref) <= 2.001 * _ulp(ref, "fp8" if fp8 else dtype)).all()
    assert (got == ref).mean() >= 0.98


def test_rmsnorm_feeds_the_matmul(pkg, oracle, dev):
    """The fused pass in front of the W4A8 matmul equals RMSNorm, then the matmul's own smoothing."""
    F = pkg.functional
    m, k, n = 8, 1024, 256
    prob = oracle.make_w4a8_problem(m, k, n, seed=5, out_dtype="bf16")
    x, gamma, _, _ = _case(oracle, m, k, "bf16", False, False, seed=9)
    from _util import preprocess
    w = preprocess(pkg, oracle, prob["q"], 4, torch.float8_e4m3fn).to(dev)
    scales = to_dev(prob["scales"], "fp16", dev)
    pqs = to_dev(prob["pre_quant_scale"], "bf16", dev)
    a8 = F.rmsnorm_prequant(to_dev(x, "bf16", dev), to_dev(gamma, "bf16", dev), pqs, 1e-5, None, torch.float8_e4m3fn)
    fused = F.woq_matmul_raw(a8, None, w, scales, None, None, n=n, k=k, group_size=128, quant_algo=F.FP8_ALPHA,
                             alpha=prob["alpha"], out_dtype=torch.bfloat16)
    normed = F.rmsnorm_prequant(to_dev(x, "bf16", dev), to_dev(gamma, "bf16", dev), None, 1e-5)
    two_step = F.woq_matmul_raw(normed, pqs, w, scales, None, None, n=n, k=k, group_size=128,
                                quant_algo=F.FP8_ALPHA | F.PRE_QUANT_SCALE, alpha=prob["alpha"], out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert torch.equal(fused, two_step)
