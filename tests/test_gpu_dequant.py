"""Bit-exact GPU checks: woq_dequantize (the device dequantize the GEMM main loop uses) and the
pre-quant scale kernel against the oracle's definitions."""
import numpy as np
import pytest
import torch

from _util import preprocess, to_dev, TORCH_DT

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 64, 128, 192, 256])
@pytest.mark.parametrize("zero", [False, True])
def test_dequantize_bit_exact(pkg, oracle, dev, dtype, bits, group, zero):
    K, N = 320, 96
    if 0 < group <= 128 and K % group:
        K = 384  # (groups above 128 may end in a shorter group: 320 = 192 + 128 = 256 + 64)
    rng = np.random.default_rng(bits * 100 + group + zero)
    q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
    gshape = (-(-K // group), N) if group else (N,)
    s = oracle.round_to(np.exp(rng.uniform(-8, 1, gshape)).astype(np.float32), dtype)
    z = oracle.round_to((rng.standard_normal(gshape) * np.exp(rng.uniform(-8, 1, gshape))).astype(np.float32),
                        dtype) if zero and group else None
    w = preprocess(pkg, oracle, q, bits).to(dev)
    got = pkg.functional.dequantize_weights(
        w, to_dev(s, dtype, dev), None if z is None else to_dev(z, dtype, dev), k=K, n=N, group_size=group,
        quant_type=0 if bits == 8 else 1, dtype=TORCH_DT[dtype])
    torch.cuda.synchronize()
    want = oracle.dequantize(q, s, z, group, dtype)
    got_f = got.float().cpu().numpy()
    assert (got_f.view(np.uint32) == want.view(np.uint32)).all(), np.abs(got_f - want).max()


def test_dequantize_fp8_bit_exact(pkg, oracle, dev):
    K, N, G = 256, 64, 128
    rng = np.random.default_rng(7)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    s = oracle.round_f16(np.exp(rng.uniform(-6, 4, (K // G, N))).astype(np.float32))
    z = oracle.round_f16((rng.standard_normal((K // G, N)) * 4).astype(np.float32))
    w = preprocess(pkg, oracle, q, 4, torch.float8_e4m3fn).to(dev)
    got = pkg.functional.dequantize_weights(w, to_dev(s, "fp16", dev), to_dev(z, "fp16", dev), k=K, n=N, group_size=G,
                                            quant_type=2, dtype=torch.float8_e4m3fn)
    torch.cuda.synchronize()
    want = oracle.dequantize(q, s, z, G, "fp8")
    assert (got.view(torch.uint8).cpu().numpy() == oracle.e4m3_bits(want)).all()


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,K", [(1, 64), (7, 4096), (300, 1024)])
def test_apply_per_channel_scale_bit_exact(pkg, oracle, dev, dtype, M, K):
    rng = np.random.default_rng(M + K)
    act = oracle.round_to((rng.standard_normal((M, K)) * np.exp(rng.uniform(-4, 4, (M, K)))).astype(np.float32), dtype)
    sc = oracle.round_to(rng.uniform(0.25, 4.0, K).astype(np.float32), dtype)
    a, s = to_dev(act, dtype, dev), to_dev(sc, dtype, dev)
    same = pkg.functional.apply_per_channel_scale(a, s)
    fp8 = pkg.functional.apply_per_channel_scale(a, s, torch.float8_e4m3fn)
    torch.cuda.synchronize()
    want = oracle.apply_per_channel_scale(act, sc, dtype)
    assert (same.float().cpu().numpy().view(np.uint32) == want.view(np.uint32)).all()
    want8 = oracle.apply_per_channel_scale(act, sc, dtype, "fp8")
    assert (fp8.view(torch.uint8).cpu().numpy() == oracle.e4m3_bits(want8)).all()
