"""The GPTQ / AutoAWQ checkpoint front-end (tensorrt-llm_amd/checkpoint.py) against packers written
from the formats' own definitions:

  AutoGPTQ  qweight[i // 8, n] holds u[i, n] in bits 4*(i % 8); qzeros[g, n // 8] holds zp[g, n] - 1 in
            bits 4*(n % 8); dequantized weight = (u - zp) * scale
  AutoAWQ   word c of a row packs columns 8c + [0, 2, 4, 6, 1, 3, 5, 7][i] in bits 4*i, for weights and
            zero-points alike; dequantized weight = (u - zp) * scale

A wrong nibble order, a dropped GPTQ "+1", a transposed unpack or a pack along the wrong axis each
break the comparison with the directly computed operands."""
import numpy as np
import pytest
import torch

AWQ_PACK_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]


def _quantized(K, N, g, seed, bits=4):
    rng = np.random.default_rng(seed)
    top = (1 << bits) - 1
    u = rng.integers(0, top + 1, size=(K, N)).astype(np.int64)
    zp = rng.integers(1, top + 1, size=(K // g, N)).astype(np.int64)  # >= 1: GPTQ stores zp - 1 unsigned
    scale = rng.uniform(0.002, 0.02, size=(K // g, N)).astype(np.float32)
    return u, zp, scale


def _pack_rows_gptq(u, per_word, bits):
    K, N = u.shape
    out = np.zeros((K // per_word, N), dtype=np.uint32)
    for i in range(K):
        out[i // per_word] |= (u[i].astype(np.uint32) << np.uint32(bits * (i % per_word)))
    return torch.from_numpy(out.view(np.int32))


def _pack_cols(u, order, per_word=8, bits=4):
    R, N = u.shape
    out = np.zeros((R, N // per_word), dtype=np.uint32)
    for c in range(N // per_word):
        for i in range(per_word):
            out[:, c] |= (u[:, per_word * c + order[i]].astype(np.uint32) << np.uint32(bits * i))
    return torch.from_numpy(out.view(np.int32))


def _expected(pkg, u, zp, scale, bits, dtype):
    half = 1 << (bits - 1)
    q_signed = (u - half).astype(np.int8)
    s = torch.from_numpy(scale).to(dtype)
    zeros = (torch.from_numpy((half - zp).astype(np.int32)).to(dtype) * s).to(dtype)
    return q_signed, s, zeros


def _decode(pkg, weight, K, bits):
    qt = torch.quint4x2 if bits == 4 else torch.int8
    raw = pkg.ops.unprocess_weights_for_mixed_gemm(weight, K, qt)
    return pkg.ops.unpack_int4_packed_tensor_to_int8(raw).numpy() if bits == 4 else raw.numpy()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gptq_int4(pkg, dtype):
    K, N, g = 256, 64, 128
    u, zp, scale = _quantized(K, N, g, 1)
    out = pkg.checkpoint.postprocess_gptq(_pack_rows_gptq(u, 8, 4), torch.from_numpy(scale),
                                          _pack_cols(zp - 1, list(range(8))), dtype)
    q, s, z = _expected(pkg, u, zp, scale, 4, dtype)
    assert (_decode(pkg, out["weight"], K, 4) == q).all()
    assert torch.equal(out["weights_scaling_factor"], s) and torch.equal(out["zero"], z)


def test_gptq_int8(pkg):
    K, N, g = 128, 32, 64
    u, zp, scale = _quantized(K, N, g, 2, bits=8)
    zp = np.clip(zp, 1, 128)  # the reference's unsigned expression is only meaningful up to 128
    out = pkg.checkpoint.postprocess_gptq(_pack_rows_gptq(u, 4, 8), torch.from_numpy(scale),
                                          _pack_cols(zp - 1, list(range(4)), 4, 8), torch.float16, bits=8)
    q, s, z = _expected(pkg, u, zp, scale, 8, torch.float16)
    assert (_decode(pkg, out["weight"], K, 8) == q).all()
    assert torch.equal(out["weights_scaling_factor"], s) and torch.equal(out["zero"], z)


def test_autoawq_int4(pkg):
    K, N, g = 128, 64, 64
    u, zp, scale = _quantized(K, N, g, 3)
    out = pkg.checkpoint.postprocess_autoawq(_pack_cols(u, AWQ_PACK_ORDER), torch.from_numpy(scale),
                                             _pack_cols(zp, AWQ_PACK_ORDER), torch.bfloat16)
    q, s, z = _expected(pkg, u, zp, scale, 4, torch.bfloat16)
    assert (_decode(pkg, out["weight"], K, 4) == q).all()
    assert torch.equal(out["weights_scaling_factor"], s) and torch.equal(out["zero"], z)


def test_unpack_orders(pkg):
    """unpack_int32_into_int8: low nibble first; the AutoAWQ gather restores column order."""
    C = pkg.checkpoint
    w = torch.tensor([[0x76543210]], dtype=torch.int32)
    assert C.unpack_int32_into_int8(w).tolist() == [[0, 1, 2, 3, 4, 5, 6, 7]]
    packed = _pack_cols(np.arange(8).reshape(1, 8), AWQ_PACK_ORDER)
    assert C.unpack_int32_into_int8(packed, True).tolist() == [[0, 1, 2, 3, 4, 5, 6, 7]]


def test_tp_split_padding_and_qkv_reorder(pkg):
    C = pkg.checkpoint
    K, N, g = 128, 96, 64
    u, zp, scale = _quantized(K, N, g, 5)
    args = (_pack_cols(u, AWQ_PACK_ORDER), torch.from_numpy(scale), _pack_cols(zp, AWQ_PACK_ORDER), torch.float16)
    # column-parallel rank 1 of 2, padded from 48 to 64 columns (the 64*tp rule of the layers)
    assert C.padded_features(128, 48, 64) == (128, 64) and C.padded_features(100, 100, 0, tp_size=2) == (128, 128)
    out = C.postprocess_autoawq(*args, tp_split=(1, 2, 1), padded_shape=(128, 64))
    q, s, z = _expected(pkg, u[:, 48:], zp[:, 48:], scale[:, 48:], 4, torch.float16)
    dec = _decode(pkg, out["weight"], K, 4)
    assert dec.shape == (128, 64) and (dec[:, :48] == q).all() and (dec[:, 48:] == 0).all()
    assert torch.equal(out["weights_scaling_factor"][:, :48], s) and (out["weights_scaling_factor"][:, 48:] == 1).all()
    assert torch.equal(out["zero"][:, :48], z)
    # row-parallel rank 0 of 2: rows and groups are cut together
    out = C.postprocess_autoawq(*args, tp_split=(0, 2, 0))
    q, s, z = _expected(pkg, u[:64], zp[:1], scale[:1], 4, torch.float16)
    assert (_decode(pkg, out["weight"], 64, 4) == q).all() and torch.equal(out["zero"], z)
    # fused QKV stored head-major (h, qkv, d) -> (qkv, h, d): heads=2, d=16
    out = C.postprocess_autoawq(*args, num_heads=2)
    perm = np.arange(96).reshape(2, 3, 16).transpose(1, 0, 2).reshape(-1)
    q, s, z = _expected(pkg, u[:, perm], zp[:, perm], scale[:, perm], 4, torch.float16)
    assert (_decode(pkg, out["weight"], K, 4) == q).all() and torch.equal(out["zero"], z)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["gptq", "awq"])
def test_checkpoint_tensors_run_through_the_matmul(pkg, oracle, dev, fmt):
    """End to end: packed checkpoint tensors -> front-end -> GPU matmul == act @ ((u - zp) * scale)."""
    K, N, g, M = 512, 256, 128, 24
    u, zp, scale = _quantized(K, N, g, 7)
    if fmt == "gptq":
        t = pkg.checkpoint.postprocess_gptq(_pack_rows_gptq(u, 8, 4), torch.from_numpy(scale),
                                            _pack_cols(zp - 1, list(range(8))), torch.bfloat16)
    else:
        t = pkg.checkpoint.postprocess_autoawq(_pack_cols(u, AWQ_PACK_ORDER), torch.from_numpy(scale),
                                               _pack_cols(zp, AWQ_PACK_ORDER), torch.bfloat16)
    rng = np.random.default_rng(8)
    act = oracle.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    F = pkg.functional
    out = F.weight_only_groupwise_quant_matmul(
        torch.from_numpy(act).to(torch.bfloat16).to(dev), None, t["weight"].to(dev),
        t["weights_scaling_factor"].to(dev), t["zero"].to(dev), None, None, F.ZERO, g, "bfloat16")
    torch.cuda.synchronize()
    s_bf = t["weights_scaling_factor"].float().numpy()
    w = (np.repeat(u - 8, 1, axis=0).astype(np.float64) * np.repeat(s_bf, g, axis=0)
         + np.repeat(t["zero"].float().numpy(), g, axis=0))
    ref = act.astype(np.float64) @ w
    assert oracle.max_rel_err(out.float().cpu().numpy(), ref) < 1e-2
    # and the folded zeros mean (u - zp) * scale up to the rounding of the zero tensor
    w_true = (u - np.repeat(zp, g, axis=0)) * np.repeat(s_bf, g, axis=0)
    assert np.abs(w - w_true).max() <= np.abs(w_true).max() * 2.0 ** -7
