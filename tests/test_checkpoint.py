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


# ---- ModelOpt AWQ, the W4A8 fold, q / k / v concatenation ------------------------------------------


def _modelopt_pack(q_signed):
    """[K, N] signed int4 -> ModelOpt's int8 [N/2, K]: output channels 2j (low nibble) and 2j + 1 of
    input k share byte (j, k)."""
    u = (q_signed.T.astype(np.int16) & 0xF).astype(np.uint8)  # [N, K]
    return torch.from_numpy((u[0::2] | (u[1::2] << 4)).view(np.int8).copy())


def test_modelopt_awq_layer_and_separate_qkv(pkg):
    """The transposed int8 tensor, the [N, K/g] scales and the smoothing vector of ModelOpt's export become
    the op's operands; q, k, v given separately are the same as one fused layer."""
    K, g = 256, 128
    rng = np.random.default_rng(5)
    parts = [rng.integers(-8, 8, size=(K, n)).astype(np.int8) for n in (64, 32, 32)]
    scales = [rng.uniform(0.002, 0.02, size=(p.shape[1], K // g)).astype(np.float32) for p in parts]
    pqs = torch.from_numpy(rng.uniform(0.5, 2.0, K).astype(np.float32))
    one = pkg.checkpoint.postprocess_modelopt_awq(_modelopt_pack(parts[0]), torch.from_numpy(scales[0]).reshape(-1), pqs,
                                                  torch.bfloat16, group_size=g)
    assert (_decode(pkg, one["weight"], K, 4) == parts[0]).all()
    assert torch.equal(one["weights_scaling_factor"], torch.from_numpy(scales[0].T.copy()).to(torch.bfloat16))
    assert one["prequant_scaling_factor"].shape == (1, K)
    fused = pkg.checkpoint.postprocess_modelopt_awq([_modelopt_pack(p) for p in parts],
                                                    [torch.from_numpy(s) for s in scales], [pqs, pqs, pqs],
                                                    torch.bfloat16, group_size=g)
    assert (_decode(pkg, fused["weight"], K, 4) == np.concatenate(parts, axis=1)).all()
    want = torch.from_numpy(np.concatenate([s.T for s in scales], axis=1)).to(torch.bfloat16)
    assert torch.equal(fused["weights_scaling_factor"], want)
    # column-parallel split of every part before the concatenation, as the reference's loader does
    half = pkg.checkpoint.postprocess_modelopt_awq([_modelopt_pack(p) for p in parts],
                                                   [torch.from_numpy(s) for s in scales], pqs, torch.bfloat16,
                                                   group_size=g, tp_split=(1, 2, 1))
    assert (_decode(pkg, half["weight"], K, 4) == np.concatenate([p[:, p.shape[1] // 2:] for p in parts], axis=1)).all()


def test_gptq_parts_concatenate_along_n(pkg):
    K, g = 128, 64
    us, zps, scs = zip(*[_quantized(K, n, g, 20 + n) for n in (32, 16, 16)])
    parts = [(_pack_rows_gptq(u, 8, 4), torch.from_numpy(s), _pack_cols(zp - 1, list(range(8))))
             for u, zp, s in zip(us, zps, scs)]
    out = pkg.checkpoint.postprocess_gptq(*pkg.checkpoint.concat_gptq_parts(parts), torch.float16)
    q, s, z = _expected(pkg, np.concatenate(us, 1), np.concatenate(zps, 1), np.concatenate(scs, 1), 4, torch.float16)
    assert (_decode(pkg, out["weight"], K, 4) == q).all() and torch.equal(out["zero"], z)


def test_w4a8_fold_is_the_loaders_and_the_oracles(pkg, oracle):
    """fold_w4a8 follows the reference loader's order of operations (modeling_utils.py:1661-1682):
    hand-computed values, and agreement with the oracle's benchmark-input generator, which folds the same
    factors on its own (float32 group scales / wsf2 -> float16; smoothing / act_sf; alpha = act_sf * wsf2)."""
    f = pkg.checkpoint.fold_w4a8(torch.tensor([[0.5, 0.25], [1.0, 3.0]]), torch.tensor([[2.0, 4.0]]),
                                 torch.tensor(0.5), torch.tensor(0.125))
    assert torch.equal(f["weights_scaling_factor"], torch.tensor([[4.0, 2.0], [8.0, 24.0]], dtype=torch.float16))
    assert torch.equal(f["prequant_scaling_factor"], torch.tensor([[4.0, 8.0]]))
    assert f["alpha"].dtype == torch.float32 and f["alpha"].item() == 0.0625
    M, K, N = 4, 256, 64
    prob = oracle.make_w4a8_problem(M, K, N, seed=9, out_dtype="bf16")
    # the same unfolded inputs, recomputed as the generator defines them
    q, scale = oracle.make_w4_groupwise_sym(K, N, 128, 9, "fp32")
    rng = np.random.default_rng(9 + 7)
    smooth = oracle.round_to(rng.uniform(0.5, 2.0, size=(K,)).astype(np.float32), "bf16")
    act = oracle.make_activations(M, K, 9 + 13, "bf16")
    act_sf = np.float32(np.abs(act * smooth).max() / 448.0)
    wsf2 = np.float32(np.abs(q.astype(np.float32).reshape(K // 128, 128, N) * scale[:, None, :]).max() / 448.0)
    f = pkg.checkpoint.fold_w4a8(torch.from_numpy(scale), torch.from_numpy(smooth), torch.tensor(act_sf),
                                 torch.tensor(wsf2))
    assert (f["weights_scaling_factor"].float().numpy() == prob["scales"]).all()
    assert (oracle.round_to(f["prequant_scaling_factor"].numpy(), "bf16") == prob["pre_quant_scale"]).all()
    assert f["alpha"].item() == np.float32(prob["alpha"])


def test_w4a8_fold_keeps_dtypes_with_the_layers_factor_shapes(pkg):
    """The layers declare alpha, activation_scaling_factor and weights_scaling_factor_2 as float32 of shape
    (1,) (quantization/layers.py).  The reference divides in place, so a bf16 model's smoothing vector stays
    bf16 and its group scales are rounded to bf16 before they become float16: quotient in float32, one
    rounding to the tensor's own type."""
    wsf = torch.tensor([[0.3, 1.7], [2.9, 0.011]], dtype=torch.bfloat16)
    pqs = torch.tensor([[1.3, 0.7, 2.9]], dtype=torch.bfloat16)
    act_sf, wsf2 = torch.tensor([0.3], dtype=torch.float32), torch.tensor([0.7], dtype=torch.float32)
    f = pkg.checkpoint.fold_w4a8(wsf, pqs, act_sf, wsf2)
    assert f["prequant_scaling_factor"].dtype == torch.bfloat16 and f["prequant_scaling_factor"].shape == (1, 3)
    assert f["weights_scaling_factor"].dtype == torch.float16 and f["alpha"].dtype == torch.float32
    assert f["alpha"].shape == (1,) and f["alpha"].item() == (act_sf * wsf2).item()
    assert torch.equal(f["prequant_scaling_factor"], (pqs.float() / 0.3).to(torch.bfloat16))
    assert torch.equal(f["weights_scaling_factor"], (wsf.float() / 0.7).to(torch.bfloat16).to(torch.float16))
    # not the same as dividing by the factor rounded to bf16 first, nor as skipping the bf16 rounding
    assert not torch.equal(f["weights_scaling_factor"], (wsf.float() / 0.7).to(torch.float16))
    assert torch.equal(wsf, torch.tensor([[0.3, 1.7], [2.9, 0.011]], dtype=torch.bfloat16))  # inputs untouched
    # fp16 model: same rule
    f = pkg.checkpoint.fold_w4a8(wsf.to(torch.float16), pqs.to(torch.float16), act_sf, wsf2)
    assert f["prequant_scaling_factor"].dtype == torch.float16


# ---- per-channel layers from float weights ----------------------------------------------------------


@pytest.mark.parametrize("quant_type,bits", [(torch.int8, 8), (torch.quint4x2, 4)])
def test_postprocess_weight_only_quantizes_like_the_oracle(pkg, oracle, quant_type, bits):
    """[out, in] float weight -> transposed, quantized per output column (amax / 2^(bits-1), half away from
    zero: the oracle's symmetric_quantize), laid out for the kernels."""
    N, K = 96, 128
    rng = np.random.default_rng(31)
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.02).astype(np.float32)).to(torch.float16)
    out = pkg.checkpoint.postprocess_weight_only(w, quant_type)
    q, scale = oracle.symmetric_quantize(w.float().numpy().T.copy(), bits, "fp16")
    assert (_decode(pkg, out["weight"], K, bits) == q).all()
    assert out["per_channel_scale"].dtype == torch.float16
    assert (out["per_channel_scale"].float().numpy() == scale).all()


def test_postprocess_weight_only_tp_split_padding_and_bias(pkg, oracle):
    """The reference's padded layers (functional.py:883-886, 896-899): a column-parallel layer with 100
    output features on 2 ranks pads to 64 per rank; ranks own runs of 64 columns of the transposed weight
    (rank 1: the remaining 36, padded with zeros); the bias is cut and padded with them.  Row-parallel
    layers cut K and keep the bias."""
    C = pkg.checkpoint
    N, K = 100, 100
    rng = np.random.default_rng(32)
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.02).astype(np.float32)).to(torch.bfloat16)
    bias = torch.arange(N, dtype=torch.float32).to(torch.bfloat16)
    k_pad, n_pad = C.padded_features(K, N, 0, tp_size=2)  # 128, 128 in total: 64 columns per rank
    assert (k_pad, n_pad) == (128, 128)
    wt = w.float().numpy().T  # [K, N]
    for rank, cols in ((0, slice(0, 64)), (1, slice(64, 100))):
        out = C.postprocess_weight_only(w, torch.int8, bias=bias, tp_split=(1, 2, rank), padded_shape=(k_pad, n_pad // 2))
        piece = np.zeros((k_pad, 64), np.float32)
        piece[:K, :cols.stop - cols.start] = wt[:, cols]
        q, scale = oracle.symmetric_quantize(piece, 8, "bf16")
        assert (_decode(pkg, out["weight"], k_pad, 8) == q).all()
        assert (out["per_channel_scale"].float().numpy() == scale).all()
        want_bias = torch.zeros(64, dtype=torch.bfloat16)
        want_bias[:cols.stop - cols.start] = bias[cols]
        assert torch.equal(out["bias"], want_bias)
    # row-parallel, unpadded: equal parts of K, bias passed through
    out = C.postprocess_weight_only(w[:96, :64].contiguous(), torch.quint4x2, bias=bias[:96], tp_split=(0, 2, 1))
    q, scale = oracle.symmetric_quantize(wt[32:64, :96].copy(), 4, "bf16")
    assert (_decode(pkg, out["weight"], 32, 4)[:32] == q).all() and torch.equal(out["bias"], bias[:96])
    assert (out["per_channel_scale"].float().numpy() == scale).all()
    with pytest.raises(ValueError):
        C.postprocess_weight_only(w.to(torch.int8), torch.int8)
    # a batch of experts [E, out, in] keeps its leading dimension
    e = C.postprocess_weight_only(torch.stack([w[:64, :64], w[:64, 36:]]).contiguous(), torch.int8)
    assert e["per_channel_scale"].shape == (2, 64)


@pytest.mark.gpu
@pytest.mark.parametrize("quant_type,bits,M", [(torch.int8, 8, 1), (torch.quint4x2, 4, 40)])
def test_postprocess_weight_only_layer_runs_through_the_matmul(pkg, oracle, dev, quant_type, bits, M):
    """Float checkpoint weight -> per-channel hook -> GPU matmul == the oracle's dequantize-then-matmul on
    the oracle's own quantization of the same weight."""
    N, K = 512, 1024
    rng = np.random.default_rng(33)
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.02).astype(np.float32)).to(torch.float16)
    t = pkg.checkpoint.postprocess_weight_only(w, quant_type)
    act = oracle.round_f16(rng.standard_normal((M, K)).astype(np.float32))
    F = pkg.functional
    out = F.weight_only_quant_matmul(torch.from_numpy(act).to(torch.float16).to(dev), t["weight"].to(dev),
                                     t["per_channel_scale"].to(dev), F.INT8 if bits == 8 else F.INT4, "float16")
    torch.cuda.synchronize()
    q, scale = oracle.symmetric_quantize(w.float().numpy().T.copy(), bits, "fp16")
    ref = oracle.woq_matmul_ref(act, q, scale, group_size=0, act_dtype="fp16")
    assert oracle.max_rel_err(out.float().cpu().numpy(), ref) < 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("M", [4, 200])
def test_modelopt_w4a8_layer_runs_through_the_matmul(pkg, oracle, dev, M):
    """A ModelOpt-style W4A8 layer (int8 [N/2, K] weight, [N, K/g] scales, smoothing vector, the two per-tensor
    factors as float32 tensors of shape (1,)) -> postprocess_modelopt_awq -> woq_matmul with 16-bit activations
    and the smoothing vector == the oracle on the operands of its own benchmark generator, which folds the same
    factors independently."""
    K, N, g = 512, 384, 128
    seed = 50 + M
    prob = oracle.make_w4a8_problem(M, K, N, seed=seed, out_dtype="bf16")
    # the unfolded tensors, as the generator defines them
    q, scale = oracle.make_w4_groupwise_sym(K, N, g, seed, "fp32")
    rng = np.random.default_rng(seed + 7)
    smooth = oracle.round_to(rng.uniform(0.5, 2.0, size=(K,)).astype(np.float32), "bf16")
    act = oracle.make_activations(M, K, seed + 13, "bf16")
    act_sf = np.float32(np.abs(act * smooth).max() / 448.0)
    wsf2 = np.float32(np.abs(q.astype(np.float32).reshape(K // g, g, N) * scale[:, None, :]).max() / 448.0)
    assert (q == prob["q"]).all()
    t = pkg.checkpoint.postprocess_modelopt_awq(
        _modelopt_pack(q), torch.from_numpy(scale.T.copy()), torch.from_numpy(smooth), torch.float32, group_size=g,
        activation_scaling_factor=torch.tensor([act_sf]), weights_scaling_factor_2=torch.tensor([wsf2]))
    assert (t["weights_scaling_factor"].float().numpy() == prob["scales"]).all()
    pqs = t["prequant_scaling_factor"].to(torch.bfloat16).reshape(-1)
    assert (pqs.float().numpy() == prob["pre_quant_scale"]).all()
    F = pkg.functional
    out = F.weight_only_groupwise_quant_matmul(
        torch.from_numpy(prob["act"]).to(torch.bfloat16).to(dev), pqs.to(dev), t["weight"].to(dev),
        t["weights_scaling_factor"].to(dev), None, None, t["alpha"], F.PRE_QUANT_SCALE | F.FP8_ALPHA, g, "bfloat16")
    torch.cuda.synchronize()
    ref = oracle.woq_matmul_ref(prob["act"], prob["q"], prob["scales"], None, None, prob["pre_quant_scale"],
                                prob["alpha"], g, "bf16", w4a8=True)
    assert abs(float(t["alpha"]) - prob["alpha"]) <= 1e-7 * prob["alpha"]
    assert oracle.max_rel_err(out.float().cpu().numpy(), ref) < 1e-2


# ---- TensorRT-LLM checkpoints (reference-layout weights) ---------------------------------------------

import json
import os

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CKPTS = sorted(d for d in os.listdir(GOLDEN) if d.startswith("trtllm_ckpt_"))


def _fixture(name):
    from safetensors.torch import load_file
    path = os.path.join(GOLDEN, name)
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    return path, cfg, load_file(os.path.join(path, "rank0.safetensors"))


@pytest.mark.parametrize("name", CKPTS)
def test_load_trtllm_linear_decodes_the_reference_layout(pkg, name):
    """Every fixture checkpoint (tests/golden/make_trtllm_checkpoint.py: weights in the reference's SM80 /
    SM89 / SM90 layouts, W8A16, W4A16, AWQ, GPTQ and W4A8 flavours) loads into this library's layout
    holding exactly the quantized values it was made from; the other tensors pass through under the op's
    argument names."""
    path, cfg, raw = _fixture(name)
    fx = cfg["_fixture"]
    layer = pkg.checkpoint.load_trtllm_linear(path, fx["layer"], sm_arch=fx["sm_arch"])
    q = raw["_expected.%s.q" % fx["layer"]].numpy()
    assert (layer["k"], layer["n"]) == (fx["k"], fx["n"]) == q.shape
    act_type = torch.float8_e4m3fn if layer["w4a8"] else torch.float16
    qt = torch.quint4x2 if layer["bits"] == 4 else torch.int8
    back = pkg.ops.unprocess_weights_for_mixed_gemm(layer["weight"], fx["k"], qt, act_type)
    back = pkg.ops.unpack_int4_packed_tensor_to_int8(back).numpy() if layer["bits"] == 4 else back.numpy()
    assert (back == q).all()
    quant = cfg["quantization"]
    assert layer["group_size"] == (quant["group_size"] or 0)
    assert (layer["zeros"] is not None) == quant["has_zero_point"]
    assert (layer["pre_quant_scale"] is not None) == quant["pre_quant_scale"]
    F = pkg.functional
    assert bool(layer["quant_algo"] & F.FP8_ALPHA) == (quant["quant_algo"] == "W4A8_AWQ")
    if layer["w4a8"]:
        assert layer["scales"].dtype == torch.float16 and abs(layer["alpha"] - 0.0123) < 1e-9
    # a wrong SM decodes to other values (80 and 90 differ by the column interleave)
    other = 90 if fx["sm_arch"] != 90 else 80
    wrong = pkg.checkpoint.load_trtllm_linear(path, fx["layer"], sm_arch=other)
    assert not torch.equal(wrong["weight"], layer["weight"])


def test_load_trtllm_linear_errors(pkg):
    path, cfg, raw = _fixture("trtllm_ckpt_w4a16_awq_sm80")
    layer = cfg["_fixture"]["layer"]
    with pytest.raises(KeyError):
        pkg.checkpoint.load_trtllm_linear(path, "transformer.layers.9.mlp.fc", sm_arch=80)
    with pytest.raises(ValueError, match="quant_algo"):
        pkg.checkpoint.load_trtllm_linear(raw, layer, sm_arch=80, quant_algo="FP8")
    # a dict of tensors instead of a directory, the algorithm given by the caller
    again = pkg.checkpoint.load_trtllm_linear(raw, layer, sm_arch=80, quant_algo="W4A16_AWQ")
    assert torch.equal(again["weight"], pkg.checkpoint.load_trtllm_linear(path, layer, sm_arch=80)["weight"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", CKPTS)
@pytest.mark.parametrize("M", [3, 40])
def test_trtllm_checkpoint_layer_runs_through_the_matmul(pkg, oracle, dev, name, M):
    """End to end: checkpoint directory -> loader -> GPU matmul == the oracle's dequantize-then-matmul on
    the values the fixture was made from (streaming kernel at 3 rows, GEMM kernels at 40)."""
    path, cfg, raw = _fixture(name)
    fx = cfg["_fixture"]
    layer = pkg.checkpoint.load_trtllm_linear(path, fx["layer"], sm_arch=fx["sm_arch"])
    dt = {"float16": "fp16", "bfloat16": "bf16"}[cfg["dtype"]]
    tdt = {"fp16": torch.float16, "bf16": torch.bfloat16}[dt]
    rng = np.random.default_rng(M)
    act = oracle.round_to(rng.standard_normal((M, fx["k"])).astype(np.float32), dt)
    out = pkg.checkpoint.linear_forward(layer, torch.from_numpy(act).to(tdt).to(dev))
    torch.cuda.synchronize()
    f32 = lambda x: None if x is None else x.float().numpy()
    q = raw["_expected.%s.q" % fx["layer"]].numpy()
    ref = oracle.woq_matmul_ref(act, q, f32(layer["scales"]), f32(layer["zeros"]), f32(layer["bias"]),
                                f32(layer["pre_quant_scale"]), layer["alpha"], layer["group_size"], dt,
                                w4a8=layer["w4a8"])
    assert oracle.max_rel_err(out.float().cpu().numpy(), ref) < 1e-2
