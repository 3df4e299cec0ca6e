"""Pins the CPU oracle itself: closed forms, brute force, invariants and the three-way agreement
of the reference-layout restatements.  No GPU, no product code."""
import ctypes

import numpy as np
import pytest

QT = [("W8_A16", 0), ("W4_A16", 1), ("W4_AFP8", 2)]


def test_pack_unpack_all_bytes(oracle):
    # brute force: every byte value decodes to (low nibble, high nibble) sign-extended, and re-encodes
    allb = np.arange(256, dtype=np.uint8).view(np.int8)
    un = oracle.unpack_int4_packed_tensor_to_int8(allb)
    for b in range(256):
        lo, hi = b & 0xF, b >> 4
        assert un[2 * b] == (lo - 16 if lo >= 8 else lo)
        assert un[2 * b + 1] == (hi - 16 if hi >= 8 else hi)
    assert (oracle.pack_int8_tensor_to_packed_int4(un) == allb).all()


def test_pack_rejects_out_of_range(oracle):
    with pytest.raises(ValueError):
        oracle.pack_int8_tensor_to_packed_int4(np.array([8, 0], np.int8))


def test_symmetric_quantize_known_answers(oracle):
    # column 0: absmax 8 -> int4 scale 1.0; ties round AWAY from zero; +8 clips to 7
    w = np.array([[8.0, 0.0, 0.0], [0.5, 0.0, 1.0], [-0.5, 0.0, -1.0], [2.5, 0.0, 0.5], [-2.5, 0.0, 0.25],
                  [-8.0, 0.0, 0.125]], np.float32)
    q, s = oracle.symmetric_quantize(w, 4, "fp32")
    assert s.tolist() == [1.0, 0.0, 0.125]
    assert q[:, 0].tolist() == [7, 1, -1, 3, -3, -8]
    assert q[:, 1].tolist() == [0] * 6                      # zero column guard
    assert q[:, 2].tolist() == [0, 7, -8, 4, 2, 1]
    # int8: scale = absmax / 128 (not /127)
    w8 = np.array([[1.0], [-1.0], [0.5], [1.0 / 256]], np.float32)
    q8, s8 = oracle.symmetric_quantize(w8, 8, "fp32")
    assert s8[0] == np.float32(1.0 / 128)
    assert q8[:, 0].tolist() == [127, -128, 64, 1]          # 0.5 tie -> away from zero


def test_symmetric_quantize_matches_c_restatement(oracle, oracle_c):
    rng = np.random.default_rng(3)
    for bits in (4, 8):
        w = rng.standard_normal((96, 40)).astype(np.float32)
        w[5, 7] = 0.5 * np.abs(w[:, 7]).max() / (1 << (bits - 1))  # a value on a rounding tie
        q, s = oracle.symmetric_quantize(w, bits, "fp32")
        qc = np.zeros_like(q)
        sc = np.zeros(40, np.float32)
        oracle_c.oracle_symmetric_quantize(qc.ctypes.data_as(ctypes.c_void_p), sc.ctypes.data_as(ctypes.c_void_p),
                                           w.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(96), ctypes.c_size_t(40),
                                           bits)
        assert (q == qc).all() and (s == sc).all()


@pytest.mark.parametrize("name,qi", QT)
@pytest.mark.parametrize("arch", [80, 90])
def test_reference_layout_three_way(oracle, oracle_c, name, qi, arch):
    """array-op form == loop-form C restatement, byte for byte, and both are inverted by the
    emulation of the reference GEMV's own addressing."""
    bits = oracle.weight_bits(name)
    K, N = (256, 128) if bits == 4 else (128, 64)
    rng = np.random.default_rng(qi * 10 + arch)
    q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
    raw = oracle.ref_preprocess(q, name, arch)
    assert raw.size == K * N * bits // 8                     # same byte count in and out
    src = q.view(np.uint8).copy() if bits == 8 else oracle.pack_int8_tensor_to_packed_int4(q).view(np.uint8).copy()
    dst = np.zeros_like(src).reshape(-1)
    rc = oracle_c.oracle_ref_preprocess(dst.ctypes.data_as(ctypes.c_void_p), src.ctypes.data_as(ctypes.c_void_p),
                                        ctypes.c_size_t(K), ctypes.c_size_t(N), qi, arch)
    assert rc == 0
    assert (dst == raw).all()
    assert (oracle.ref_layout_decode(raw, K, N, name, arch) == q).all()
    if arch != 90:
        for cta_n in (4, 8):                                   # with / without zeros in the reference dispatcher
            assert (oracle.ref_gemv_decode(raw, K, N, name, cta_n) == q).all()


@pytest.mark.parametrize("name,qi", QT)
def test_reference_layout_is_a_bijection_on_positions(oracle, name, qi):
    """Push element ids (not 4-bit values) through the index form: every position is hit once."""
    bits = oracle.weight_bits(name)
    K, N = 128, 64
    perm = oracle._PERM[name]
    tile_k, il = oracle.ref_layout_constants(name)
    ids = np.arange(K * N).reshape(K, N)
    x = ids.reshape(K // len(perm), len(perm), N)[:, perm, :].reshape(K, N).T
    x = x.reshape(N // il, il, K // tile_k, tile_k).transpose(0, 2, 1, 3).reshape(-1)
    x = x.reshape(-1, 32 // bits)[:, oracle._WORD_ORDER[bits]].reshape(-1)
    assert sorted(x.tolist()) == list(range(K * N))
    # closed form of a6 for one probe element: logical (k, n) -> flat position
    k, n = 70, 13
    kp = k - k % len(perm) + perm.index(k % len(perm))
    flat = (n // il) * (il * K) + (kp // tile_k) * (il * tile_k) + (n % il) * tile_k + kp % tile_k
    word, within = divmod(flat, 32 // bits)
    slot = oracle._WORD_ORDER[bits].index(within)
    assert x[word * (32 // bits) + slot] == ids[k, n]


def test_w8_row_permutation_is_not_an_involution(oracle):
    perm = oracle._PERM["W8_A16"]
    assert perm[2] == 8 and perm.index(2) == 4


def test_gfx950_layout_roundtrip_and_padding(oracle):
    rng = np.random.default_rng(5)
    for bits, K, N in [(4, 256, 64), (4, 192, 32), (8, 128, 48), (8, 96, 16)]:
        q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
        raw = oracle.gfx950_preprocess(q, bits)
        assert raw.size == oracle.gfx950_preprocessed_bytes(K, N, bits)
        assert (oracle.gfx950_decode(raw, K, N, bits) == q).all()
    # one hand-checked position: int4, (k, n) = (37, 18): strip 1, tile 0, slab 1, kg 0, e 5, c 2
    q = np.zeros((128, 32), np.int8)
    q[37, 18] = -3
    raw = oracle.gfx950_preprocess(q, 4)
    byte = (1 * 1 + 0) * 1024 + (0 * 16 + 2) * 16 + 1 * 4      # strip 1, lane 2, dword 1
    word = int.from_bytes(raw[byte:byte + 4].tobytes(), "little")
    slot = 4 + 5 // 2                                          # odd element 5 -> nibble 6
    assert (word >> (4 * slot)) & 0xF == (-3 + 8)
    assert sum(1 for v in oracle._unpack_unsigned(raw, 4) if v != 8) == 1


def test_float_helpers_against_torch(oracle):
    import torch
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-12, 8, 20000))).astype(np.float32)
    assert (oracle.round_bf16(x) == torch.from_numpy(x).to(torch.bfloat16).float().numpy()).all()
    assert (oracle.round_f16(x) == torch.from_numpy(x).to(torch.float16).float().numpy()).all()
    xs = np.clip(x, -448, 448)
    ref8 = torch.from_numpy(xs).to(torch.float8_e4m3fn)
    assert (oracle.round_e4m3(xs) == ref8.float().numpy()).all()
    assert (oracle.e4m3_bits(oracle.round_e4m3(xs)) == ref8.view(torch.uint8).numpy()).all()
    assert oracle.round_e4m3(np.array([1e6, -1e6], np.float32)).tolist() == [448.0, -448.0]  # saturating


def test_dequantize_special_cases(oracle):
    rng = np.random.default_rng(1)
    K, N, G = 256, 32, 64
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    ones = np.ones((K // G, N), np.float32)
    for dt in ("bf16", "fp16"):
        assert (oracle.dequantize(q, ones, None, G, dt) == q).all()                    # scale 1 -> exact ints
        s = oracle.round_to(rng.uniform(0.001, 0.1, (K // G, N)).astype(np.float32), dt)
        zero = np.zeros_like(s)
        assert (oracle.dequantize(q, s, None, G, dt) == oracle.dequantize(q, s, zero, G, dt)).all()
        # per-channel == groupwise with one group spanning K
        assert (oracle.dequantize(q, s[0], None, 0, dt) == oracle.dequantize(q, s[:1], None, K, dt)).all()
    # fp16: single rounding of the exact value; a case where rounding the product first would differ
    s = np.array([[np.float32(np.float16(0.1))]]); z = np.array([[np.float32(np.float16(0.05))]])
    qq = np.array([[7]], np.int8)
    exact = 7 * float(s[0, 0]) + float(z[0, 0])
    assert oracle.dequantize(qq, s, z, 1, "fp16")[0, 0] == np.float32(np.float16(exact))


def test_matmul_ref_properties(oracle):
    rng = np.random.default_rng(2)
    K, N, G, M = 128, 32, 64, 3
    q, s, z = oracle.make_w4_groupwise_asym(K, N, G, 4, "bf16")
    a = oracle.make_activations(M, K, 5, "bf16")
    base = oracle.woq_matmul_ref(a, q, s, z, group_size=G)
    # identity activation recovers the dequantized weight
    eye = np.eye(K, dtype=np.float32)
    assert (oracle.woq_matmul_ref(eye, q, s, z, group_size=G) == oracle.dequantize(q, s, z, G, "bf16")).all()
    # all-ones activation = column sums; alpha linearity; bias is additive
    assert np.allclose(oracle.woq_matmul_ref(np.ones((1, K), np.float32), q, s, z, group_size=G)[0],
                       oracle.dequantize(q, s, z, G, "bf16").astype(np.float64).sum(0))
    assert np.allclose(oracle.woq_matmul_ref(a, q, s, z, group_size=G, alpha=0.5), 0.5 * base)
    b = rng.standard_normal(N).astype(np.float32)
    assert np.allclose(oracle.woq_matmul_ref(a, q, s, z, bias=b, group_size=G), base + b)
    # pre-quant scale == pre-multiplying the activation (in the activation type)
    p = oracle.round_bf16(rng.uniform(0.5, 2, K).astype(np.float32))
    assert (oracle.woq_matmul_ref(a, q, s, z, pre_quant_scale=p, group_size=G)
            == oracle.woq_matmul_ref(oracle.round_bf16(a * p), q, s, z, group_size=G)).all()
    # zero folding rule: (8 - zp) * scale
    assert oracle.fold_zero_points(np.array([3.0]), np.array([0.5]), 4, False, "bf16")[0] == 2.5
    assert oracle.fold_zero_points(np.array([3.0]), np.array([0.5]), 4, True, "bf16")[0] == 2.0
    assert oracle.fold_zero_points(np.array([100.0]), np.array([0.5]), 8, False, "bf16")[0] == 14.0


def test_c_dequant_matmul_matches_numpy(oracle, oracle_c):
    K, N, G, M = 128, 48, 64, 2
    q, s, z = oracle.make_w4_groupwise_asym(K, N, G, 9, "bf16")
    a = oracle.make_activations(M, K, 10, "bf16")
    out = np.zeros((M, N), np.float32)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    oracle_c.oracle_dequant_matmul_f32(vp(out), vp(a), vp(q), vp(s), vp(z), ctypes.c_size_t(M), ctypes.c_size_t(N),
                                       ctypes.c_size_t(K), ctypes.c_size_t(G))
    w = q.astype(np.float32) * np.repeat(s, G, 0) + np.repeat(z, G, 0)
    assert oracle.max_rel_err(out, a.astype(np.float64) @ w.astype(np.float64)) < 1e-5


def test_grouped_matmul_ref_is_a_per_row_expert_gather(oracle):
    """The grouped reference against an independent formulation: every row multiplied with the
    dequantized matrix of the expert that owns it (rows -> expert by searching the prefix sums)."""
    rng = np.random.default_rng(5)
    E, K, N = 4, 128, 32
    rows = [3, 0, 5, 2]
    total = np.cumsum(np.asarray(rows, np.int64))
    q = rng.integers(-8, 8, size=(E, K, N)).astype(np.int8)
    s = oracle.round_to(rng.uniform(0.01, 0.1, (E, K // 64, N)).astype(np.float32), "fp16")
    z = oracle.round_to(rng.standard_normal((E, K // 64, N)).astype(np.float32) * 0.1, "fp16")
    b = oracle.round_to(rng.standard_normal((E, N)).astype(np.float32), "fp16")
    a = oracle.round_to(rng.standard_normal((10, K)).astype(np.float32), "fp16")
    got = oracle.grouped_matmul_ref(a, q, s, z, b, total, 64, "fp16")
    owner = np.searchsorted(total, np.arange(10), side="right")
    w = np.stack([oracle.dequantize(q[e], s[e], z[e], 64, "fp16") for e in range(E)]).astype(np.float64)
    want = np.einsum("rk,rkn->rn", a.astype(np.float64), w[owner]) + b[owner]
    assert np.allclose(got, want, rtol=0, atol=1e-9)


def test_activation_ref_known_values(oracle):
    """Closed-form points of the activation restatement: silu(0) = 0, silu(x) - silu(-x) = x,
    gelu(x) - gelu(-x) = x, gelu(1) = Phi(1), relu; the gated forms take value = first half."""
    x = np.array([-3.0, -1.0, 0.0, 0.5, 1.0, 4.0])
    silu, gelu = oracle.activation_ref(x, "silu"), oracle.activation_ref(x, "gelu")
    assert silu[2] == 0 and np.allclose(silu - oracle.activation_ref(-x, "silu"), x)
    assert np.allclose(gelu - oracle.activation_ref(-x, "gelu"), x)
    assert abs(gelu[4] - 0.8413447460685429) < 1e-12 and abs(silu[4] - 0.7310585786300049) < 1e-12
    assert (oracle.activation_ref(x, "relu") == np.maximum(x, 0)).all()
    assert (oracle.activation_ref(x, "identity") == x).all()
    pair = np.array([[2.0, 3.0, 1.0, -1.0]])  # value (2, 3), gate (1, -1)
    assert np.allclose(oracle.activation_ref(pair, "swiglu"), [[2.0 * silu[4], 3.0 * silu[1]]])
    assert np.allclose(oracle.activation_ref(pair, "geglu"), [[2.0 * gelu[4], 3.0 * gelu[1]]])


def test_rmsnorm_ref_against_torch_and_closed_forms(oracle):
    """rmsnorm_ref: a row of equal values c normalises to sign(c) * gamma / sqrt(1 + eps / c^2); scaling
    a row leaves the result unchanged (eps = 0); and it agrees with torch's float32 rms_norm rounded
    to the type, up to the last place."""
    import torch
    k = 256
    gamma = oracle.round_to(np.linspace(0.5, 1.5, k).astype(np.float32), "bf16")
    x = np.full((1, k), -2.0, np.float32)
    want = oracle.round_to((-gamma / np.sqrt(1.0 + 1e-5 / 4.0)).astype(np.float32), "bf16")
    assert (oracle.rmsnorm_ref(x, gamma, 1e-5, "bf16") == want).all()
    rng = np.random.default_rng(2)
    x = oracle.round_to(rng.standard_normal((4, k)).astype(np.float32), "fp16")
    assert (oracle.rmsnorm_ref(x, gamma, 0.0, "fp16") == oracle.rmsnorm_ref(4.0 * x, gamma, 0.0, "fp16")).all()
    beta = oracle.round_to(rng.standard_normal(k).astype(np.float32), "fp16")
    t = torch.nn.functional.rms_norm(torch.from_numpy(x), (k,), torch.from_numpy(gamma), 1e-5) + torch.from_numpy(beta)
    want = t.to(torch.float16).float().numpy()
    got = oracle.rmsnorm_ref(x, gamma, 1e-5, "fp16", beta)
    assert (got == want).mean() > 0.99 and np.abs(got - want).max() <= 2.0 ** -10 * np.abs(want).max()
