"""GPU parity of the W4A8 path (fp8 e4m3 activations x int4 weights, fp8 MFMA) against the oracle:
both operands rounded to e4m3, float accumulation, alpha in the epilogue.  Tolerance 1e-2 of
max|ref| as for the other kernels (the oracle rounds exactly like the kernel, so observed errors
are output-rounding only)."""
import numpy as np
import pytest
import torch

from _util import preprocess, to_dev, TORCH_DT

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _run(pkg, oracle, dev, prob, M, K, N, out_dtype, zeros=None, bias=None, direct_fp8=False, regime=0, group=128):
    F = pkg.functional
    w = preprocess(pkg, oracle, prob["q"], 4, torch.float8_e4m3fn).to(dev)
    scales = to_dev(prob["scales"], "fp16", dev)
    algo = F.FP8_ALPHA | (F.ZERO if zeros is not None else 0) | (F.BIAS if bias is not None else 0)
    z = None if zeros is None else to_dev(zeros, "fp16", dev)
    b = None if bias is None else to_dev(bias, out_dtype, dev)
    if direct_fp8:
        a8 = oracle.apply_per_channel_scale(prob["act"], prob["pre_quant_scale"], out_dtype, "fp8")
        act = torch.from_numpy(a8).to(dev).to(torch.float8_e4m3fn)
        out = F.woq_matmul_raw(act, None, w, scales, z, b, n=N, k=K, group_size=group, quant_algo=algo,
                               alpha=prob["alpha"], out_dtype=TORCH_DT[out_dtype], regime=regime)
        ref = oracle.woq_matmul_ref(a8, prob["q"], prob["scales"], zeros, bias, None, prob["alpha"], group, out_dtype,
                                    w4a8=True)
    else:
        algo |= F.PRE_QUANT_SCALE
        out = F.woq_matmul_raw(to_dev(prob["act"], out_dtype, dev), to_dev(prob["pre_quant_scale"], out_dtype, dev), w,
                               scales, z, b, n=N, k=K, group_size=group, quant_algo=algo, alpha=prob["alpha"],
                               out_dtype=TORCH_DT[out_dtype], regime=regime)
        ref = oracle.woq_matmul_ref(prob["act"], prob["q"], prob["scales"], zeros, bias, prob["pre_quant_scale"],
                                    prob["alpha"], group, out_dtype, w4a8=True)
    torch.cuda.synchronize()
    # floor of the per-column norm: the expected output magnitude of each column for these operands
    a8 = oracle.apply_per_channel_scale(prob["act"], prob["pre_quant_scale"], out_dtype, "fp8")
    prob["_col_floor"] = oracle.column_magnitude(a8, oracle.dequantize(prob["q"], prob["scales"], zeros, group, "fp8"),
                                                 prob["alpha"])
    return out.float().cpu().numpy(), ref


def _perr(oracle, out, ref, prob):
    """global norm and per-output-column norm, whichever is larger"""
    return max(oracle.max_rel_err(out, ref), oracle.max_col_rel_err(out, ref, prob["_col_floor"]))


@pytest.mark.parametrize("out_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M", [1, 16, 256, 300])
@pytest.mark.parametrize("direct", [False, True])
def test_w4a8_awq_style(pkg, oracle, dev, out_dtype, M, direct):
    """The benchmark's W4A8 configuration at test size: symmetric int4 g128, smoothing vector,
    per-tensor scales folded into alpha; activations given as 16-bit + smoothing vector (the
    reference plugin's input) or directly as fp8."""
    K, N = 1024, 384
    prob = oracle.make_w4a8_problem(M, K, N, seed=M, out_dtype=out_dtype)
    out, ref = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, direct_fp8=direct)
    assert _perr(oracle, out, ref, prob) < TOL


def test_w4a8_zeros_and_bias(pkg, oracle, dev):
    M, K, N = 130, 512, 272
    prob = oracle.make_w4a8_problem(M, K, N, seed=3, out_dtype="bf16")
    rng = np.random.default_rng(4)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
    out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=zeros, bias=bias)
    assert _perr(oracle, out, ref, prob) < TOL


@pytest.mark.parametrize("M,K,N", [(17, 4096, 256), (100, 2048, 272), (128, 1024, 512), (200, 2048, 1040), (520, 512, 256)])
def test_w4a8_tile_heights_and_split_k(pkg, oracle, dev, M, K, N):
    """64 / 128 / 256-row tiles, K split across workgroups (with a shorter last slice) and not,
    N off the 256-column tile, zeros and bias (bias is added by the finish pass when K is split)."""
    prob = oracle.make_w4a8_problem(M, K, N, seed=M + N, out_dtype="bf16")
    rng = np.random.default_rng(M)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
    for z in (None, zeros):
        out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=bias)
        assert _perr(oracle, out, ref, prob) < TOL, (M, K, N, z is not None)


def test_w4a8_identity_recovers_e4m3_weight(pkg, oracle, dev):
    """Identity activation (exact in e4m3) returns the e4m3-rounded dequantized weight times alpha."""
    K, N = 256, 128
    rng = np.random.default_rng(6)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    s = oracle.round_f16(np.exp(rng.uniform(-2, 3, (K // 128, N))).astype(np.float32))
    prob = dict(q=q, scales=s, act=np.eye(K, dtype=np.float32), pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
    out, _ = _run(pkg, oracle, dev, prob, K, K, N, "fp16", direct_fp8=True)
    w8 = oracle.dequantize(q, s, None, 128, "fp8")
    assert (out == oracle.round_f16(w8)).all()


STREAM, GEMM = 1, 2


def _launch(pkg):
    return (pkg._lib.lib.woq_last_launch() or b"").decode()


@pytest.mark.parametrize("M,K,N,with_zeros", [(2250, 512, 7680, False), (4000, 1024, 8192, True), (2304, 768, 8192, False)])
def test_w4a8_persistent_tile_loop(pkg, oracle, dev, woq_env, M, K, N, with_zeros):
    """More 256 x 256 tiles than CUs, bf16 output, no bias: one workgroup per CU walks its tiles (the
    next tile's first weights and A tile requested in the current tile's last two steps, the outputs
    stored between the next tile's first matrix instructions).  The bits of the one-tile-per-workgroup
    launch, which in turn meets the oracle's bar; rows ragged against the tile."""
    prob = oracle.make_w4a8_problem(M, K, N, seed=M + K, out_dtype="bf16")
    rng = np.random.default_rng(N)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32)) if with_zeros else None
    out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=zeros, direct_fp8=True, regime=GEMM)
    assert "persistent=1" in _launch(pkg), _launch(pkg)
    woq_env(WOQ_GEMM_PERSIST="0")
    plain, _ = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=zeros, direct_fp8=True, regime=GEMM)
    assert "persistent=0" in _launch(pkg), _launch(pkg)
    assert (out.view(np.uint32) == plain.view(np.uint32)).all()
    assert _perr(oracle, out, ref, prob) < TOL


@pytest.mark.parametrize("out_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("direct", [False, True])
def test_w4a8_streaming_kernel(pkg, oracle, dev, out_dtype, M, direct):
    """Decode sizes on the weight-streaming W4A8 kernel (forced, and what AUTO picks for M <= 16):
    same oracle, same bar; the GEMM kernel on the same inputs agrees to float32 summation order."""
    K, N = 1024, 384
    prob = oracle.make_w4a8_problem(M, K, N, seed=40 + M, out_dtype=out_dtype)
    out, ref = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, direct_fp8=direct, regime=STREAM)
    assert _perr(oracle, out, ref, prob) < TOL
    auto, _ = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, direct_fp8=direct)
    assert (auto == out).all()
    gemm, _ = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, direct_fp8=direct, regime=GEMM)
    assert oracle.max_rel_err(gemm, out) < 2e-3


@pytest.mark.parametrize("M,K,N", [(1, 128, 16), (5, 640, 272), (16, 2176, 1040), (2, 8192, 48), (9, 4096, 4112)])
def test_w4a8_streaming_shapes(pkg, oracle, dev, M, K, N):
    """Fewer tile rows than wavefronts, a last column group that is only partly there, long K,
    both launch shapes; with and without zeros, bias."""
    prob = oracle.make_w4a8_problem(M, K, N, seed=M + N, out_dtype="bf16")
    rng = np.random.default_rng(M)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
    for z in (None, zeros):
        out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=bias, regime=STREAM)
        assert _perr(oracle, out, ref, prob) < TOL, (M, K, N, z is not None)


@pytest.mark.parametrize("shape", ["1,8,2,0", "1,16,2,0", "2,8,2,0", "2,8,3,0", "2,4,4,0", "4,8,2,0", "1,8,2,1", "1,8,4,1",
                                   "2,8,2,1", "2,4,4,1", "4,8,2,1", "1,8,2,2", "1,8,4,2", "2,8,2,2",
                                   "1,8,2,3", "2,8,2,3", "2,8,3,3", "2,4,4,3", "4,8,2,3"])
def test_w4a8_streaming_launch_shapes(pkg, oracle, dev, woq_env, shape):
    """Every instantiated launch shape (strips per wavefront, wavefronts, tile rows in flight, LDS mode:
    0 nothing staged, 1 activations, 2 activations + group scales and zeros, 3 scales and zeros only), whatever
    the table would pick: K with a tile-row count that no shape divides, N that ends inside a group."""
    woq_env(WOQ_STREAM_SHAPE=shape)
    M, K, N = 7, 2176, 272
    prob = oracle.make_w4a8_problem(M, K, N, seed=17, out_dtype="fp16")
    rng = np.random.default_rng(18)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    for z in (None, zeros):
        out, ref = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=STREAM)
        assert _perr(oracle, out, ref, prob) < TOL, (shape, z is not None)


@pytest.mark.parametrize("regime", [STREAM, GEMM])
def test_w4a8_saturating_scales(pkg, oracle, dev, regime):
    """Group scales (and zeros) large enough that dequantized weights pass +-448: the conversion
    saturates as the oracle's e4m3 rounding does, in both kernels, bit for bit.  A second call with
    a large alpha overflows fp16: those outputs are infinite, not clamped."""
    M, K, N = 4, 512, 64
    rng = np.random.default_rng(21)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    s = oracle.round_f16(rng.uniform(40, 120, (K // 128, N)).astype(np.float32))
    s[0, :8] = 0.01  # some columns stay far from saturation within the same call
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 300).astype(np.float32))
    rows = [3, 130, 300, 511]
    act = np.zeros((M, K), np.float32)
    act[np.arange(M), rows] = 1.0
    for z in (None, zeros):
        w8 = oracle.dequantize(q, s, z, 128, "fp8")
        assert np.abs(w8).max() == 448.0
        prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
        out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=regime)
        assert (out == oracle.round_f16(w8[rows])).all()
        prob["alpha"] = 1024.0
        out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=regime)
        expect = oracle.round_f16(1024.0 * w8[rows])
        assert np.isinf(expect).any()
        assert (out == expect).all()


def test_w4a8_streaming_one_hot_rows_recover_e4m3_weight(pkg, oracle, dev):
    """One-hot activation rows (exact in e4m3): row r of the output is row k_r of the e4m3-rounded
    dequantized weight, bit for bit - with and without zero-points."""
    M, K, N = 16, 1024, 256
    rng = np.random.default_rng(8)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    s = oracle.round_f16(np.exp(rng.uniform(-2, 3, (K // 128, N))).astype(np.float32))
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    rows = rng.choice(K, size=M, replace=False)
    act = np.zeros((M, K), np.float32)
    act[np.arange(M), rows] = 1.0
    prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
    for z in (None, zeros):
        out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=STREAM)
        w8 = oracle.dequantize(q, s, z, 128, "fp8")
        assert (out == oracle.round_f16(w8[rows])).all()


def test_w4a8_streaming_kernel_refuses_more_than_32_rows(pkg, oracle, dev):
    prob = oracle.make_w4a8_problem(33, 256, 64, seed=1, out_dtype="bf16")
    with pytest.raises(RuntimeError, match="unsupported m"):
        _run(pkg, oracle, dev, prob, 33, 256, 64, "bf16", direct_fp8=True, regime=STREAM)


@pytest.mark.parametrize("out_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,K,N", [(17, 1024, 384), (32, 2176, 1040), (24, 4096, 4112), (31, 512, 10240 + 16),
                                   (20, 8192, 48), (32, 256, 16)])
def test_w4a8_streaming_two_row_tiles(pkg, oracle, dev, out_dtype, M, K, N):
    """17 ... 32 rows on the streaming kernel (two 16-row tiles per wavefront, activations from registers;
    one, two and four strips per wavefront by the built-in rule, a last column group that is only partly
    there, fewer tile rows than wavefronts): same oracle, same bar, with and without zeros and bias; what
    AUTO picks here; the GEMM kernel on the same inputs agrees to float32 summation order."""
    prob = oracle.make_w4a8_problem(M, K, N, seed=M + N, out_dtype=out_dtype)
    rng = np.random.default_rng(M)
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
    for z, b in ((None, None), (zeros, bias)):
        out, ref = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, zeros=z, bias=b, regime=STREAM)
        assert "stream w4a8 mt=2" in _launch(pkg), _launch(pkg)
        assert _perr(oracle, out, ref, prob) < TOL, (M, K, N, z is not None)
        gemm, _ = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, zeros=z, bias=b, regime=GEMM)
        assert oracle.max_rel_err(gemm, out) < 2e-3
    auto, _ = _run(pkg, oracle, dev, prob, M, K, N, out_dtype, zeros=zeros, bias=bias)
    expect_stream = not (M > (19 if N <= 4096 else 30) and K >= 2 * N)
    assert ("stream w4a8 mt=2" in _launch(pkg)) == expect_stream, _launch(pkg)
    if expect_stream:
        assert (auto == out).all()


def test_w4a8_streaming_two_row_tiles_one_hot_rows(pkg, oracle, dev):
    """One-hot activation rows through the two-tile variant: row r of the output is row k_r of the
    e4m3-rounded dequantized weight, bit for bit - with and without zero-points."""
    M, K, N = 32, 1024, 528
    rng = np.random.default_rng(9)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    s = oracle.round_f16(np.exp(rng.uniform(-2, 3, (K // 128, N))).astype(np.float32))
    zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
    rows = rng.choice(K, size=M, replace=False)
    act = np.zeros((M, K), np.float32)
    act[np.arange(M), rows] = 1.0
    prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
    for z in (None, zeros):
        out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=STREAM)
        w8 = oracle.dequantize(q, s, z, 128, "fp8")
        assert (out == oracle.round_f16(w8[rows])).all()


# the reference's own grid for e4m3 activations with group sizes above 128
# (tests/quantization/test_weight_only_groupwise_quant_matmul.py:429-455: m, n, k, dtype, pre-quant scale,
# zeros, bias, group size - a group may be longer than K, or leave a shorter last group)
_FLEX_GRID = [(32, 1024, 128, "fp16", True, True, 128), (32, 1024, 128, "fp16", True, True, 256),
              (32, 1024, 256, "fp16", True, False, 384), (32, 1024, 256, "bf16", True, True, 384),
              (32, 2048, 1024, "fp16", False, True, 512), (64, 2048, 2048, "bf16", False, False, 640),
              (64, 2048, 2048, "fp16", False, False, 640),
              # beyond the reference's grid: decode rows, long K with a shorter last group, staged scales
              (1, 512, 8192, "bf16", True, True, 384), (7, 272, 8192 + 128, "fp16", True, False, 640),
              (16, 4112, 4096, "bf16", False, True, 256), (300, 528, 2304, "bf16", True, True, 512)]


@pytest.mark.parametrize("m,n,k,dtype,has_zero,has_bias,group", _FLEX_GRID)
def test_w4a8_flexible_group_sizes(pkg, oracle, dev, m, n, k, dtype, has_zero, has_bias, group):
    """Group sizes that are multiples of 128 (what the reference's Hopper launcher accepts for e4m3
    activations, launchers/fpA_intB_launcher_sm90.inl:190-198) in both regimes and as AUTO picks, 16-bit
    activations with the smoothing vector as in the reference's test: the tables hold ceil(k / group) rows."""
    rng = np.random.default_rng(m * 7 + n + k + group)
    rows = -(-k // group)
    q = rng.integers(-8, 8, size=(k, n)).astype(np.int8)
    s = oracle.round_f16(np.exp(rng.uniform(-3, 0, (rows, n))).astype(np.float32))
    zeros = oracle.round_f16((rng.standard_normal((rows, n)) * 2).astype(np.float32)) if has_zero else None
    bias = oracle.round_to(rng.standard_normal(n).astype(np.float32), dtype) if has_bias else None
    prob = dict(q=q, scales=s, alpha=0.37,
                act=oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), dtype),
                pre_quant_scale=oracle.round_to(rng.uniform(0.5, 2.0, k).astype(np.float32), dtype))
    regimes = [0, GEMM] + ([STREAM] if m <= 32 else [])
    outs = {}
    for regime in regimes:
        for direct in (False, True):
            out, ref = _run(pkg, oracle, dev, prob, m, k, n, dtype, zeros=zeros, bias=bias, direct_fp8=direct,
                            regime=regime, group=group)
            assert _perr(oracle, out, ref, prob) < TOL, (regime, direct, _launch(pkg))
            outs[regime, direct] = out
        # the smoothing pass in front of the kernel and fp8 activations handed over directly: the same bits
        assert (outs[regime, False] == outs[regime, True]).all()


def test_w4a8_flexible_groups_one_hot_rows(pkg, oracle, dev):
    """One-hot rows return the e4m3-rounded dequantized weight rows bit for bit with groups of 384 (rows of
    different groups inside one 128-row tile row never occur, rows of one group span three): every
    tile row reads its group's table row, in both kernels."""
    M, K, N, G = 32, 1280, 272, 384
    rng = np.random.default_rng(12)
    q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    rows_g = -(-K // G)
    s = oracle.round_f16(np.exp(rng.uniform(-2, 3, (rows_g, N))).astype(np.float32))
    zeros = oracle.round_f16((rng.standard_normal((rows_g, N)) * 20).astype(np.float32))
    rows = np.concatenate([[0, 127, 128, 383, 384, 767, 768, 1151, 1152, 1279],
                           rng.choice(K, size=M - 10, replace=False)])
    act = np.zeros((M, K), np.float32)
    act[np.arange(M), rows] = 1.0
    prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
    for regime in (STREAM, GEMM):
        for z in (None, zeros):
            out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, regime=regime, group=G)
            w8 = oracle.dequantize(q, s, z, G, "fp8")
            assert (out == oracle.round_f16(w8[rows])).all(), (regime, z is not None)


@pytest.mark.parametrize("shape", ["4,8", "8,8", "16,8", "4,4", "8,4", "16,4", "14,4", "16,7"])
@pytest.mark.parametrize("K,N", [(2176, 272), (128, 16), (8192, 48), (14336, 32)])
def test_w4a8_row_kernel_forced(pkg, oracle, dev, woq_env, shape, K, N):
    """The W4A8 row kernel (one workgroup per strip, no staging pass, weights converted through the table of
    their (group, column)), forced through WOQ_ROW_SHAPE for one to four rows: several passes over K, wavefronts
    without tiles, with and without zeros; 16-bit activations through the smoothing pass and e4m3 activations
    handed over directly give the same bits.  A shape whose tiles x rows exceed the 16 MFMA rows is refused
    and the call runs on the strip-group kernel."""
    tiles = int(shape.split(",")[1])
    for M in (1, 2, 3, 4):
        fits = tiles * (1 if M == 1 else (2 if M == 2 else 4)) <= 16
        prob = oracle.make_w4a8_problem(M, K, N, seed=K + N + M, out_dtype="bf16")
        rng = np.random.default_rng(M + K)
        zeros = oracle.round_f16((rng.standard_normal((K // 128, N)) * 20).astype(np.float32))
        bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
        for z, b in ((None, None), (zeros, bias)):
            woq_env(WOQ_ROW_SHAPE=shape)
            out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, regime=STREAM)
            assert ("stream row w4a8" in _launch(pkg)) == fits, (M, _launch(pkg))
            assert _perr(oracle, out, ref, prob) < TOL, (shape, M, z is not None)
            direct, _ = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, direct_fp8=True, regime=STREAM)
            assert (direct == out).all()
            woq_env(WOQ_ROW_SHAPE="0")
            other, _ = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, regime=STREAM)
            assert "stream w4a8" in _launch(pkg), _launch(pkg)
            assert oracle.max_rel_err(other, out) < 2e-3


def test_w4a8_row_kernel_rule_and_exact_rows(pkg, oracle, dev):
    """One to four rows with K up to 4096, or up to 8192 on at most 1024 strips (and two to four rows of a narrow
    matrix with K = 14336), run on the row kernel; one-hot
    rows and saturating scales come back as the e4m3-rounded dequantized weight rows, bit for bit (the table is
    built with the arithmetic form's own FMA and saturating conversion), also with groups of 256."""
    rng = np.random.default_rng(31)
    for M, K, N, G, want in ((1, 4096, 272, 128, "waves=8 tpw=4 passes=1 rows=1"), (4, 1024, 64, 128, "waves=8 tpw=4 passes=1 rows=4"),
                             (2, 8192, 48, 256, "waves=16 tpw=4 passes=1 rows=2"), (3, 8192, 16400, 128, None),
                             (1, 14336, 32, 128, None), (5, 1024, 64, 128, None),
                             (2, 14336, 32, 128, "waves=16 tpw=7 passes=1 rows=2"), (4, 14336, 32, 256, "waves=14 tpw=4 passes=2 rows=4")):
        rows_g = -(-K // G)
        q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
        s = oracle.round_f16(np.exp(rng.uniform(-2, 4.5, (rows_g, N))).astype(np.float32))  # up to 90: saturates
        zeros = oracle.round_f16((rng.standard_normal((rows_g, N)) * 100).astype(np.float32))
        hot = rng.choice(K, size=M, replace=False)
        act = np.zeros((M, K), np.float32)
        act[np.arange(M), hot] = 1.0
        prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
        for z in (None, zeros):
            out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, group=G)
            if want is None:
                assert "stream row w4a8" not in _launch(pkg), (M, K, N, _launch(pkg))
            else:
                assert "stream row w4a8 " + want in _launch(pkg), (M, K, N, _launch(pkg))
            w8 = oracle.dequantize(q, s, z, G, "fp8")
            assert np.abs(w8).max() == 448.0
            assert (out == oracle.round_f16(w8[hot])).all(), (M, K, N, z is not None)


@pytest.mark.parametrize("shape", ["8,1,2", "8,2,2", "8,4,2", "16,2,2", "4,1,4"])
@pytest.mark.parametrize("K,N,G", [(2048, 272, 128), (1408, 1040, 128), (128, 16, 128), (4096 + 128, 528, 256)])
def test_w4a8_multirow_kernel_forced(pkg, oracle, dev, woq_env, shape, K, N, G):
    """The W4A8 multi-row kernel (a workgroup owns a few strips, its wavefronts split K and request a pass at
    once, no staging), forced through WOQ_ROWS_SHAPE for 1 ... 16 rows: several passes, wavefronts without tile
    rows, a strip count the strips per workgroup do not divide, groups of two tile rows with a shorter last one;
    zeros and bias; 16-bit activations through the smoothing pass and e4m3 activations handed over directly give
    the same bits, and the staged kernel agrees."""
    rows_g = -(-K // G)
    for M in (1, 3, 8, 13, 16):
        prob = oracle.make_w4a8_problem(M, K, N, seed=K + N + M, out_dtype="bf16")
        rng = np.random.default_rng(M + K)
        prob["scales"] = oracle.round_f16(np.exp(rng.uniform(-3, 0, (rows_g, N))).astype(np.float32))
        zeros = oracle.round_f16((rng.standard_normal((rows_g, N)) * 2).astype(np.float32))
        bias = oracle.round_bf16(rng.standard_normal(N).astype(np.float32))
        for z, b in ((None, None), (zeros, bias)):
            woq_env(WOQ_ROWS_SHAPE=shape, WOQ_ROW_SHAPE="0")
            out, ref = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, regime=STREAM, group=G)
            assert "stream multirow w4a8" in _launch(pkg), (M, _launch(pkg))
            assert _perr(oracle, out, ref, prob) < TOL, (shape, M, z is not None)
            direct, _ = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, direct_fp8=True, regime=STREAM, group=G)
            assert (direct == out).all()
            woq_env(WOQ_ROWS_SHAPE="0", WOQ_ROW_SHAPE="0")
            other, _ = _run(pkg, oracle, dev, prob, M, K, N, "bf16", zeros=z, bias=b, regime=STREAM, group=G)
            assert "stream w4a8" in _launch(pkg), _launch(pkg)
            assert oracle.max_rel_err(other, out) < 2e-3


def test_w4a8_multirow_kernel_rule_and_exact_rows(pkg, oracle, dev):
    """From five rows on, matrices with K up to 4096 (and mid-width ones with K up to 8192 from ten rows) run on
    the multi-row kernel; one-hot rows and saturating scales come back as the e4m3-rounded dequantized weight
    rows, bit for bit, in fp16 output."""
    rng = np.random.default_rng(37)
    for M, K, N, G, want in ((8, 4096, 4096, 128, "waves=8 ns=1 tpw=2"), (16, 2048, 6144 + 16, 128, "waves=8 ns=2 tpw=2"),
                             (6, 1024, 16384, 128, "waves=8 ns=2 tpw=2"), (10, 1024, 16384 + 48, 256, "waves=8 ns=4 tpw=2"),
                             (12, 8192, 10240, 128, "waves=8 ns=4 tpw=2"), (12, 1024, 16384, 128, None),
                             (8, 8192, 10240, 128, None), (4, 4096, 4096, 128, None), (16, 8192 + 128, 256, 128, None)):
        rows_g = -(-K // G)
        q = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
        s = oracle.round_f16(np.exp(rng.uniform(-2, 4.5, (rows_g, N))).astype(np.float32))  # up to 90: saturates
        zeros = oracle.round_f16((rng.standard_normal((rows_g, N)) * 100).astype(np.float32))
        hot = rng.choice(K, size=M, replace=False)
        act = np.zeros((M, K), np.float32)
        act[np.arange(M), hot] = 1.0
        prob = dict(q=q, scales=s, act=act, pre_quant_scale=np.ones(K, np.float32), alpha=1.0)
        for z in (None, zeros):
            out, _ = _run(pkg, oracle, dev, prob, M, K, N, "fp16", zeros=z, direct_fp8=True, group=G)
            if want is None:
                assert "stream multirow w4a8" not in _launch(pkg), (M, K, N, _launch(pkg))
            else:
                assert "stream multirow w4a8 " + want in _launch(pkg), (M, K, N, _launch(pkg))
            w8 = oracle.dequantize(q, s, z, G, "fp8")
            assert np.abs(w8).max() == 448.0
            assert (out == oracle.round_f16(w8[hot])).all(), (M, K, N, z is not None)
