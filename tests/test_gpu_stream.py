"""GPU parity of the weight-streaming kernel (decode GEMV / skinny M) against the CPU oracle,
through the C ABI.  Tolerance: max|out - ref| / max|ref| <= 1e-2 against the float64-accumulated
dequantize-then-matmul reference (the bar the benchmark definition states); observed errors are
~1e-3 (one rounding of the output to fp16/bf16)."""
import numpy as np
import pytest
import torch

from _util import parity_err, random_problem, reference, run_product, preprocess, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-2
STREAM = 1


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 64, 128])
@pytest.mark.parametrize("M", [1, 3, 16])
def test_stream_basic(pkg, oracle, dev, dtype, bits, group, M):
    p = random_problem(oracle, M, 512, 128, bits, group, dtype, seed=M + bits + group)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("zero,bias,pqs", [(1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 1, 0), (1, 0, 1), (0, 1, 1), (1, 1, 1)])
@pytest.mark.parametrize("bits,group", [(4, 64), (4, 128), (8, 64), (8, 128)])
def test_stream_optional_inputs(pkg, oracle, dev, dtype, zero, bias, pqs, bits, group):
    """The eight (act_scale, zero, bias) variants of the reference dispatcher (kernelDispatcher.h:101-143)."""
    p = random_problem(oracle, 5, 1024, 256, bits, group, dtype, zero, bias, pqs, seed=zero * 4 + bias * 2 + pqs)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("M", [1, 2, 4, 7, 8, 15, 16, 17, 32, 33, 64, 100, 128])
def test_stream_m_sweep(pkg, oracle, dev, M):
    p = random_problem(oracle, M, 1024, 1024, 4, 128, "bf16", zero=True, seed=M)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("K,N", [(64, 1024), (128, 16), (192, 48), (320, 2048), (1024, 1040), (4096, 4096)])
def test_stream_ragged_shapes(pkg, oracle, dev, K, N):
    """K that is not a multiple of the 128-row weight tile (padded tail), N not a multiple of 128
    (partly empty XCD chunks), and the reference's own small test shapes."""
    for bits, group in [(4, 64), (8, 64), (4, 0)]:
        p = random_problem(oracle, 3, K, N, bits, group, "bf16", zero=group != 0, seed=K + N)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
        assert err < TOL, (bits, group, err)


def test_stream_identity_recovers_weight(pkg, oracle, dev):
    """The reference's conversion test (test_weight_only_quant_matmul.py:147-164): an identity
    activation pulls the dequantized weight out of the kernel.  Here the result must equal the
    oracle's dequantize to within one output rounding of q*s+z computed in float32."""
    K, N = 128, 64
    p = random_problem(oracle, K, K, N, 4, 128, "bf16", zero=True, seed=3)
    p["act"] = np.eye(K, dtype=np.float32)
    out = run_product(pkg, oracle, dev, p, STREAM)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 128, "bf16")
    assert oracle.max_rel_err(out, w) < 4e-3


def test_stream_all_ones_and_zeros(pkg, oracle, dev):
    p = random_problem(oracle, 2, 512, 128, 4, 128, "bf16", zero=True, seed=8)
    p["act"] = np.stack([np.ones(512, np.float32), np.zeros(512, np.float32)])
    out = run_product(pkg, oracle, dev, p, STREAM)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 128, "bf16").astype(np.float64)
    assert oracle.max_rel_err(out[0], w.sum(0)) < TOL
    assert (out[1] == 0).all()


def test_stream_zero_none_equals_zero_zero_and_is_deterministic(pkg, oracle, dev):
    p = random_problem(oracle, 4, 1024, 256, 4, 128, "bf16", seed=11)
    a = run_product(pkg, oracle, dev, p, STREAM)
    p2 = dict(p, zeros=np.zeros_like(p["scales"]))
    b = run_product(pkg, oracle, dev, p2, STREAM)
    assert (a == b).all()
    assert (a == run_product(pkg, oracle, dev, p, STREAM)).all()       # fixed reduction order


def test_stream_large_activations_offset_cancellation(pkg, oracle, dev):
    """The kernel removes the (BASE + 8) operand offset with activation row sums; activations
    with a large common mean stress that cancellation."""
    for dtype in ("bf16", "fp16"):
        for bits, group in [(4, 128), (8, 0)]:
            p = random_problem(oracle, 2, 4096, 64, bits, group, dtype, seed=5)
            p["act"] = oracle.round_to(p["act"] + 3.0, dtype)
            err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
            assert err < TOL, (dtype, bits, err)


def test_m_zero_is_a_noop(pkg, dev):
    F = pkg.functional
    act = torch.zeros((0, 128), dtype=torch.bfloat16, device=dev)
    w = torch.zeros((128, 8), dtype=torch.int8, device=dev)
    s = torch.ones((1, 16), dtype=torch.bfloat16, device=dev)
    out = F.weight_only_groupwise_quant_matmul(act, None, w, s, None, None, None, 0, 128, "bfloat16")
    assert out.shape == (0, 16)


def test_functional_and_plugin_mirrors(pkg, oracle, dev):
    """Per-channel op + both plugin wrappers give the same numbers as the raw call."""
    F, P = pkg.functional, pkg.plugin
    p = random_problem(oracle, 4, 512, 256, 8, 0, "fp16", seed=21)
    w = preprocess(pkg, oracle, p["q"], 8, torch.float16).to(dev)
    act, s = to_dev(p["act"], "fp16", dev), to_dev(p["scales"], "fp16", dev)
    out = F.weight_only_quant_matmul(act, w, s, F.INT8, "float16")
    assert parity_err(oracle, out.float().cpu().numpy(), p) < TOL
    out2 = torch.empty_like(out)
    assert P.WeightOnlyQuantMatmulPlugin(torch.float16, F.INT8).enqueue([act, w, s], [out2]) == 0
    assert (out2 == out).all()
    # int4: the plugin receives N/2 packed columns and doubles them
    p4 = random_problem(oracle, 4, 512, 256, 4, 0, "fp16", seed=22)
    w4 = preprocess(pkg, oracle, p4["q"], 4, torch.float16).to(dev)
    out4 = F.weight_only_quant_matmul(to_dev(p4["act"], "fp16", dev), w4, to_dev(p4["scales"], "fp16", dev), F.INT4)
    assert out4.shape == (4, 256)
    assert parity_err(oracle, out4.float().cpu().numpy(), p4) < TOL
    # groupwise plugin: inputs in plugin order, weight typed as the activation dtype ([K, N/4] halfs)
    pg = random_problem(oracle, 3, 512, 256, 4, 128, "bf16", zero=True, bias=True, pqs=True, seed=23)
    wg = preprocess(pkg, oracle, pg["q"], 4).to(dev).view(torch.bfloat16)
    assert wg.shape == (512, 64)
    plug = P.WeightOnlyGroupwiseQuantMatmulPlugin(torch.bfloat16, F.BIAS | F.ZERO | F.PRE_QUANT_SCALE, 128)
    outg = torch.empty((3, 256), dtype=torch.bfloat16, device=dev)
    ins = [to_dev(pg[k], "bf16", dev) for k in ("act", "pqs")] + [wg] + [to_dev(pg[k], "bf16", dev) for k in
                                                                         ("scales", "zeros", "bias")]
    assert plug.enqueue(ins, [outg]) == 0
    torch.cuda.synchronize()
    assert parity_err(oracle, outg.float().cpu().numpy(), pg) < TOL


STREAM_SHAPES = ["1,8,4,1", "1,8,6,1", "1,16,4,1", "2,8,4,1", "2,4,4,1", "4,4,2,1", "4,4,4,1", "4,8,2,1", "4,8,4,1",
                 "1,8,4,0", "2,8,2,0", "4,4,2,0", "1,8,4,2", "2,8,2,2", "4,4,2,2"]


@pytest.mark.parametrize("shape", STREAM_SHAPES)
@pytest.mark.parametrize("M", [1, 5])
def test_stream_every_launch_shape(pkg, oracle, dev, woq_env, shape, M):
    """Every instantiated (strips per wavefront, wavefronts, prefetch depth, LDS staging) variant
    of the decode kernel, forced through WOQ_STREAM_SHAPE, against the oracle - including a strip
    count that is not a multiple of the strips per wavefront."""
    woq_env(WOQ_STREAM_SHAPE=shape)
    for bits, group, N in [(4, 128, 272), (8, 64, 64), (4, 0, 48)]:
        p = random_problem(oracle, M, 1280, N, bits, group, "bf16", zero=group != 0, pqs=True, seed=M + N)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
        assert err < TOL, (shape, bits, group, err)


@pytest.mark.parametrize("N", [6144, 16384])
def test_stream_wide_n_default_heuristic(pkg, oracle, dev, woq_env, N):
    """Wide outputs take the multi-strip launch shapes of the heuristic (strip-group kernel: the single-row
    kernel is switched off)."""
    woq_env(WOQ_ROW_SHAPE="0")
    p = random_problem(oracle, 1, 512, N, 4, 128, "bf16", zero=True, seed=N)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("M,K,group,bits", [(1, 8192, 64, 4), (3, 8192, 64, 4), (2, 4160, 64, 4), (5, 4096, 128, 8)])
def test_stream_long_k_staged_operands(pkg, oracle, dev, woq_env, M, K, group, bits):
    """Long K with four strips per wavefront (launch shape forced): the activations, the group scales / zeros and the
    activation row sums staged in LDS exceed what a thread keeps in registers across the weight
    prefetch (the staging tail loops run), take more than 64 KiB of LDS, and K = 4160 ends in half
    a weight tile whose scales, zeros and row sums must read as zero."""
    N = 16384
    woq_env(WOQ_STREAM_SHAPE="4,8,2,1")
    p = random_problem(oracle, M, K, N, bits, group, "bf16", zero=True, pqs=True, seed=K + M)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("M", [2, 4])
@pytest.mark.parametrize("forced", [False, True])
def test_stream_narrow_n_long_k_stages_beyond_64k(pkg, oracle, dev, woq_env, M, forced):
    """Few column groups and a long K (a down projection at M = 2..4): the activations are staged in
    LDS although they take 57 / 115 KiB (by the heuristic up to 3 rows, since one workgroup per CU
    covers the problem anyway; forced for 4)."""
    woq_env(WOQ_ROW_SHAPE="0")  # the strip-group kernel's test: the row kernel would take these
    if forced:
        woq_env(WOQ_STREAM_SHAPE="1,8,4,1")
    p = random_problem(oracle, M, 14336, 256, 4, 128, "bf16", zero=True, bias=True, seed=M)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


def test_stream_activations_too_large_for_lds(pkg, oracle, dev):
    """M x K beyond the LDS staging area falls back to register-held activation fragments."""
    p = random_problem(oracle, 16, 4096, 64, 4, 128, "bf16", zero=True, seed=77)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("K,group", [(28672, 64), (66048, 128)])
def test_stream_register_activations_long_k(pkg, oracle, dev, K, group):
    """More rows than the LDS holds and a long K: the group scales / zeros are staged in more than
    one pass (28672 / 64 groups), or not at all when even they are too many (K = 66048)."""
    p = random_problem(oracle, 9, K, 48, 4, group, "bf16", zero=True, seed=K % 1000)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
    assert err < TOL, err


@pytest.mark.parametrize("shape,M", [("2,8,2,2", 17), ("1,8,2,2", 32), ("2,8,2,0", 25), ("1,8,1,2", 33), ("2,8,1,2", 64),
                                     ("1,8,1,0", 50), ("1,4,1,0", 100), ("1,8,1,0", 128)])
def test_stream_skinny_m_launch_shapes(pkg, oracle, dev, woq_env, shape, M):
    """The launch shapes of 17..128 rows (two, four and eight row tiles per wavefront), with and
    without the group scales staged in LDS: a tile-row count no wavefront count divides, N that ends
    inside a workgroup's strips."""
    woq_env(WOQ_STREAM_SHAPE=shape)
    for bits, group, dtype in [(4, 128, "bf16"), (4, 64, "fp16"), (8, 128, "bf16")]:
        p = random_problem(oracle, M, 1408, 272, bits, group, dtype, zero=True, bias=True, pqs=True, seed=M)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
        assert err < TOL, (shape, bits, group, dtype, err)


@pytest.mark.parametrize("shape", ["2,4,4", "1,4,4"])
@pytest.mark.parametrize("bits,group,dtype,K,N", [(4, 128, "bf16", 2176, 272), (4, 64, "fp16", 1408, 1040),
                                                  (8, 64, "bf16", 1088, 144), (4, 128, "fp16", 128, 16),
                                                  (4, 64, "bf16", 4160, 528)])
def test_wide_decode_kernel_forced(pkg, oracle, dev, woq_env, shape, bits, group, dtype, K, N):
    """The wide-matrix decode kernel (a wavefront owns whole columns; 16 groups of K share the MFMA
    rows, scales applied once per 16 groups), forced through WOQ_WIDE_SHAPE on small problems: group
    counts that end inside a window of 16, K that ends in half a weight tile, N that ends inside a
    workgroup's strips or inside a wavefront's pair of strips; every optional input."""
    woq_env(WOQ_WIDE_SHAPE=shape)
    for zero, bias, pqs in [(True, True, True), (False, False, False), (True, False, False), (False, True, True)]:
        p = random_problem(oracle, 1, K, N, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
        assert err < TOL, (shape, zero, bias, pqs, err)


def test_wide_decode_kernel_is_what_wide_single_row_int8_problems_run_on(pkg, oracle, dev, woq_env):
    """One row, int8 weights with group scales, K <= 4096, at least 1536 column strips: the built-in rule takes
    the wide kernel (switching it off changes the float32 summation order, hence some output bits, while both
    stay within the bar), and a one-hot activation returns the dequantized weight row through it.  (int4
    weights with group scales of 64 / 128 run on the single-row kernel.)"""
    K, N = 512, 24576 + 48
    p = random_problem(oracle, 1, K, N, 8, 64, "bf16", zero=True, seed=77)
    auto = run_product(pkg, oracle, dev, p, 0)
    assert "stream wide" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, auto, p) < TOL
    woq_env(WOQ_WIDE_SHAPE="0")
    other = run_product(pkg, oracle, dev, p, 0)
    assert "stream mt=1" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, other, p) < TOL
    assert (auto != other).any()
    woq_env(WOQ_WIDE_SHAPE=None)
    p["act"] = np.zeros((1, K), np.float32)
    p["act"][0, 300] = 1.0
    out = run_product(pkg, oracle, dev, p, 0)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 64, "bf16")[300]
    assert (np.abs(out[0] - w) <= np.abs(w) * 2.0 ** -7 + 2.5e-7).all()


@pytest.mark.parametrize("shape", ["4,8", "8,8", "16,8", "4,4", "8,4", "16,2", "8,7", "7,4"])
@pytest.mark.parametrize("group,dtype,K,N", [(128, "bf16", 2176, 272), (64, "fp16", 1408, 1040), (128, "fp16", 128, 16),
                                             (64, "bf16", 4160, 528), (128, "bf16", 14336, 48)])
def test_row_decode_kernel_forced(pkg, oracle, dev, woq_env, shape, group, dtype, K, N):
    """The row kernel (one workgroup per strip, every wavefront a few consecutive tiles, no staging pass),
    forced through WOQ_ROW_SHAPE for one to four rows: K that needs several passes of the workgroup or leaves
    wavefronts without tiles, a last tile that is only half inside K, groups that end inside a wavefront's
    rows; every optional input.  (A shape whose groups x rows exceed the 16 MFMA rows is refused and the call
    falls through to the strip-group kernel.)"""
    woq_env(WOQ_ROW_SHAPE=shape)
    tiles = int(shape.split(",")[1])
    for M in (1, 2, 3, 4):
        fits = tiles * (128 // group) * (1 if M == 1 else (2 if M == 2 else 4)) <= 16
        for zero, bias, pqs in [(True, True, True), (False, False, False), (True, False, False), (False, True, True)]:
            p = random_problem(oracle, M, K, N, 4, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N + M)
            err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
            assert ("stream row" in _last_launch(pkg)) == fits, (M, _last_launch(pkg))
            assert err < TOL, (shape, M, zero, bias, pqs, err)


@pytest.mark.parametrize("shape", ["8,1,2", "8,2,2", "8,4,2", "16,2,2", "4,1,4"])
@pytest.mark.parametrize("group,dtype,K,N", [(128, "bf16", 2176, 272), (64, "fp16", 2112, 1040), (128, "fp16", 128, 16),
                                             (64, "bf16", 4160, 528), (128, "bf16", 14336, 48)])
def test_multirow_kernel_forced(pkg, oracle, dev, woq_env, shape, group, dtype, K, N):
    """The multi-row kernel without a staging pass (a workgroup owns a few strips, its wavefronts split K and
    request everything of a pass at once), forced through WOQ_ROWS_SHAPE for 2 ... 16 rows: K that needs several
    passes or leaves wavefronts without tile rows, a last tile that is only half inside K (g64), a strip count
    that the strips per workgroup do not divide; every optional input (zeros, bias, smoothing vector)."""
    woq_env(WOQ_ROWS_SHAPE=shape, WOQ_ROW_SHAPE="0")
    for M in (2, 5, 8, 13, 16):
        for zero, bias, pqs in [(True, True, True), (False, False, False), (True, False, False), (False, True, True)]:
            p = random_problem(oracle, M, K, N, 4, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N + M)
            err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
            assert "stream multirow" in _last_launch(pkg), (M, _last_launch(pkg))
            assert err < TOL, (shape, M, zero, bias, pqs, err)


@pytest.mark.parametrize("shape", ["8,1,2", "8,4,2", "16,2,2"])
@pytest.mark.parametrize("bits,group,dtype,K,N", [(8, 0, "fp16", 2112, 272), (8, 0, "bf16", 4160, 528), (8, 64, "bf16", 2112, 272),
                                                 (8, 128, "fp16", 1408, 1040), (4, 0, "bf16", 2176, 272), (4, 0, "fp16", 128, 16)])
def test_multirow_kernel_forced_int8_and_per_channel(pkg, oracle, dev, woq_env, shape, bits, group, dtype, K, N):
    """The multi-row kernel's other weight formats, forced through WOQ_ROWS_SHAPE: int8 (64 rows of K per tile)
    with per-channel scales or group scales of 64 / 128 rows (a group of 128 spans two tile rows), int4 with
    per-channel scales; 1 ... 16 rows, zeros where the format has them, bias, smoothing vector."""
    woq_env(WOQ_ROWS_SHAPE=shape, WOQ_ROW_SHAPE="0")
    for M in (1, 3, 8, 16):
        for zero, bias, pqs in [(group != 0, True, True), (False, False, False)]:
            p = random_problem(oracle, M, K, N, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N + M + bits)
            err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
            assert "stream multirow" in _last_launch(pkg), (M, _last_launch(pkg))
            assert err < TOL, (shape, M, zero, bias, pqs, err)


def test_multirow_kernel_rule_and_exact_rows(pkg, oracle, dev, woq_env):
    """The built-in rule takes the multi-row kernel for 5 ... 16 rows on narrow matrices with K up to 4096 (one
    strip per workgroup up to 256 strips, two up to 512), with or without a smoothing vector, and for int8
    per-channel weights on the same matrices; not for int8 with group scales, int4 per-channel or one row; one-hot activation rows return the dequantized weight rows through it, row for row;
    rows past m stay untouched in the output buffer's neighbours (the kernel stores rows below m only)."""
    K, N = 4096, 4096
    p = random_problem(oracle, 8, K, N, 4, 128, "bf16", zero=True, seed=91)
    auto = run_product(pkg, oracle, dev, p, 0)
    assert "stream multirow waves=8 ns=1 tpw=2 passes=2" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, auto, p) < TOL
    woq_env(WOQ_ROWS_SHAPE="0")
    staged = run_product(pkg, oracle, dev, p, 0)
    assert "stream multirow" not in _last_launch(pkg) and parity_err(oracle, staged, p) < TOL
    woq_env(WOQ_ROWS_SHAPE=None)
    p = random_problem(oracle, 12, 4096, 6144, 4, 64, "fp16", zero=False, seed=92)
    assert parity_err(oracle, run_product(pkg, oracle, dev, p, 0), p) < TOL
    assert "stream multirow waves=8 ns=2 tpw=2" in _last_launch(pkg), _last_launch(pkg)
    q = random_problem(oracle, 8, 1024, 256, 4, 128, "bf16", zero=True, pqs=True, seed=93)
    assert parity_err(oracle, run_product(pkg, oracle, dev, q, 0), q) < TOL and "stream multirow" in _last_launch(pkg)
    q = random_problem(oracle, 8, 4096, 4096, 8, 0, "fp16", seed=95)  # int8 per-channel on a narrow matrix
    assert parity_err(oracle, run_product(pkg, oracle, dev, q, 0), q) < TOL
    assert "stream multirow waves=8 ns=1 tpw=2" in _last_launch(pkg), _last_launch(pkg)
    for kw in (dict(bits=8, group=128), dict(bits=4, group=0), dict(bits=4, group=128, M=1), dict(bits=8, group=0, M=1)):
        q = random_problem(oracle, kw.get("M", 8), 1024, 256, kw["bits"], kw["group"], "bf16", zero=kw["group"] != 0, seed=93)
        run_product(pkg, oracle, dev, q, 0)
        assert "stream multirow" not in _last_launch(pkg), (kw, _last_launch(pkg))
    M, K, N = 11, 2048, 272
    p = random_problem(oracle, M, K, N, 4, 128, "bf16", zero=True, seed=94)
    hot = [(997 * r + 127) % K for r in range(M)]
    p["act"] = np.zeros((M, K), np.float32)
    for r, h in enumerate(hot):
        p["act"][r, h] = 1.0
    woq_env(WOQ_ROWS_SHAPE="8,2,2", WOQ_ROW_SHAPE="0")
    out = run_product(pkg, oracle, dev, p, STREAM)
    assert "stream multirow" in _last_launch(pkg)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 128, "bf16")
    for r, h in enumerate(hot):
        assert (np.abs(out[r] - w[h]) <= np.abs(w[h]) * 2.0 ** -7 + 2.5e-7).all(), r


def test_row_decode_kernel_is_what_few_row_int4_problems_run_on(pkg, oracle, dev, woq_env):
    """One row, int4 with group scales of 64 or 128: the built-in rule takes the row kernel, with one pass over
    K where sixteen wavefronts x eight tiles reach that far; two rows except at K = 8192 on matrices of 513 ... 2047 strips;
    three and four rows on narrow matrices with K up to 4096 or beyond 8192.  int8 weights, more rows,
    per-channel scales or larger groups do not.  Every one-hot activation returns the dequantized weight row
    through it; switched off, the strip-group kernel meets the same bar."""
    K, N = 4096, 272
    p = random_problem(oracle, 1, K, N, 4, 128, "bf16", zero=True, seed=78)
    auto = run_product(pkg, oracle, dev, p, 0)
    assert "stream row waves=4 tpw=8 passes=1 rows=1" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, auto, p) < TOL
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 128, "bf16")
    for M in (1, 2, 4):
        hot = [(997 * r + 127) % K for r in range(M)]
        p = random_problem(oracle, M, K, N, 4, 128, "bf16", zero=True, seed=78)
        p["act"] = np.zeros((M, K), np.float32)
        p["act"][np.arange(M), hot] = 1.0
        out = run_product(pkg, oracle, dev, p, 0)
        assert "stream row" in _last_launch(pkg), _last_launch(pkg)
        assert (np.abs(out - w[hot]) <= np.abs(w[hot]) * 2.0 ** -7 + 2.5e-7).all(), M
    woq_env(WOQ_ROW_SHAPE="0")
    p = random_problem(oracle, 1, K, N, 4, 128, "bf16", zero=True, seed=78)
    other = run_product(pkg, oracle, dev, p, 0)
    assert "stream mt=1" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, other, p) < TOL
    woq_env(WOQ_ROW_SHAPE=None)
    for M, K2, group, want in ((1, 8192, 64, "waves=8 tpw=4 passes=2 rows=1"), (1, 14336, 128, "waves=8 tpw=7 passes=2 rows=1"), (1, 12288, 128, "waves=16 tpw=8 passes=1 rows=1"),
                               (4, 14336, 128, "waves=7 tpw=4 passes=4 rows=4"),
                               (1, 28672, 128, "waves=4 tpw=4 passes=14 rows=1"), (1, 128, 64, "waves=4 tpw=8 passes=1 rows=1"),
                               (2, 4096, 128, "waves=4 tpw=8 passes=1 rows=2"), (2, 8192, 128, "waves=4 tpw=4 passes=4 rows=2"), (2, 28672, 64, "waves=4 tpw=4 passes=14 rows=2"),
                               (3, 4096, 128, "waves=8 tpw=4 passes=1 rows=4"), (4, 14336, 64, "waves=16 tpw=2 passes=4 rows=4")):
        q = random_problem(oracle, M, K2, 48, 4, group, "fp16", zero=True, bias=True, pqs=True, seed=K2 + M)
        assert parity_err(oracle, run_product(pkg, oracle, dev, q, 0), q) < TOL
        assert "stream row " + want in _last_launch(pkg), (M, K2, _last_launch(pkg))
    for kw in (dict(M=5), dict(M=2, K=8192, N=640 * 16), dict(M=4, K=8192), dict(M=4, N=513 * 16), dict(bits=8, group=64),
               dict(group=0), dict(group=256)):
        a = dict(M=1, K=K, N=N, bits=4, group=128)
        a.update(kw)
        q = random_problem(oracle, a["M"], a["K"], a["N"], a["bits"], a["group"], "bf16", seed=79)
        assert parity_err(oracle, run_product(pkg, oracle, dev, q, 0), q) < TOL
        assert "stream row" not in _last_launch(pkg), (kw, _last_launch(pkg))


def _last_launch(pkg):
    return (pkg._lib.lib.woq_last_launch() or b"").decode()


@pytest.mark.parametrize("M,bits,group,dtype,K,N", [(1, 4, 128, "bf16", 512, 9216), (1, 4, 64, "fp16", 384, 12288 - 16),
                                                    (2, 4, 128, "bf16", 256, 8208), (4, 8, 64, "bf16", 256, 10240),
                                                    (1, 8, 0, "fp16", 320, 12288), (3, 4, 0, "bf16", 512, 9232)])
def test_stream_three_strips_per_workgroup(pkg, oracle, dev, woq_env, M, bits, group, dtype, K, N):
    """513 ... 768 column strips and few rows: the built-in rule gives a workgroup three strips (a last
    workgroup with one or two, N that is not a multiple of 48); every optional input; one-hot rows return
    the dequantized weight.  (The single-row kernel, which would take the one-row int4 cases, is switched
    off: this is the strip-group kernel's test.)"""
    woq_env(WOQ_ROW_SHAPE="0")
    for zero, bias, pqs in [(group != 0, True, True), (False, False, False)]:
        p = random_problem(oracle, M, K, N, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N + M)
        out = run_product(pkg, oracle, dev, p, 0)
        assert "ns=3" in _last_launch(pkg), _last_launch(pkg)
        assert parity_err(oracle, out, p) < TOL, (zero, bias, pqs)
    p = random_problem(oracle, M, K, N, bits, group, dtype, zero=group != 0, seed=N)
    p["act"] = np.zeros((M, K), np.float32)
    for r in range(M):
        p["act"][r, (37 * r + 5) % K] = 1.0
    out = run_product(pkg, oracle, dev, p, 0)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], group, dtype)
    for r in range(M):
        row = w[(37 * r + 5) % K]
        assert (np.abs(out[r] - row) <= np.abs(row) * 2.0 ** -7 + 2.5e-7).all(), r


@pytest.mark.parametrize("M,K,group", [(1, 14336, 128), (3, 14336, 64), (1, 20480, 128), (2, 16384 + 64, 64)])
def test_stream_staged_chunks_beyond_the_first_batch(pkg, oracle, dev, woq_env, M, K, group):
    """Activations of more than two (and more than four) 16-byte chunks per thread and group tables of more
    than one: the chunks a thread keeps across the weight prefetch, the batched loop behind it, a ragged
    last batch (strip-group kernel: the single-row kernel is switched off)."""
    woq_env(WOQ_ROW_SHAPE="0")
    p = random_problem(oracle, M, K, 272, 4, group, "bf16", zero=True, bias=True, pqs=True, seed=K + M)
    out = run_product(pkg, oracle, dev, p, 0)
    assert "stream" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, out, p) < TOL


@pytest.mark.parametrize("splits", [2, 3, 7])
@pytest.mark.parametrize("M,bits,group,dtype,K,N", [(16, 4, 128, "bf16", 2176, 272), (5, 4, 64, "fp16", 1408, 144),
                                                    (9, 8, 0, "bf16", 1088, 64), (2, 4, 128, "bf16", 4096, 48),
                                                    (1, 4, 128, "fp16", 1536, 528), (40, 8, 128, "bf16", 1024, 272)])
def test_stream_split_k_forced(pkg, oracle, dev, woq_env, splits, M, bits, group, dtype, K, N):
    """K split across workgroups (float32 slabs in the workspace, summed in slice order by the finish
    pass), forced through WOQ_STREAM_SPLITS: slice counts that do not divide the tile rows, a last slice
    that ends in half a weight tile, staged and register-held activations, the single-row group-slot
    variant, more than 16 rows (no split: it must still be right); every optional input; the same bits
    on every call."""
    woq_env(WOQ_STREAM_SPLITS=splits)
    for zero, bias, pqs in [(group != 0, True, True), (False, False, False)]:
        p = random_problem(oracle, M, K, N, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=K + N + splits)
        first = run_product(pkg, oracle, dev, p, STREAM)
        assert parity_err(oracle, first, p) < TOL, (zero, bias, pqs)
        again = run_product(pkg, oracle, dev, p, STREAM)
        assert (again.view(np.uint32) == first.view(np.uint32)).all()


@pytest.mark.parametrize("M,N", [(16, 272), (8, 4096), (4, 528)])
def test_stream_split_k_by_the_built_in_rule(pkg, oracle, dev, woq_env, M, N):
    """Long K, few columns, 4..16 rows: the rule splits K when it is given the workspace for the slabs
    (woq_workspace_bytes asks for it) and does not without one; both are within the bar, and they
    differ in float32 summation order."""
    K = 8192
    p = random_problem(oracle, M, K, N, 4, 128, "bf16", zero=True, bias=True, seed=M + N)
    L = pkg._lib
    assert L.lib.woq_workspace_bytes(M, N, K, L.ALGO_ZERO | L.ALGO_BIAS, L.BF16) >= 2 * M * N * 4
    split = run_product(pkg, oracle, dev, p, STREAM)
    assert parity_err(oracle, split, p) < TOL
    woq_env(WOQ_STREAM_SPLITS=1)
    plain = run_product(pkg, oracle, dev, p, STREAM)
    assert parity_err(oracle, plain, p) < TOL
    assert (split != plain).any()


@pytest.mark.parametrize("M", [1, 3, 16, 40])
@pytest.mark.parametrize("bits,group,dtype,K,N", [(4, 192, "fp16", 256, 1024), (4, 256, "bf16", 384, 2048),
                                                  (4, 320, "fp16", 1024, 528), (8, 192, "bf16", 1088, 272),
                                                  (4, 256, "bf16", 4160, 144)])
def test_stream_flexible_group_sizes(pkg, oracle, dev, M, bits, group, dtype, K, N):
    """Group sizes that are multiples of 64 above 128 (the reference's Hopper kernels take them) on the
    streaming kernels: staged and register-held activations, the single-row group-slot variant, a last
    group that is shorter than the others, K that ends in half a weight tile."""
    for zero, bias, pqs in [(True, True, True), (False, False, False)]:
        p = random_problem(oracle, M, K, N, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=group + M)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, STREAM), p)
        assert err < TOL, (zero, bias, pqs, err)
