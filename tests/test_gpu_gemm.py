"""GPU parity of the prefill MFMA GEMM against the CPU oracle, through the C ABI.  Same bar as the
streaming kernel: max|out - ref| / max|ref| <= 1e-2 against the float64-accumulated
dequantize-then-matmul reference."""
import numpy as np
import pytest
import torch

from _util import parity_err, random_problem, reference, run_product

pytestmark = pytest.mark.gpu
TOL = 1e-2
GEMM = 2


def _last_launch(pkg):
    return (pkg._lib.lib.woq_last_launch() or b"").decode()


@pytest.fixture(params=["exact", "skinny"], autouse=True)
def gemm_kernel(request, woq_env):
    """The GEMM regime has two kernels (exact-dequantize 256-row tiles, deferred-scale 64-row tiles);
    every test below runs on each, whatever the library would pick for the shape."""
    woq_env(WOQ_GEMM_KERNEL=request.param)
    return request.param


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits,group", [(4, 128), (4, 64), (4, 0), (8, 0), (8, 64), (8, 128)])
@pytest.mark.parametrize("zero", [False, True])
def test_gemm_variants(pkg, oracle, dev, dtype, bits, group, zero):
    if group == 0 and zero:
        pytest.skip("per-channel has no zeros")
    p = random_problem(oracle, 300, 512, 512, bits, group, dtype, zero=zero, seed=bits + group)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
    assert err < TOL, err


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("group,zero", [(128, False), (128, True), (64, False), (64, True), (0, False)])
@pytest.mark.parametrize("M", [5, 17, 32])
def test_gemm_at_most_32_rows(pkg, oracle, dev, dtype, group, zero, M):
    """M <= 32 with int4 weights: the deferred-scale kernel switches to 32-row tiles; K long enough
    that it also splits K, N ragged."""
    p = random_problem(oracle, M, 2048, 784, 4, group, dtype, zero=zero, bias=True, seed=M + group)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
    assert err < TOL, err


@pytest.mark.parametrize("M", [1, 16, 129, 256, 257, 512, 1000])
def test_gemm_m_edges(pkg, oracle, dev, M):
    """Row counts around the 256-row tile, including the decode sizes forced onto this kernel."""
    p = random_problem(oracle, M, 256, 256, 4, 128, "bf16", zero=True, bias=True, seed=M)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
    assert err < TOL, err


@pytest.mark.parametrize("K,N", [(64, 256), (192, 272), (320, 16), (1024, 784), (2048, 4096)])
def test_gemm_ragged_shapes(pkg, oracle, dev, K, N):
    """K with a padded last weight tile row, N that is not a multiple of the 256-column tile."""
    for bits, group in [(4, 64), (8, 64), (4, 0)]:
        p = random_problem(oracle, 260, K, N, bits, group, "bf16", zero=group != 0, seed=K + N)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
        assert err < TOL, (bits, group, err)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_gemm_prequant_scale_goes_through_workspace(pkg, oracle, dev, dtype):
    """AWQ smoothing in the GEMM regime: the smoothing pass writes the workspace, the GEMM reads it."""
    p = random_problem(oracle, 384, 512, 256, 4, 128, dtype, zero=True, bias=True, pqs=True, seed=5)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
    assert err < TOL, err


def test_gemm_identity_recovers_dequantized_weight_exactly(pkg, oracle, dev, gemm_kernel):
    """Identity activation: every output is ONE product 1 * w, so the GEMM returns the dequantized
    weight bit for bit - the in-kernel dequantize equals the oracle's definition."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel applies scales to float32 sums, not to single weights")
    K, N = 256, 256
    for dtype in ("bf16", "fp16"):
        p = random_problem(oracle, K, K, N, 4, 64, dtype, zero=True, seed=9)
        p["act"] = np.eye(K, dtype=np.float32)
        out = run_product(pkg, oracle, dev, p, GEMM)
        w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 64, dtype)
        assert (out.view(np.uint32) == w.view(np.uint32)).all(), dtype


@pytest.mark.parametrize("rt", [4, 8, 16])
@pytest.mark.parametrize("bits,dtype", [(4, "bf16"), (4, "fp16"), (8, "bf16")])
def test_gemm_identity_every_tile_height(pkg, oracle, dev, woq_env, gemm_kernel, rt, bits, dtype):
    """The same bit-exact identity at every tile height (64 / 128 / 256 rows): the accumulators are read
    behind hand-placed waits that the compiler does not see, and a missed one would show here."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel applies scales to float32 sums, not to single weights")
    woq_env(WOQ_GEMM_RT=str(rt))
    K, N = 256, 512
    p = random_problem(oracle, K, K, N, bits, 64, dtype, zero=True, seed=rt + bits)
    p["act"] = np.eye(K, dtype=np.float32)
    out = run_product(pkg, oracle, dev, p, GEMM)
    assert "rt=%d" % rt in _last_launch(pkg), _last_launch(pkg)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 64, dtype)
    assert (out.view(np.uint32) == w.view(np.uint32)).all()


def test_gemm_identity_through_the_persistent_loop(pkg, oracle, dev, gemm_kernel):
    """Identity activation on a shape that takes the persistent kernel (258 tiles): the first matrix
    instruction of every tile starts a fresh sum and the finished tile leaves through the explicit
    accumulator reads - bit for bit the dequantized weight."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel has no persistent form")
    K, N = 512, 256 * 129
    p = random_problem(oracle, K, K, N, 4, 128, "bf16", zero=True, seed=21)
    p["act"] = np.eye(K, dtype=np.float32)
    out = run_product(pkg, oracle, dev, p, GEMM)
    assert "persistent=1" in _last_launch(pkg), _last_launch(pkg)
    w = oracle.dequantize(p["q"], p["scales"], p["zeros"], 128, "bf16")
    assert (out.view(np.uint32) == w.view(np.uint32)).all()


def test_gemm_matches_stream_kernel(pkg, oracle, dev):
    """The two regimes agree with each other at their crossover size."""
    p = random_problem(oracle, 128, 1024, 512, 4, 128, "bf16", zero=True, seed=31)
    a = run_product(pkg, oracle, dev, p, 1)
    b = run_product(pkg, oracle, dev, p, GEMM)
    assert oracle.max_rel_err(a, b) < 1e-2  # each is within 1e-2 of the oracle; they round differently


def test_auto_regime_and_kernel_choice(pkg, oracle, dev, woq_env):
    woq_env(WOQ_GEMM_KERNEL=None)
    for m in (200, 640):
        p = random_problem(oracle, m, 512, 256, 4, 128, "bf16", zero=True, seed=40 + m)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, 0), p)
        assert err < TOL, (m, err)
    p = random_problem(oracle, 640, 256, 256, 8, 0, "fp16", seed=41)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, 0), p)
    assert err < TOL, err


@pytest.mark.parametrize("M", [17, 64, 65, 100, 128, 200, 512])
@pytest.mark.parametrize("K,N", [(4096, 256), (2048, 1024), (1152, 528)])
def test_gemm_skinny_m_splits_k(pkg, oracle, dev, M, K, N):
    """Skinny M x narrow N: 64/128/256-row tiles and K split across workgroups through the float32
    partial buffer (ragged K slices, a last slice shorter than the others, bias in the finish pass)."""
    for bits, group, dtype in [(4, 128, "bf16"), (8, 64, "fp16"), (4, 0, "fp16")]:
        p = random_problem(oracle, M, K, N, bits, group, dtype, zero=group != 0, bias=True, seed=M + K)
        err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
        assert err < TOL, (bits, group, dtype, err)


def test_gemm_split_k_reuses_a_dirty_workspace(pkg, oracle, dev):
    """Every element of the partial slabs is written by the call before the finish pass reads it: a
    workspace full of garbage, used twice."""
    F = pkg.functional
    p = random_problem(oracle, 48, 4096, 256, 4, 128, "bf16", zero=True, pqs=True, seed=77)
    need = pkg._lib.lib.woq_workspace_bytes(48, 256, 4096, F.ZERO | F.PRE_QUANT_SCALE, pkg._lib.BF16)
    assert need > 48 * 4096 * 2  # smoothing region plus partial sums
    ws = torch.full((need,), 0x7F, dtype=torch.uint8, device=dev)
    from _util import TORCH_DT, preprocess, to_dev
    w = preprocess(pkg, oracle, p["q"], 4).to(dev)
    ref = reference(oracle, p)
    for _ in range(2):
        out = F.woq_matmul_raw(to_dev(p["act"], "bf16", dev), to_dev(p["pqs"], "bf16", dev), w,
                               to_dev(p["scales"], "bf16", dev), to_dev(p["zeros"], "bf16", dev), None, n=256,
                               k=4096, group_size=128, quant_algo=F.ZERO | F.PRE_QUANT_SCALE, regime=GEMM,
                               workspace=ws)
        torch.cuda.synchronize()
        assert oracle.max_rel_err(out.float().cpu().numpy(), ref) < TOL


@pytest.mark.parametrize("bits,group,dtype", [(4, 128, "bf16"), (8, 0, "fp16")])
def test_gemm_split_k_is_bit_reproducible(pkg, oracle, dev, woq_env, bits, group, dtype):
    """The K slices are summed in slice order, whichever workgroup finishes first: repeated calls
    return the same bits, on either GEMM kernel (the fixture's) and for several split counts."""
    p = random_problem(oracle, 96, 4096, 512, bits, group, dtype, zero=group != 0, bias=True, seed=13)
    for splits in (2, 5, 8):
        woq_env(WOQ_GEMM_SPLITS=str(splits))
        first = run_product(pkg, oracle, dev, p, GEMM)
        assert parity_err(oracle, first, p) < TOL, splits
        for _ in range(3):
            again = run_product(pkg, oracle, dev, p, GEMM)
            assert (again.view(np.uint32) == first.view(np.uint32)).all(), splits


# the reference's own grid for group sizes beyond 128 (m, n, k, dtype, pre-quant scale, zeros, bias, group:
# tests/quantization/test_weight_only_groupwise_quant_matmul.py:405-420, its Hopper-only
# test_hopper_flexible_groups) plus a longer K; k = 256 with groups of 192 leaves a last group of 64 rows
FLEXIBLE = [(32, 1024, 256, "fp16", True, True, False, 192), (32, 2048, 384, "bf16", True, False, True, 256),
            (64, 2048, 1024, "fp16", True, False, False, 320), (200, 528, 1536, "bf16", False, True, True, 192),
            (96, 272, 4096, "bf16", True, True, True, 256)]


@pytest.mark.parametrize("m,n,k,dtype,pqs,zero,bias,group", FLEXIBLE)
@pytest.mark.parametrize("bits", [4, 8])
def test_gemm_flexible_group_sizes(pkg, oracle, dev, m, n, k, dtype, pqs, zero, bias, group, bits):
    """Group sizes that are multiples of 64 above 128, on either GEMM kernel (the fixture's), int4 and
    int8, split K included (k = 4096 at 96 rows)."""
    p = random_problem(oracle, m, k, n, bits, group, dtype, zero=zero, bias=bias, pqs=pqs, seed=group + m)
    assert p["scales"].shape[0] == -(-k // group)
    err = parity_err(oracle, run_product(pkg, oracle, dev, p, GEMM), p)
    assert err < TOL, err


# more 256 x 256 tiles than the chip has CUs, N a multiple of 256, an even number (>= 4) of weight tile
# rows, no bias: the shapes that take the persistent kernel; M ragged against the tile and against 16
PERSISTENT = [(4000, 512, 8192, 4, 128, "bf16", True), (2250, 1024, 16384, 4, 64, "fp16", True),
              (2250, 960, 16384, 4, 64, "bf16", False), (4096, 512, 8192, 8, 0, "fp16", False),
              (3000, 256, 12288, 8, 128, "bf16", True), (2304, 1024, 8192, 4, 0, "bf16", False)]


@pytest.mark.parametrize("m,k,n,bits,group,dtype,zero", PERSISTENT)
def test_gemm_persistent_tile_loop(pkg, oracle, dev, woq_env, gemm_kernel, m, k, n, bits, group, dtype, zero):
    """One workgroup per CU walking several tiles (the next tile's first loads requested during the
    current tile's last tile row, the outputs stored between the next tile's first matrix
    instructions) returns the bits of the one-tile-per-workgroup launch, which in turn meets the
    oracle's bar."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel has no persistent form")
    p = random_problem(oracle, m, k, n, bits, group, dtype, zero=zero, seed=m + k)
    out = run_product(pkg, oracle, dev, p, GEMM)
    assert "persistent=1" in _last_launch(pkg), _last_launch(pkg)
    woq_env(WOQ_GEMM_PERSIST="0")
    plain = run_product(pkg, oracle, dev, p, GEMM)
    assert "persistent=0" in _last_launch(pkg), _last_launch(pkg)
    assert (out.view(np.uint32) == plain.view(np.uint32)).all()
    assert parity_err(oracle, out, p) < TOL


def test_gemm_persistent_needs_whole_tiles_and_no_bias(pkg, oracle, dev, gemm_kernel):
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel has no persistent form")
    for n, bias in [(8192 + 16, False), (8192, True)]:
        p = random_problem(oracle, 4000, 512, n, 4, 128, "bf16", zero=True, bias=bias, seed=n)
        out = run_product(pkg, oracle, dev, p, GEMM)
        assert "persistent=0" in _last_launch(pkg), _last_launch(pkg)
        assert parity_err(oracle, out, p) < TOL


@pytest.mark.parametrize("m,k,n,bits,group,dtype,zero,bias", [
    (300, 512, 768, 4, 128, "bf16", True, True), (257, 1024, 384, 8, 0, "fp16", False, False),
    (520, 448, 960, 4, 64, "fp16", True, False), (4000, 512, 192 * 43, 4, 128, "bf16", True, False),
    (2250, 256, 192 * 120, 8, 128, "bf16", False, False)])
def test_gemm_192_column_tiles(pkg, oracle, dev, woq_env, gemm_kernel, m, k, n, bits, group, dtype, zero, bias):
    """256-row tiles of 192 columns (three strips per wavefront): against the oracle, and bit for bit
    against the 256-column tiles; the last two shapes take the persistent loop."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel has one tile width")
    p = random_problem(oracle, m, k, n, bits, group, dtype, zero=zero, bias=bias, seed=n)
    woq_env(WOQ_GEMM_COLS="192", WOQ_GEMM_RT="16", WOQ_GEMM_SPLITS="1")
    out = run_product(pkg, oracle, dev, p, GEMM)
    assert "columns=192" in _last_launch(pkg), _last_launch(pkg)
    if m >= 2000:
        assert "persistent=1" in _last_launch(pkg), _last_launch(pkg)
    woq_env(WOQ_GEMM_COLS="256")
    wide = run_product(pkg, oracle, dev, p, GEMM)
    assert "columns=256" in _last_launch(pkg), _last_launch(pkg)
    assert (out.view(np.uint32) == wide.view(np.uint32)).all()
    assert parity_err(oracle, out, p) < TOL


def test_gemm_picks_192_columns_where_256_leave_a_round_mostly_empty(pkg, oracle, dev, gemm_kernel):
    """Llama-3-8B qkv (N = 6144) at 2048 rows: 192 tiles of 256 columns fill three quarters of the CUs,
    256 tiles of 192 columns fill them all."""
    if gemm_kernel == "skinny":
        pytest.skip("the deferred-scale kernel has one tile width")
    p = random_problem(oracle, 2048, 256, 6144, 4, 128, "bf16", zero=True, seed=6)
    out = run_product(pkg, oracle, dev, p, GEMM)
    assert "columns=192" in _last_launch(pkg), _last_launch(pkg)
    assert parity_err(oracle, out, p) < TOL
