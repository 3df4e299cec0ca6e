"""Argument validation and regime selection of woq_matmul, exercised without a GPU through
woq_matmul_check (same checks, no launch).  Error behaviour follows the reference's
TLLM_CHECK / runtime_error sites (fpA_intB_gemm_template.h:129-196, kernelDispatcher.h:30-166)."""
import ctypes

import pytest


def make_args(L, **kw):
    a = L.MatmulArgs()
    base = dict(act=0x1000, pre_quant_scale=None, weight=0x2000, scales=0x3000, zeros=None, bias=None, out=0x4000,
                alpha=1.0, m=4, n=256, k=512, group_size=128, quant_algo=0, act_dtype=L.BF16, out_dtype=L.BF16,
                regime=0, workspace=None, workspace_bytes=0)
    base.update(kw)
    for k, v in base.items():
        setattr(a, k, v)
    return a


def status(pkg, **kw):
    L = pkg._lib
    return L.lib.woq_matmul_check(ctypes.byref(make_args(L, **kw))), (L.lib.woq_last_error() or b"").decode()


def test_valid_combinations(pkg):
    L = pkg._lib
    assert status(pkg)[0] == 0
    assert status(pkg, zeros=0x5000, quant_algo=L.ALGO_ZERO)[0] == 0
    assert status(pkg, bias=0x5000, quant_algo=L.ALGO_BIAS, group_size=64)[0] == 0
    # multiples of 64 above 128 (the reference's Hopper kernels), also with a shorter last group
    assert status(pkg, k=768, group_size=192)[0] == 0
    assert status(pkg, k=512, group_size=320)[0] == 0
    assert status(pkg, pre_quant_scale=0x5000, quant_algo=L.ALGO_PRE_QUANT_SCALE)[0] == 0
    assert status(pkg, group_size=0, quant_algo=L.ALGO_INT8_WEIGHT, act_dtype=L.FP16, out_dtype=L.FP16)[0] == 0
    assert status(pkg, m=0)[0] == 0                                     # m == 0 is a no-op, not an error
    assert status(pkg, quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3, alpha=0.5)[0] == 0
    # e4m3 activations: multiples of 128 above 128 as the reference's Hopper kernels, shorter last group too
    assert status(pkg, quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3, group_size=256)[0] == 0
    assert status(pkg, quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3, k=1024, group_size=384)[0] == 0
    assert status(pkg, quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3, k=128, group_size=256)[0] == 0


@pytest.mark.parametrize("kw,code,text", [
    (dict(scales=None), -1, "scales"),
    (dict(act=None), -1, "NULL"),
    (dict(group_size=32), -3, "group_size"),
    (dict(group_size=96), -3, "multiple of 64"),
    (dict(quant_algo=8, act_dtype=2, group_size=192), -3, "multiples of 128"),
    (dict(k=96), -2, "multiple of 64"),
    (dict(k=576, group_size=128), -2, "group_size"),
    (dict(n=250), -2, "multiple of 16"),
    (dict(zeros=0x5000), -1, "ZERO"),
    (dict(quant_algo=2), -1, "ZERO"),
    (dict(quant_algo=1), -1, "BIAS"),
    (dict(quant_algo=4), -1, "PRE_QUANT_SCALE"),
    (dict(group_size=0, zeros=0x5000, quant_algo=2), -1, "scale only"),
    (dict(out_dtype=2), -1, "out_dtype"),
    (dict(act_dtype=0), -1, "activation dtype"),
    (dict(quant_algo=8 | 16, act_dtype=2), -3, "INT4"),
    (dict(quant_algo=8, act_dtype=2, group_size=64), -3, "128"),
    (dict(quant_algo=8, act_dtype=2, k=192, group_size=64), -3, "128"),
    (dict(quant_algo=8), -1, "PRE_QUANT_SCALE"),
    (dict(act_dtype=2), -1, "FP8_ALPHA"),
    (dict(regime=1, m=129), -3, "unsupported m"),
    (dict(regime=7), -1, "regime"),
    (dict(m=300000, k=4096), -3, "2 GiB"),                  # activations: 300000 * 4096 * 2 bytes
    (dict(n=65536, k=65536), -3, "2 GiB"),                  # one int4 weight matrix of 2 GiB
    (dict(m=-1), -2, "non-negative"),
    (dict(quant_algo=64), -1, "quant_algo"),
])
def test_rejections(pkg, kw, code, text):
    rc, msg = status(pkg, **kw)
    assert rc == code, msg
    assert text.lower() in msg.lower()


def test_null_args(pkg):
    assert pkg._lib.lib.woq_matmul_check(None) == -1


def test_workspace_rule(pkg):
    L = pkg._lib
    lib = L.lib
    algo = L.ALGO_PRE_QUANT_SCALE
    # the split-K partial buffer (one float32 [rows, n] slab per slice of K): none at m=4096 x n=4096
    # itself (256 tiles fill the chip), but the size covers every smaller m too, and a few hundred
    # rows still split K on this narrow N: whole float32 rows of the output
    split = lib.woq_workspace_bytes(4096, 4096, 8192, 0, L.BF16)
    # (never more than 512 workgroups x one 256 x 256 float32 tile = 128 MiB)
    assert split % (4096 * 4) == 0 and 2 * 64 * 4096 * 4 <= split <= 512 * 256 * 256 * 4
    # the smoothed activations come on top
    assert lib.woq_workspace_bytes(4096, 4096, 8192, algo, L.BF16) == 4096 * 8192 * 2 + split
    small = lib.woq_workspace_bytes(64, 4096, 8192, 0, L.BF16)
    assert small % (4096 * 4) == 0 and 2 * 64 * 4096 * 4 <= small <= split
    # a wide N fills the chip with few rows: only the smallest row counts split
    wide = lib.woq_workspace_bytes(4096, 20480, 8192, 0, L.BF16)
    assert wide % (20480 * 4) == 0 and wide <= 512 * 256 * 256 * 4
    # never shrinks as m grows
    sizes = [lib.woq_workspace_bytes(m, 1024, 4096, algo, L.FP16) for m in range(1, 3000, 37)]
    assert sizes == sorted(sizes)
    # the size asked for m rows is enough for every call with fewer rows, whatever plan those get
    for n, k, algo2, act in [(4096, 8192, 0, L.BF16), (256, 8192, 0, L.BF16), (1024, 4096, L.ALGO_INT8_WEIGHT, L.BF16),
                             (6144, 4096, L.ALGO_FP8_ALPHA, L.FP8_E4M3)]:
        group = 0 if algo2 & L.ALGO_INT8_WEIGHT else 128
        bound = lib.woq_workspace_bytes(30000, n, k, algo2, act)
        for m in list(range(1, 2600, 13)) + list(range(2600, 30000, 511)):
            rc, msg = status(pkg, m=m, n=n, k=k, quant_algo=algo2, act_dtype=act, group_size=group, regime=2,
                             workspace=0x9000, workspace_bytes=bound)
            assert rc == 0, (m, n, k, msg)
    # GEMM regime with smoothing needs the workspace; the streaming regime fuses it
    rc, msg = status(pkg, m=512, pre_quant_scale=0x5000, quant_algo=algo)
    assert rc == -4 and "workspace" in msg
    assert status(pkg, m=512, pre_quant_scale=0x5000, quant_algo=algo, workspace=0x9000,
                  workspace_bytes=512 * 512 * 2)[0] == 0
    assert status(pkg, m=8, pre_quant_scale=0x5000, quant_algo=algo)[0] == 0


def test_regime_table(pkg):
    L = pkg._lib
    sel = L.lib.woq_select_regime
    for m in (1, 2, 4, 15, 16, 17, 32):
        assert sel(m, 4096, 4096, 0) == L.REGIME_STREAM
    for m in (65, 128, 129, 256, 4096, 8192):
        assert sel(m, 4096, 4096, 0) == L.REGIME_GEMM
    # 17..64 rows: streaming where its cost estimate beats the GEMM plan's (small N, short K)
    for algo in (0, L.ALGO_INT8_WEIGHT):
        assert sel(16, 28672, 4096, algo) == L.REGIME_STREAM
        assert sel(32, 28672, 4096, algo) == L.REGIME_GEMM
        assert sel(32, 6144, 4096, algo) == L.REGIME_STREAM   # 384 strips, two per workgroup: one round of 192
        assert sel(20, 10240, 8192, algo) == L.REGIME_GEMM    # 320 workgroups: two rounds
        assert sel(20, 4096, 14336, algo) == L.REGIME_GEMM    # long K: split-K GEMM
        assert sel(48, 8192, 8192, algo) == L.REGIME_GEMM
        # the choice never goes back to streaming as the rows grow
        for n, k in ((4096, 4096), (6144, 4096), (8192, 8192), (2048, 4096), (5120, 8192)):
            picks = [sel(m, n, k, algo) for m in range(17, 130)]
            assert picks == sorted(picks, key=lambda r: r != L.REGIME_STREAM), (n, k, algo)
    # W4A8: streaming kernel up to two 16-row tiles (30 / 19 rows on long-K shapes of 8192 / 4096 columns), the fp8 GEMM above
    assert sel(1, 4096, 4096, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(16, 57344, 8192, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(17, 4096, 4096, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(32, 57344, 8192, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(30, 8192, 28672, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(31, 8192, 28672, L.ALGO_FP8_ALPHA) == L.REGIME_GEMM
    assert sel(19, 4096, 14336, L.ALGO_FP8_ALPHA) == L.REGIME_STREAM
    assert sel(20, 4096, 14336, L.ALGO_FP8_ALPHA) == L.REGIME_GEMM
    assert sel(33, 4096, 4096, L.ALGO_FP8_ALPHA) == L.REGIME_GEMM
    rc, msg = status(pkg, m=33, quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3, regime=1)
    assert rc == -3 and "unsupported m" in msg
    # 16-bit activations reach the W4A8 streaming kernel through the smoothing pass: workspace needed
    rc, msg = status(pkg, m=4, quant_algo=L.ALGO_FP8_ALPHA | L.ALGO_PRE_QUANT_SCALE, pre_quant_scale=0x5000)
    assert rc == -4 and "workspace" in msg


def test_python_wrappers_refuse_cpu_tensors(pkg):
    import torch
    a = torch.zeros(1, 128, dtype=torch.bfloat16)
    w = torch.zeros(128, 8, dtype=torch.int8)
    s = torch.zeros(1, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        pkg.functional.weight_only_groupwise_quant_matmul(a, None, w, s, None, None, None, 0, 128, "bfloat16")


def test_last_error_is_per_thread(pkg):
    import threading
    L = pkg._lib
    status(pkg, group_size=32)
    seen = {}

    def other():
        seen["msg"] = (L.lib.woq_last_error() or b"").decode()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["msg"] == ""
    assert "group_size" in (L.lib.woq_last_error() or b"").decode()


def test_grouped_matmul_validation(pkg):
    """woq_grouped_matmul_check: the single-matrix checks on `base` plus the grouping arguments."""
    import ctypes
    L = pkg._lib

    def gstatus(num_experts=4, total=0x7000, activation=L.ACT_IDENTITY, residual=None, **kw):
        g = L.GroupedMatmulArgs(base=make_args(L, **kw), total_rows_before_expert=total, num_experts=num_experts,
                                activation=activation, residual=residual)
        return L.lib.woq_grouped_matmul_check(ctypes.byref(g)), (L.lib.woq_last_error() or b"").decode()

    assert gstatus()[0] == 0
    assert gstatus(m=5000, regime=1)[0] == 0            # streaming passes cover any row count per expert
    assert gstatus(bias=0x5000, quant_algo=L.ALGO_BIAS, group_size=0)[0] == 0
    rc, msg = gstatus(total=None)
    assert rc == -1 and "total_rows_before_expert" in msg
    assert gstatus(total=None, m=0)[0] == 0             # nothing to do, nothing to read
    rc, msg = gstatus(num_experts=0)
    assert rc == -2 and "num_experts" in msg
    rc, msg = gstatus(quant_algo=L.ALGO_FP8_ALPHA, act_dtype=L.FP8_E4M3)
    assert rc == -3 and "not supported" in msg
    rc, msg = gstatus(pre_quant_scale=0x5000, quant_algo=L.ALGO_PRE_QUANT_SCALE)
    assert rc == -3 and "not supported" in msg
    rc, msg = gstatus(k=96)                             # base checks still apply
    assert rc == -2
    assert L.lib.woq_grouped_matmul_check(None) == -1
    # one expert may come without prefix sums; more may not
    assert gstatus(num_experts=1, total=None)[0] == 0
    # activations: every value of the reference's enum; gated ones need n % 32 == 0
    for act in range(6):
        assert gstatus(activation=act, n=256)[0] == 0
    rc, msg = gstatus(activation=6)
    assert rc == -1 and "activation" in msg
    rc, msg = gstatus(activation=L.ACT_SWIGLU, n=48)
    assert rc == -2 and "32" in msg
    assert gstatus(activation=L.ACT_SWIGLU, m=4096, n=256)[0] == 0
    assert gstatus(residual=0xA000)[0] == 0


def test_rmsnorm_prequant_validation(pkg):
    L = pkg._lib
    f = L.lib.woq_rmsnorm_prequant
    err = lambda: (L.lib.woq_last_error() or b"").decode()
    assert f(None, 0x1000, 0x2000, None, None, 1e-5, 4, 64, L.BF16, L.BF16, None) == -1 and "null" in err()
    assert f(0x3000, 0x1000, 0x2000, None, None, 1e-5, 4, 60, L.BF16, L.BF16, None) == -2
    assert f(0x3000, 0x1000, 0x2000, None, None, 1e-5, 4, 64, L.FP8_E4M3, L.BF16, None) == -1
    assert f(0x3000, 0x1000, 0x2000, None, None, 1e-5, 4, 64, L.BF16, L.FP16, None) == -1
    assert f(0x3000, 0x1000, 0x2000, None, None, 1e-5, 0, 64, L.BF16, L.FP8_E4M3, None) == 0  # m == 0: nothing to do


@pytest.mark.gpu
def test_python_wrapper_refuses_operands_of_another_dtype(pkg, dev):
    """The C ABI takes untyped pointers, so the wrapper checks element types: a float32 smoothing vector
    (what an unguarded W4A8 fold returns), bf16 scales next to fp16 activations or a float32 bias would
    otherwise be read as 16-bit values without any error."""
    import torch
    F = pkg.functional
    K, N = 256, 64
    a = torch.zeros(2, K, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(K, N // 2, dtype=torch.int8, device=dev)
    s = torch.ones(K // 128, N, dtype=torch.bfloat16, device=dev)
    kw = dict(n=N, k=K, group_size=128)
    F.woq_matmul_raw(a, None, w, s, None, None, quant_algo=0, **kw)
    with pytest.raises(RuntimeError, match="scales has dtype"):
        F.woq_matmul_raw(a, None, w, s.to(torch.float16), None, None, quant_algo=0, **kw)
    with pytest.raises(RuntimeError, match="pre_quant_scale has dtype"):
        F.woq_matmul_raw(a, torch.ones(K, device=dev), w, s, None, None, quant_algo=F.PRE_QUANT_SCALE, **kw)
    with pytest.raises(RuntimeError, match="bias has dtype"):
        F.woq_matmul_raw(a, None, w, s, None, torch.ones(N, device=dev), quant_algo=F.BIAS, **kw)
    with pytest.raises(RuntimeError, match="zeros has dtype"):
        F.woq_matmul_raw(a, None, w, s, s.float(), None, quant_algo=F.ZERO, **kw)
    with pytest.raises(RuntimeError, match="activation dtype"):
        F.woq_matmul_raw(a.to(torch.float16), None, w, s, None, None, quant_algo=0, out_dtype=torch.bfloat16, **kw)
    # W4A8: float16 scales whatever the output type, or the same bits under the output type's name
    a8 = torch.zeros(2, K, dtype=torch.float8_e4m3fn, device=dev)
    h = torch.ones(K // 128, N, dtype=torch.float16, device=dev)
    for sc in (h, h.view(torch.bfloat16)):
        F.woq_matmul_raw(a8, None, w, sc, None, None, quant_algo=F.FP8_ALPHA, out_dtype=torch.bfloat16, **kw)
    with pytest.raises(RuntimeError, match="scales has dtype"):
        F.woq_matmul_raw(a8, None, w, h.float(), None, None, quant_algo=F.FP8_ALPHA, out_dtype=torch.bfloat16, **kw)
    torch.cuda.synchronize()
