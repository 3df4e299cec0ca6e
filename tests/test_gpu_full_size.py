"""Parity at the benchmark's full layer shapes (Llama-3-8B and 70B), where the CPU oracle would take
minutes: every (configuration, shape, M) of the benchmark list is run through the C ABI and compared
with a plain torch float32 dequantize-then-matmul on the GPU.  The dequantize follows the oracle's
definition (w = T(q * scale + zero), T = bf16 / fp16; W4A8: both operands rounded to e4m3fn by
torch's own cast, which tests/test_oracle.py shows equal to the oracle's rounding).  Two norms, both
at the benchmark's bar of 1e-2: the global one, max|out - ref| / max|ref|, and a per-output-column one
(max over rows of |out - ref| against the column's largest |ref|, floored by the column's expected
output magnitude so that a column whose few outputs all lie near zero does not divide by nothing).
Size-independent exact properties follow: one-hot activation rows return the dequantized weight
rows, doubling the activations doubles every output bit for bit, permuting activation rows permutes
output rows bit for bit.

Test ids name the benchmark configuration: c2 = W4A16 g128 decode on the 8B shapes, c3 = the same
shapes at prefill row counts (int4 g128 and int8 per-channel), c4 = the 70B shapes with g64 / g128 over
the GEMV-to-GEMM crossover, c5 = W4A8 on the 70B shapes."""
import zlib

import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 1e-2

SHAPES = {
    "8b_qkv": (4096, 6144), "8b_o_proj": (4096, 4096), "8b_gate_up": (4096, 28672), "8b_down": (14336, 4096),
    "70b_qkv": (8192, 10240), "70b_o_proj": (8192, 8192), "70b_gate_up": (8192, 57344), "70b_down": (28672, 8192),
}
TDT = {"bf16": torch.bfloat16, "fp16": torch.float16}
_cache = {}


def _seed(*parts):
    """Reproducible from run to run (Python's own hash() of a string is salted per process)."""
    return zlib.crc32("/".join(str(p) for p in parts).encode()) & 0x7FFFFFFF


def layer(pkg, dev, name, kind="w4", group=128, dtype="bf16"):
    """Seeded random layer of a benchmark shape, built on the GPU.  kind "w4": uint4 with scales
    ~ U(0.002, 0.02) and additive zeros ~ N(0, 0.02) per group; "w8": int8, one scale per column;
    "w4a8": symmetric int4 g128 with fp16 scales sized so that |q * s| reaches into the upper e4m3
    binades without saturating (what the loader's per-tensor fold produces)."""
    key = (name, kind, group, dtype)
    if key not in _cache:
        _cache.clear()  # one layer resident at a time
        torch.cuda.empty_cache()
        F = pkg.functional
        k, n = SHAPES[name]
        t = TDT[dtype]
        bits = 8 if kind == "w8" else 4
        group = 0 if kind == "w8" else group
        g = torch.Generator(device=dev).manual_seed(_seed(name, kind, group, dtype))
        lo = -(1 << (bits - 1))
        q = torch.randint(lo, -lo, (k, n), generator=g, device=dev, dtype=torch.int8)
        gshape = (k // group, n) if group else (n,)
        zeros = None
        if kind == "w4a8":
            scales = (torch.rand(gshape, generator=g, device=dev) * 50 + 2).to(torch.float16)
            algo = F.FP8_ALPHA
        else:
            scales = (torch.rand(gshape, generator=g, device=dev) * 0.018 + 0.002).to(t)
            zeros = (torch.randn(gshape, generator=g, device=dev) * 0.02).to(t) if group else None
            algo = F.ZERO if group else F.INT8_WEIGHT
        if bits == 4:
            packed = ((q[:, 0::2] & 0xF) | (q[:, 1::2] << 4)).to(torch.int8).cpu().contiguous()
            w = pkg.ops.preprocess_weights_for_mixed_gemm(
                packed, torch.quint4x2, torch.float8_e4m3fn if kind == "w4a8" else t).to(dev)
        else:
            w = pkg.ops.preprocess_weights_for_mixed_gemm(q.cpu().contiguous(), torch.int8, t).to(dev)
        # the oracle's dequantize.  bf16 / e4m3: float32 q * s + z (exact product, one float32 rounding),
        # rounded to the type; fp16: one rounding of the exact value, i.e. of the float64 sum
        acc = torch.float64 if dtype == "fp16" and kind != "w4a8" else torch.float32
        if group:
            deq = q.to(acc).view(k // group, group, n) * scales.to(acc)[:, None, :]
            if zeros is not None:
                deq = deq + zeros.to(acc)[:, None, :]
        else:
            deq = q.to(acc) * scales.to(acc)[None, :]
        deq = deq.view(k, n)
        if kind == "w4a8":
            assert deq.abs().max().item() <= 448.0  # no saturation: torch's cast does not saturate
            deq = deq.float().to(torch.float8_e4m3fn)
        else:
            deq = deq.to(t)
        del q
        _cache[key] = dict(k=k, n=n, group=group, weight=w, scales=scales, zeros=zeros, deq=deq, algo=algo,
                           kind=kind, dtype=t, alpha=0.37e-3 if kind == "w4a8" else 1.0)
    return _cache[key]


def run(pkg, L, act, regime=0):
    out = pkg.functional.woq_matmul_raw(act, None, L["weight"], L["scales"], L["zeros"], None, n=L["n"], k=L["k"],
                                        group_size=L["group"], quant_algo=L["algo"], alpha=L["alpha"],
                                        out_dtype=L["dtype"], regime=regime)
    torch.cuda.synchronize()
    return out


def activations(dev, L, m, seed):
    g = torch.Generator(device=dev).manual_seed(_seed("act", seed, m, L["k"]))
    a = torch.randn((m, L["k"]), generator=g, device=dev)
    if L["kind"] == "w4a8":
        # per-tensor scaled into the e4m3 range, as the benchmark's configuration does
        return (a * (448.0 / a.abs().max())).to(torch.float8_e4m3fn)
    return a.to(L["dtype"])


def check_against_torch(pkg, L, act, regime=0):
    out = run(pkg, L, act, regime).float()
    a, w = act.float(), L["deq"].float()
    ref = (a @ w) * L["alpha"]
    err = (out - ref).abs()
    glob = (err.max() / ref.abs().max()).item()
    assert glob < TOL, ("global norm", glob)
    # per output column, floored by sqrt(mean_m sum_k (a w)^2): the column's expected output magnitude
    floor = ((a * a) @ (w * w)).mean(dim=0).sqrt() * abs(L["alpha"])
    col = (err.max(dim=0).values / torch.maximum(ref.abs().max(dim=0).values, floor)).max().item()
    assert col < TOL, ("per-column norm", col)


def _cases():
    out = []
    for s in ("8b_qkv", "8b_o_proj", "8b_gate_up", "8b_down"):
        out += [("c2", s, "w4", 128, "bf16", m) for m in (1, 4, 8, 16)]
        out += [("c3", s, "w4", 128, "bf16", m) for m in (512, 2048, 4096, 8192)]
    for s in ("8b_qkv", "8b_o_proj", "8b_gate_up", "8b_down"):
        out += [("c3", s, "w8", 0, "bf16", m) for m in (512, 2048, 4096, 8192)]
        out += [("c1", s, "w8", 0, "bf16", m) for m in (1, 16)]
    for s in ("70b_qkv", "70b_o_proj", "70b_gate_up", "70b_down"):
        for group in (128, 64):
            out += [("c4", s, "w4", group, "bf16", m) for m in (1, 2, 4, 8, 16, 32, 64, 128, 256)]
    for s in ("70b_qkv", "70b_o_proj", "70b_gate_up", "70b_down"):
        out += [("c5", s, "w4a8", 128, "bf16", m) for m in (1, 16, 32, 256, 4096)]
    # fp16: one case per regime and kernel family (streaming, deferred-scale, exact-dequantize, fp8)
    out += [("fp16", "8b_qkv", "w4", 128, "fp16", m) for m in (1, 16, 48, 4096)]
    out += [("fp16", "70b_o_proj", "w4", 64, "fp16", m) for m in (4, 128)]
    out += [("fp16", "8b_down", "w8", 0, "fp16", m) for m in (1, 512)]
    out += [("fp16", "70b_o_proj", "w4a8", 128, "fp16", m) for m in (1, 256)]
    return out


CASES = _cases()


@pytest.mark.parametrize("cfg,name,kind,group,dtype,m", CASES,
                         ids=["%s-%s-%s-g%d-%s-m%d" % c for c in CASES])
def test_full_size_matches_torch_float32(pkg, dev, cfg, name, kind, group, dtype, m):
    L = layer(pkg, dev, name, kind, group, dtype)
    check_against_torch(pkg, L, activations(dev, L, m, cfg))


def test_torch_e4m3_cast_on_the_gpu_equals_the_cpu_cast(dev):
    """The W4A8 reference above rounds with the GPU's float32 -> e4m3fn cast; the oracle's rounding
    is pinned against the CPU cast: both agree on every float32 bit pattern drawn here, ties and
    subnormals included."""
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(1 << 20, generator=g) * 100, torch.randn(1 << 18, generator=g) * 0.02,
                   torch.arange(-448, 449, dtype=torch.float32) / 1.0, torch.arange(0, 1024, dtype=torch.float32) / 1024])
    x = x.clamp(-448, 448)
    assert torch.equal(x.to(torch.float8_e4m3fn).float(), x.to(dev).to(torch.float8_e4m3fn).float().cpu())


ONE_HOT = [("8b_gate_up", "w4", 128), ("8b_down", "w4", 128), ("70b_gate_up", "w4", 64), ("70b_qkv", "w4", 128),
           ("8b_qkv", "w8", 0)]


@pytest.mark.parametrize("name,kind,group", ONE_HOT)
@pytest.mark.parametrize("regime", [1, 2])
def test_full_size_one_hot_rows_return_weight_rows(pkg, dev, name, kind, group, regime):
    """act = 16 one-hot rows: every output is a single product 1 * w[k, n].  The exact-dequantize
    kernels return bf16(q * s + z) itself; the deferred-scale kernels (16 rows run on them in both
    regimes) form s * (q + OFFSET) + (z - OFFSET * s) in float32, OFFSET = 136 for int4 in bf16: the
    folded constant is rounded at the magnitude of OFFSET * s (<= 2.72 here, half a float32 unit =
    1.2e-7), which shows only where |w| itself is that small.  Allowed: one bf16 unit of w plus that."""
    L = layer(pkg, dev, name, kind, group)
    g = torch.Generator(device=dev).manual_seed(7)
    rows = torch.randint(0, L["k"], (16,), generator=g, device=dev)
    act = torch.zeros((16, L["k"]), dtype=torch.bfloat16, device=dev)
    act[torch.arange(16, device=dev), rows] = 1.0
    out = run(pkg, L, act, regime).float()
    want = L["deq"][rows].float()
    assert ((out - want).abs() <= want.abs() * 2.0 ** -7 + 2.5e-7).all()


@pytest.mark.parametrize("name", ["70b_qkv", "70b_o_proj", "70b_gate_up", "70b_down"])
@pytest.mark.parametrize("m", [16, 24, 256])
def test_full_size_w4a8_one_hot_rows_return_e4m3_weight_rows(pkg, dev, name, m):
    """W4A8 (streaming kernel at 16 rows and, with two row tiles per wavefront, at 24; fp8 GEMM at 256): one-hot rows are exact in e4m3, so row r
    of the output is alpha * (row k_r of the e4m3-rounded dequantized weight), rounded once to bf16 -
    bit for bit, at the full layer shapes."""
    L = layer(pkg, dev, name, "w4a8")
    g = torch.Generator(device=dev).manual_seed(11)
    rows = torch.randint(0, L["k"], (m,), generator=g, device=dev)
    act = torch.zeros((m, L["k"]), dtype=torch.float32, device=dev)
    act[torch.arange(m, device=dev), rows] = 1.0
    out = run(pkg, L, act.to(torch.float8_e4m3fn))
    want = (L["deq"][rows].float() * L["alpha"]).to(torch.bfloat16)
    assert torch.equal(out, want)


EXACT = [("8b_gate_up", "w4", 128, 1), ("8b_gate_up", "w4", 128, 16), ("8b_gate_up", "w4", 128, 4096),
         ("8b_down", "w4", 128, 4), ("8b_down", "w4", 128, 64), ("8b_qkv", "w8", 0, 8192),
         ("70b_down", "w4", 128, 1), ("70b_down", "w4", 128, 16), ("70b_down", "w4", 128, 256),
         ("70b_o_proj", "w4", 64, 8), ("70b_o_proj", "w4a8", 128, 16), ("70b_o_proj", "w4a8", 128, 256)]


@pytest.mark.parametrize("name,kind,group,m", EXACT)
def test_full_size_doubling_and_row_permutation_are_exact(pkg, dev, name, kind, group, m):
    """Scaling by two is exact in every product, sum and rounding, and rows do not interact: both
    properties hold bit for bit whatever the kernel, tile height or K split."""
    L = layer(pkg, dev, name, kind, group)
    act = activations(dev, L, m, "exact")
    if kind == "w4a8":
        act = (act.float() * 0.5).to(torch.float8_e4m3fn)  # room for the doubling below 448
        twice = (act.float() * 2).to(torch.float8_e4m3fn)
        assert torch.equal(twice.float(), act.float() * 2)
    else:
        twice = act * 2
    out = run(pkg, L, act)
    assert torch.equal(run(pkg, L, twice), out * 2)
    if m > 1:
        perm = torch.randperm(m, generator=torch.Generator(device=dev).manual_seed(m), device=dev)
        permuted = act.view(torch.uint8)[perm].contiguous().view(act.dtype) if kind == "w4a8" else act[perm].contiguous()
        assert torch.equal(run(pkg, L, permuted), out[perm])


def test_full_size_regimes_agree(pkg, dev):
    L = layer(pkg, dev, "8b_gate_up")
    act = activations(dev, L, 16, "regimes")
    a, b = run(pkg, L, act, 1).float(), run(pkg, L, act, 2).float()
    assert ((a - b).abs().max() / a.abs().max()).item() < TOL


def test_full_size_config1_literally(pkg, dev):
    """Benchmark configuration 1 as written: M = 1, K = N = 4096, fp16 activations ~ N(0, 1), weights float32
    ~ N(0, 0.02) quantized symmetrically to int8 with one fp16 scale per output column, absmax / 127."""
    k = n = 4096
    g = torch.Generator(device=dev).manual_seed(_seed("c1", k, n))
    w = torch.randn((k, n), generator=g, device=dev) * 0.02
    scale = (w.abs().amax(0) / 127.0).to(torch.float16)
    q = torch.round(w / scale.float()).clamp(-127, 127).to(torch.int8)
    act = torch.randn((1, k), generator=g, device=dev).to(torch.float16)
    F = pkg.functional
    wq = pkg.ops.preprocess_weights_for_mixed_gemm(q.cpu().contiguous(), torch.int8, torch.float16).to(dev)
    out = F.weight_only_quant_matmul(act, wq, scale, F.INT8, "float16")
    torch.cuda.synchronize()
    assert "stream" in (pkg._lib.lib.woq_last_launch() or b"").decode()
    deq = (q.double() * scale.double()[None, :]).to(torch.float16)  # one rounding of the exact product
    ref = act.float() @ deq.float()
    err = (out.float() - ref).abs()
    assert (err.max() / ref.abs().max()).item() < TOL
    floor = ((act.float() ** 2) @ (deq.float() ** 2)).sqrt()
    assert (err / torch.maximum(ref.abs(), floor)).max().item() < TOL


@pytest.mark.parametrize("name", ["70b_down", "70b_gate_up"])
@pytest.mark.parametrize("m", [1, 256, 4096])
def test_full_size_w4a8_smoothing_leg(pkg, dev, name, m):
    """Configuration 5 with its smoothing vector: bf16 activations ~ N(0, 1) and a per-input-channel vector
    ~ U(0.5, 2) (per-tensor scaled into the e4m3 range) go through PRE_QUANT_SCALE | FP8_ALPHA - the smoothing
    pass writes m * k bytes of e4m3 activations to the front of the workspace, the fp8 kernels (and their
    split-K slabs) work behind it.  Reference on the GPU: (bf16(act * pqs) -> e4m3).float() @ deq.float() *
    alpha.  Handing the same e4m3 activations over directly gives the same bits; so does woq_matmul_static
    where its scratch is large enough, which otherwise says so and launches nothing."""
    L = layer(pkg, dev, name, "w4a8")
    F = pkg.functional
    k, n = L["k"], L["n"]
    g = torch.Generator(device=dev).manual_seed(_seed("c5-smooth", name, m))
    act = torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16)
    pqs = torch.rand((k,), generator=g, device=dev) * 1.5 + 0.5
    pqs = (pqs * (440.0 / (act.float() * pqs).abs().max())).to(torch.bfloat16)
    smoothed = (act.float() * pqs.float()).to(torch.bfloat16)  # the product of two bf16 values, rounded once
    assert smoothed.float().abs().max().item() < 464.0          # below the first value that e4m3 cannot hold
    a8 = smoothed.float().to(torch.float8_e4m3fn)
    algo = L["algo"] | F.PRE_QUANT_SCALE
    args = dict(n=n, k=k, group_size=128, quant_algo=algo, alpha=L["alpha"], out_dtype=torch.bfloat16)
    out = F.woq_matmul_raw(act, pqs, L["weight"], L["scales"], None, None, **args)
    torch.cuda.synchronize()
    direct = run(pkg, L, a8)
    assert torch.equal(out, direct)
    ref = (a8.float() @ L["deq"].float()) * L["alpha"]
    err = (out.float() - ref).abs()
    assert (err.max() / ref.abs().max()).item() < TOL
    floor = ((a8.float() ** 2) @ (L["deq"].float() ** 2)).mean(dim=0).sqrt() * abs(L["alpha"])
    assert (err.max(dim=0).values / torch.maximum(ref.abs().max(dim=0).values, floor)).max().item() < TOL
    # the entry point that allocates nothing: same bits, or a clear refusal when m * k bytes (plus the
    # split-K slabs) exceed its scratch
    lib = pkg._lib.lib
    need = lib.woq_workspace_bytes(m, n, k, algo, pkg._lib.BF16)
    fits = m * k <= lib.woq_static_scratch_bytes()
    if fits and need <= lib.woq_static_scratch_bytes():
        got = F.woq_matmul_raw(act, pqs, L["weight"], L["scales"], None, None, static_scratch=True, **args)
        torch.cuda.synchronize()
        assert torch.equal(got, out)
    elif not fits:
        with pytest.raises(RuntimeError, match="static scratch"):
            F.woq_matmul_raw(act, pqs, L["weight"], L["scales"], None, None, static_scratch=True, **args)
