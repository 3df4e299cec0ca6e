"""Parity at the benchmark's full layer shapes (Llama-3-8B and 70B), where the CPU oracle would take
minutes: the product is checked through the C ABI against a plain torch float32
dequantize-then-matmul on the GPU (tolerance 1e-2 of max|ref|, the benchmark's bar; the dequantize
follows the oracle's definition w = bf16(q * scale + zero)) and through size-independent exact
properties: one-hot activation rows return the dequantized weight rows, doubling the activations
doubles every output bit for bit, permuting activation rows permutes output rows bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 1e-2

SHAPES = {
    "8b_qkv": (4096, 6144, 128), "8b_o_proj": (4096, 4096, 128), "8b_gate_up": (4096, 28672, 128),
    "8b_down": (14336, 4096, 128), "70b_gate_up_g64": (8192, 57344, 64), "70b_down": (28672, 8192, 128),
}
_cache = {}


def layer(pkg, dev, name, bits=4):
    """Seeded random layer of a benchmark shape, built on the GPU: q uniform over the integer range,
    bf16 scales ~ U(0.002, 0.02), bf16 zeros ~ N(0, 0.02) (per-channel int8: scales only)."""
    key = (name, bits)
    if key not in _cache:
        _cache.clear()  # one layer resident at a time
        torch.cuda.empty_cache()
        k, n, group = SHAPES[name]
        group = group if bits == 4 else 0
        g = torch.Generator(device=dev).manual_seed(hash(name) % 1000 + bits)
        lo = -(1 << (bits - 1))
        q = torch.randint(lo, -lo, (k, n), generator=g, device=dev, dtype=torch.int8)
        gshape = (k // group, n) if group else (n,)
        scales = (torch.rand(gshape, generator=g, device=dev) * 0.018 + 0.002).to(torch.bfloat16)
        zeros = (torch.randn(gshape, generator=g, device=dev) * 0.02).to(torch.bfloat16) if group else None
        if bits == 4:
            packed = ((q[:, 0::2] & 0xF) | (q[:, 1::2] << 4)).to(torch.int8).cpu().contiguous()
            w = pkg.ops.preprocess_weights_for_mixed_gemm(packed, torch.quint4x2, torch.bfloat16).to(dev)
        else:
            w = pkg.ops.preprocess_weights_for_mixed_gemm(q.cpu().contiguous(), torch.int8, torch.bfloat16).to(dev)
        # the oracle's dequantize: float32 q * s + z, rounded to bf16
        if group:
            deq = q.float().view(k // group, group, n) * scales.float()[:, None, :] + zeros.float()[:, None, :]
        else:
            deq = q.float() * scales.float()[None, :]
        deq = deq.view(k, n).to(torch.bfloat16)
        _cache[key] = dict(k=k, n=n, group=group, weight=w, scales=scales, zeros=zeros, deq=deq,
                           algo=(pkg.functional.ZERO if group else pkg.functional.INT8_WEIGHT))
    return _cache[key]


def run(pkg, L, act, regime=0):
    out = pkg.functional.woq_matmul_raw(act, None, L["weight"], L["scales"], L["zeros"], None, n=L["n"], k=L["k"],
                                        group_size=L["group"], quant_algo=L["algo"], out_dtype=torch.bfloat16,
                                        regime=regime)
    torch.cuda.synchronize()
    return out


def activations(dev, m, k, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    return torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16)


CASES = [("8b_qkv", 1), ("8b_qkv", 16), ("8b_qkv", 512), ("8b_o_proj", 1), ("8b_o_proj", 4), ("8b_o_proj", 32),
         ("8b_gate_up", 1), ("8b_gate_up", 8), ("8b_gate_up", 4096), ("8b_down", 1), ("8b_down", 16),
         ("8b_down", 2048), ("70b_gate_up_g64", 1), ("70b_gate_up_g64", 2), ("70b_gate_up_g64", 256),
         ("70b_down", 1), ("70b_down", 64), ("70b_down", 128)]


@pytest.mark.parametrize("name,m", CASES)
def test_full_size_matches_torch_float32(pkg, dev, name, m):
    L = layer(pkg, dev, name)
    act = activations(dev, m, L["k"], m)
    out = run(pkg, L, act).float()
    ref = act.float() @ L["deq"].float()
    err = ((out - ref).abs().max() / ref.abs().max()).item()
    assert err < TOL, err


@pytest.mark.parametrize("name,m", [("8b_gate_up", 1), ("8b_gate_up", 4096), ("8b_down", 16), ("8b_qkv", 2048)])
def test_full_size_int8_per_channel_matches_torch_float32(pkg, dev, name, m):
    L = layer(pkg, dev, name, bits=8)
    act = activations(dev, m, L["k"], m + 1)
    out = run(pkg, L, act).float()
    ref = act.float() @ L["deq"].float()
    err = ((out - ref).abs().max() / ref.abs().max()).item()
    assert err < TOL, err


@pytest.mark.parametrize("name", ["8b_gate_up", "8b_down", "70b_gate_up_g64"])
@pytest.mark.parametrize("regime", [1, 2])
def test_full_size_one_hot_rows_return_weight_rows(pkg, dev, name, regime):
    """act = 16 one-hot rows: every output is a single product 1 * w[k, n].  The exact-dequantize
    kernels return bf16(q * s + z) itself; the deferred-scale kernels (16 rows run on them in both
    regimes) form s * (q + OFFSET) + (z - OFFSET * s) in float32, OFFSET = 136 for int4 in bf16: the
    folded constant is rounded at the magnitude of OFFSET * s (<= 2.72 here, half a float32 unit =
    1.2e-7), which shows only where |w| itself is that small.  Allowed: one bf16 unit of w plus that."""
    L = layer(pkg, dev, name)
    g = torch.Generator(device=dev).manual_seed(7)
    rows = torch.randint(0, L["k"], (16,), generator=g, device=dev)
    act = torch.zeros((16, L["k"]), dtype=torch.bfloat16, device=dev)
    act[torch.arange(16, device=dev), rows] = 1.0
    out = run(pkg, L, act, regime).float()
    want = L["deq"][rows].float()
    assert ((out - want).abs() <= want.abs() * 2.0 ** -7 + 2.5e-7).all()


@pytest.mark.parametrize("name,m", [("8b_gate_up", 1), ("8b_gate_up", 16), ("8b_gate_up", 4096), ("8b_down", 4),
                                    ("8b_down", 64), ("70b_down", 1), ("70b_down", 256)])
def test_full_size_doubling_and_row_permutation_are_exact(pkg, dev, name, m):
    """Scaling by two is exact in every product, sum and rounding, and rows do not interact: both
    properties hold bit for bit whatever the kernel, tile height or K split."""
    L = layer(pkg, dev, name)
    act = activations(dev, m, L["k"], 100 + m)
    out = run(pkg, L, act)
    assert torch.equal(run(pkg, L, act * 2), out * 2)
    if m > 1:
        perm = torch.randperm(m, generator=torch.Generator(device=dev).manual_seed(m), device=dev)
        assert torch.equal(run(pkg, L, act[perm].contiguous()), out[perm])


def test_full_size_regimes_agree(pkg, dev):
    L = layer(pkg, dev, "8b_gate_up")
    act = activations(dev, 16, L["k"], 5)
    a, b = run(pkg, L, act, 1).float(), run(pkg, L, act, 2).float()
    assert ((a - b).abs().max() / a.abs().max()).item() < TOL
