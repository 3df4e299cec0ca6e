"""CPU tests of the product's host side: the C-ABI library loads and exports every symbol the
header declares, and its weight-preparation functions agree with the oracle bit for bit."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "woq.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(woq_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    lib = ctypes.CDLL(pkg.lib_path())
    for name in sorted(declared):
        assert hasattr(lib, name), "libwoq.so does not export %s" % name
    assert declared == set(pkg._lib.EXPORTED), "python binding and header disagree"
    # the measurement probes live in an internal header: in the library, not in the boundary
    probes = open(os.path.join(ROOT, "tensorrt-llm_amd", "csrc", "woq_probes.h")).read()
    probes = set(re.findall(r"\b(woq_[a-z0-9_]+)\s*\(", re.sub(r"/\*.*?\*/", "", probes, flags=re.S)))
    assert probes == set(pkg._lib.PROBES) and not (probes & declared)
    for name in sorted(probes):
        assert hasattr(lib, name), "libwoq.so does not export %s" % name
    assert lib.woq_abi_version() == 1 and lib.woq_layout_version() == 1


def test_matmul_args_struct_layout(pkg):
    # the ctypes mirror must match the C struct: 7 pointers, float + 8 int32, pointer, size_t
    assert ctypes.sizeof(pkg._lib.MatmulArgs) == 7 * 8 + 4 + 8 * 4 + 4 + 8 + 8


def test_pack_unpack_ops(pkg, oracle):
    allb = torch.arange(256, dtype=torch.uint8).view(torch.int8)
    un = pkg.ops.unpack_int4_packed_tensor_to_int8(allb)
    assert (un.numpy() == oracle.unpack_int4_packed_tensor_to_int8(allb.numpy())).all()
    assert (pkg.ops.pack_int8_tensor_to_packed_int4(un) == allb).all()
    with pytest.raises(RuntimeError, match="int4 range"):
        pkg.ops.pack_int8_tensor_to_packed_int4(torch.tensor([8, 0], dtype=torch.int8))
    with pytest.raises(RuntimeError, match="empty"):
        pkg.ops.unpack_int4_packed_tensor_to_int8(torch.zeros(0, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="int8"):
        pkg.ops.unpack_int4_packed_tensor_to_int8(torch.zeros(4, dtype=torch.int16))
    # registered under the reference's torch.ops namespace as well
    assert (torch.ops.trtllm.unpack_int4_packed_tensor_to_int8(allb) == un).all()


@pytest.mark.parametrize("bits,K,N", [(4, 256, 64), (4, 128, 16), (4, 192, 32), (8, 128, 48), (8, 96, 16),
                                      (4, 4096, 128)])
def test_preprocess_matches_oracle_layout(pkg, oracle, bits, K, N):
    rng = np.random.default_rng(K + N + bits)
    q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
    src = torch.from_numpy(q if bits == 8 else oracle.pack_int8_tensor_to_packed_int4(q))
    qt = torch.int8 if bits == 8 else torch.quint4x2
    out = pkg.ops.preprocess_weights_for_mixed_gemm(src, qt, torch.bfloat16)
    assert out.dtype == torch.int8
    assert out.numel() == oracle.gfx950_preprocessed_bytes(K, N, bits)
    if K % (128 if bits == 4 else 64) == 0:
        assert out.shape == src.shape                           # same shape in and out, as in the reference
    assert (out.numpy().view(np.uint8).reshape(-1) == oracle.gfx950_preprocess(q, bits)).all()
    back = pkg.ops.unprocess_weights_for_mixed_gemm(out, K, qt)
    assert (back == src).all()


def test_preprocess_batched_and_checks(pkg, oracle):
    rng = np.random.default_rng(0)
    q = rng.integers(-8, 8, size=(3, 128, 32)).astype(np.int8)
    src = torch.from_numpy(oracle.pack_int8_tensor_to_packed_int4(q))
    out = pkg.ops.preprocess_weights_for_mixed_gemm(src, torch.quint4x2, torch.float16)
    for e in range(3):
        assert (out[e].numpy().view(np.uint8).reshape(-1) == oracle.gfx950_preprocess(q[e], 4)).all()
    with pytest.raises(RuntimeError, match="int8 dtype"):
        pkg.ops.preprocess_weights_for_mixed_gemm(src.to(torch.int16), torch.quint4x2, torch.float16)
    with pytest.raises(RuntimeError, match="int4 or int8"):
        pkg.ops.preprocess_weights_for_mixed_gemm(src, torch.int16, torch.float16)
    with pytest.raises(RuntimeError, match="dim"):
        pkg.ops.preprocess_weights_for_mixed_gemm(src[0, 0], torch.quint4x2, torch.float16)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        pkg.ops.preprocess_weights_for_mixed_gemm(torch.zeros(128, 4, dtype=torch.int8), torch.quint4x2, torch.float16)
    with pytest.raises(RuntimeError, match="multiple of 32"):
        pkg.ops.preprocess_weights_for_mixed_gemm(torch.zeros(48, 16, dtype=torch.int8), torch.int8, torch.float16)


@pytest.mark.parametrize("wdtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("qt,bits", [(torch.int8, 8), (torch.quint4x2, 4)])
def test_symmetric_quantize_matches_oracle(pkg, oracle, wdtype, qt, bits):
    torch.manual_seed(bits)
    w = (torch.randn(128, 64) * 0.02).to(wdtype)
    w[:, 5] = 0                                                  # zero column
    w[3, 9] = w[:, 9].float().abs().max().to(wdtype) * 0.5 ** bits  # w/scale lands on x.5
    un, proc, scales = pkg.ops._symmetric_quantize_last_axis_of_batched_matrix(w, qt)
    dt = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}[wdtype]
    q_ref, s_ref = oracle.symmetric_quantize(w.float().numpy(), bits, dt)
    assert scales.dtype == wdtype and scales.shape == (64,)
    assert (scales.float().numpy() == s_ref).all()
    q_got = un.numpy() if bits == 8 else oracle.unpack_int4_packed_tensor_to_int8(un.numpy())
    assert (q_got == q_ref).all()
    assert un.shape == (128, 64 * bits // 8)
    assert (proc.numpy().view(np.uint8).reshape(-1) == oracle.gfx950_preprocess(q_ref, bits)).all()
    p2, s2 = pkg.ops.symmetric_quantize_last_axis_of_batched_matrix(w, qt)
    assert (p2 == proc).all() and (s2 == scales).all()


def test_symmetric_quantize_batched(pkg, oracle):
    torch.manual_seed(1)
    w = torch.randn(2, 64, 32, dtype=torch.float16)
    un, proc, scales = pkg.ops._symmetric_quantize_last_axis_of_batched_matrix(w, torch.int8)
    assert scales.shape == (2, 32) and un.shape == (2, 64, 32)
    for e in range(2):
        q_ref, s_ref = oracle.symmetric_quantize(w[e].float().numpy(), 8, "fp16")
        assert (un[e].numpy() == q_ref).all() and (scales[e].float().numpy() == s_ref).all()


@pytest.mark.parametrize("name,qt,act", [("W8_A16", torch.int8, torch.float16), ("W4_A16", torch.quint4x2, torch.float16),
                                         ("W4_AFP8", torch.quint4x2, torch.float8_e4m3fn)])
@pytest.mark.parametrize("arch", [80, 89, 90])
def test_import_reference_layout(pkg, oracle, name, qt, act, arch):
    """Bytes laid out the reference's way (oracle restatement) decode back to the row-major input."""
    bits = oracle.weight_bits(name)
    K, N = 256, 128
    rng = np.random.default_rng(arch)
    q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
    raw = oracle.ref_preprocess(q, name, arch)
    ref_t = torch.from_numpy(raw.view(np.int8)).reshape(K, N * bits // 8)
    got = pkg.ops.import_reference_weights(ref_t, qt, act, arch)
    want = q if bits == 8 else oracle.pack_int8_tensor_to_packed_int4(q)
    assert (got.numpy() == want).all()


def test_host_float16_conversions_roundtrip(pkg):
    # the quantizer's host-side fp16/bf16 conversions: scales of an fp16 weight are stored as fp16 RNE
    vals = torch.tensor([65504.0, 1e-7, 6.1e-5, 3.0e-5, 1.0 / 3, 2049.0, 0.0], dtype=torch.float32)
    for dt in (torch.float16, torch.bfloat16):
        w = torch.zeros(32, 16, dtype=torch.float32)
        w[0, : len(vals)] = vals * 8                              # int4 scale = absmax / 8 = vals
        _, scales = pkg.ops.symmetric_quantize_last_axis_of_batched_matrix(w.to(dt), torch.quint4x2)
        expect = ((w.to(dt).float().abs().max(0).values) * 0.125).to(dt)
        assert (scales == expect).all()


def test_every_op_is_reachable_through_torch_ops_trtllm(pkg):
    """The five ops the reference registers for weight preparation (thop/weightOnlyQuantOp.cpp:358-369),
    called the way its conversion scripts and tests call them - by name under torch.ops.trtllm, positional
    arguments, torch dtypes for the ScalarType parameters - give what the python functions give."""
    T = torch.ops.trtllm
    for name in pkg.ops.REGISTERED_TORCH_OPS:
        assert hasattr(T, name), name
    g = torch.Generator().manual_seed(3)
    w = torch.randn((128, 64), generator=g, dtype=torch.float16)
    for qt in (torch.int8, torch.quint4x2):
        processed, scales = T.symmetric_quantize_last_axis_of_batched_matrix(w, qt)
        want = pkg.ops.symmetric_quantize_last_axis_of_batched_matrix(w, qt)
        assert torch.equal(processed, want[0]) and torch.equal(scales, want[1])
        unprocessed, processed2, scales2 = T._symmetric_quantize_last_axis_of_batched_matrix(w, qt)
        assert torch.equal(processed2, processed) and torch.equal(scales2, scales)
        again = T.preprocess_weights_for_mixed_gemm(unprocessed, qt, torch.float16)
        assert torch.equal(again, processed)
    q = torch.randint(-8, 8, (16, 32), generator=g, dtype=torch.int8)
    packed = T.pack_int8_tensor_to_packed_int4(q)
    assert packed.shape == (16, 16) and torch.equal(T.unpack_int4_packed_tensor_to_int8(packed), q)
    # the fp8 activation type selects the W4A8 flavour (get_ft_quant_type, thop/weightOnlyQuantOp.cpp:41-62)
    a8 = T.preprocess_weights_for_mixed_gemm(packed.repeat(8, 2).contiguous(), torch.quint4x2, torch.float8_e4m3fn)
    assert a8.shape == (128, 32)


def _packed(oracle, q, bits):
    return torch.from_numpy(q if bits == 8 else oracle.pack_int8_tensor_to_packed_int4(q))


def _unpacked(oracle, t, bits):
    return t.numpy() if bits == 8 else oracle.unpack_int4_packed_tensor_to_int8(t.numpy())


@pytest.mark.parametrize("name,qt", [("W8_A16", torch.int8), ("W4_A16", torch.quint4x2)])
def test_reference_debug_ops_step_by_step(pkg, oracle, name, qt):
    """The reference's test-only operators (thop/weightOnlyQuantOp.cpp:371-385), called by their
    torch.ops.trtllm names: each step against plain numpy indexing on the unpacked elements, and their
    composition (permute, transpose, bias + word interleave - the reference's order without the column
    interleave, which is what its preprocess does for SM90) against the oracle's byte stream."""
    T = torch.ops.trtllm
    bits = oracle.weight_bits(name)
    K, N = 128, 192
    rng = np.random.default_rng(bits)
    q = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), size=(K, N)).astype(np.int8)
    perm = np.asarray(oracle._PERM[name])
    permuted = T._permute_B_rows_for_mixed_gemm(_packed(oracle, q, bits), qt, 80)
    want = q.reshape(K // perm.size, perm.size, N)[:, perm, :].reshape(K, N)
    assert (_unpacked(oracle, permuted, bits) == want).all()
    transposed = T._subbyte_transpose(permuted, qt)
    assert transposed.shape == permuted.shape  # the reference keeps the tensor shape; the elements are [N][K]
    assert (_unpacked(oracle, transposed.reshape(N, -1), bits) == want.T).all()
    interleave = T._add_bias_and_interleave_int8s if bits == 8 else T._add_bias_and_interleave_int4s
    final = interleave(transposed)
    flat = want.T.reshape(-1).astype(np.int32) + (1 << (bits - 1))
    order = np.asarray(oracle._WORD_ORDER[bits])
    flat = flat.reshape(-1, order.size)[:, order].reshape(-1)
    assert (final.numpy().view(np.uint8).reshape(-1) == oracle._pack_unsigned(flat, bits)).all()
    assert (final.numpy().view(np.uint8).reshape(-1) == oracle.ref_preprocess(q, name, 90)).all()
    # three-dimensional input: every expert on its own
    q3 = np.stack([q, np.roll(q, 1, axis=0)])
    p3 = T._permute_B_rows_for_mixed_gemm(_packed(oracle, q3.reshape(-1, N), bits).reshape(2, K, -1), qt, 80)
    assert torch.equal(p3[0], permuted)
    t3 = T._subbyte_transpose(p3, qt)
    assert torch.equal(t3[0], transposed)
    with pytest.raises(RuntimeError, match="multiple of"):
        T._permute_B_rows_for_mixed_gemm(_packed(oracle, q[:24], bits), qt, 80)
    with pytest.raises(RuntimeError, match="int8"):
        T._subbyte_transpose(torch.zeros((32, 32), dtype=torch.int16), qt)
