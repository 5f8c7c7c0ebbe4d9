"""Pins the oracle's fp8 GEMM: exact small-integer cases, agreement of the C
loops with the PyTorch twin, the reference's scale forms and tolerances."""
import pytest
import torch

from helpers import E4, E5, FP8_DTYPES, gemm_errors


def small_int_fp8(shape, dtype, gen, lo=-4, hi=5):
    return torch.randint(lo, hi, shape, generator=gen).float().to(dtype)


@pytest.mark.parametrize("fa", FP8_DTYPES)
@pytest.mark.parametrize("fb", FP8_DTYPES)
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_exact_small_integers(oracle, fa, fb, ta, tb):
    """Integer-valued operands with K <= 1024 make fp32 accumulation exact, so
    the result must equal the integer matmul bit for bit whatever the order."""
    g = torch.Generator().manual_seed(3)
    M, N, K = 24, 40, 96
    A = small_int_fp8((K, M) if ta else (M, K), fa, g)
    B = small_int_fp8((N, K) if tb else (K, N), fb, g)
    a = A.float().t() if ta else A.float()
    b = B.float().t() if tb else B.float()
    expect = (a.long() @ b.long()).float()
    got = oracle.c_fp8_gemm(A, ta, B, tb, torch.float32)
    assert torch.equal(got, expect)
    twin = oracle.torch_fp8_gemm(A, ta, B, tb, torch.float32)
    assert torch.equal(twin, expect)
    # power-of-two scales stay exact; bias and accumulate inputs are added in fp32
    bias = torch.randint(-8, 8, (N,), generator=g).float()
    D = torch.randint(-8, 8, (M, N), generator=g).float()
    got = oracle.c_fp8_gemm(A, ta, B, tb, torch.float32, 0.5, 4.0, bias=bias, D=D)
    assert torch.equal(got, expect * 2.0 + bias + D)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_c_loops_agree_with_twin(oracle, out_dtype):
    g = torch.Generator().manual_seed(4)
    A = torch.randn(48, 256, generator=g).to(E4)
    B = (torch.randn(256, 80, generator=g) * 0.02).to(E4)
    sa = torch.rand(48, 1, generator=g) + 0.5
    sb = torch.rand(80, generator=g) + 0.5
    bias = (torch.randn(80, generator=g) * 0.01).to(out_dtype)
    c = oracle.c_fp8_gemm(A, False, B, False, out_dtype, sa, sb, bias=bias, B_scale_shape=[1, 80])
    t = oracle.torch_fp8_gemm(A, False, B, False, out_dtype, sa, sb, bias=bias, B_scale_shape=[1, 80])
    rel, ok = gemm_errors(c, t)
    assert ok and rel < 4e-3, rel


@pytest.mark.parametrize("axis", [0, 1])
def test_scale_shape_case_of_reference(oracle, axis):
    """test_hpu_fp8_ops_any_mode.py:599-657: fp8-exact inputs, scalar A scale (list of 1),
    vector B scale broadcast as [M,1] (axis=1) or [1,N] (axis=0), atol=1e-3, rtol=1e-2."""
    A = (torch.rand(12, 24).bfloat16() * 10 + 30.0).to(E4)
    B = (torch.rand(24, 36).bfloat16() * 10 + 30.0).to(E4)
    sa = (torch.rand(1) * 100).tolist()
    n = 12 if axis == 1 else 36
    sbv = (torch.rand(n) * 100)
    sb_t = sbv.unsqueeze(axis)
    ref = torch.matmul(A.to(torch.bfloat16), B.to(torch.bfloat16)) * (torch.tensor(sa) * sb_t)
    got = oracle.c_fp8_gemm(A, False, B, False, torch.bfloat16, sa, sbv.tolist(), B_scale_shape=list(sb_t.shape))
    torch.testing.assert_close(got.float(), ref.float(), atol=1e-3 * ref.abs().max().item(), rtol=1e-2)


@pytest.mark.parametrize("scale_a", [16, 14])
@pytest.mark.parametrize("scale_b", [0.00390625, 0.23])
def test_scalar_scales_case_of_reference(oracle, scale_a, scale_b):
    """test :660-704."""
    A = (torch.rand(12, 24) * 10 + 30.0).to(E4)
    B = (torch.rand(24, 36) * 10 + 30.0).to(E4)
    ref = torch.matmul(A.float(), B.float()) * (scale_a * scale_b)
    got = oracle.c_fp8_gemm(A, False, B, False, torch.float32, float(scale_a), float(scale_b))
    torch.testing.assert_close(got, ref, atol=1e-3, rtol=1e-2)


def test_nan_and_inf_codes_propagate(oracle):
    A = torch.ones(4, 16).to(E5)
    B = torch.ones(16, 4).to(E5)
    A.view(torch.uint8)[1, 3] = 0x7C  # +inf
    A.view(torch.uint8)[2, 5] = 0x7F  # nan
    out = oracle.c_fp8_gemm(A, False, B, False, torch.float32)
    assert torch.isinf(out[1]).all() and torch.isnan(out[2]).all() and (out[0] == 16).all()


def test_scaled_mm_oracle_known_answers(oracle):
    """torch_scaled_mm against hand-computed values, the reference test's own formula
    (any_mode/test_hpu_scaled_mm.py:177, evaluated in bf16 as there) and the fp8_gemm oracle."""
    E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
    a = torch.tensor([[1.0, 2.0]]).to(E4)
    b = torch.tensor([[3.0], [4.0]]).to(E4)
    out = oracle.torch_scaled_mm(a, b, torch.tensor(2.5), torch.tensor(0.5), torch.tensor([1.0]), torch.tensor(2.0), torch.float32)
    assert out.item() == 11 * 2.5 * 0.5 * 2.0 + 1.0
    # default out dtype is mat1's, and an fp8 result saturates instead of overflowing
    big = oracle.torch_scaled_mm(torch.full((2, 8), 16.0).to(E5), torch.full((8, 2), 16.0).to(E4),
                                 torch.tensor(4.0), torch.tensor(8.0))
    assert big.dtype == E5 and torch.equal(big.float(), torch.full((2, 2), 57344.0))
    g = torch.Generator().manual_seed(11)
    a = (torch.rand(12, 16, generator=g) * 5.0).to(E5)
    b = (torch.rand(16, 24, generator=g) * 10.0).to(E4)
    sa, sb = torch.tensor(2.71), torch.tensor(3.14)
    bias = (torch.randn(24, generator=g) * 50.0).bfloat16()
    mine = oracle.torch_scaled_mm(a, b, sa, sb, bias, None, torch.bfloat16)
    theirs = torch.mm(a.bfloat16(), b.bfloat16()) * (sa * sb).bfloat16() * torch.tensor(1.0).bfloat16() + bias
    torch.testing.assert_close(mine, theirs, atol=1e-3, rtol=0.015)
    same = oracle.torch_fp8_gemm(a, False, b, False, torch.bfloat16, sa, sb, bias=bias)
    assert torch.equal(mine, same)
    # row-wise scales broadcast as [M,1] x [1,N]
    ra, rb = torch.rand(12, 1, generator=g) + 0.5, torch.rand(1, 24, generator=g) + 0.5
    rw = oracle.torch_scaled_mm(a, b, ra, rb, None, None, torch.float32)
    assert torch.allclose(rw, (a.float() @ b.float()) * ra * rb, rtol=1e-6)
