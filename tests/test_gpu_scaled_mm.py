"""GPU parity of mi355q::scaled_mm (aten::_scaled_mm on the fp8 GEMM kernel) against the CPU oracle.

The cases follow the reference's tests/pytest_working/any_mode/test_hpu_scaled_mm.py:120-202
(shapes 12x16 @ 16x24, scales 2.71 / 3.14 / 0.05, bias, mixed operand formats, float / bfloat16 /
fp8 outputs and its tolerances), plus shapes that reach the MFMA kernels, row-wise scales, operand
layouts, and the opt-in replacement of torch._scaled_mm.
"""
import pytest
import torch

from helpers import E4, E5, gemm_errors

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-2, torch.bfloat16: 0.015, E5: 0.25, E4: 0.125}  # the reference's, :190-197


def operands(shape_a, shape_b, dtype_a, dtype_b, gen):
    a = (torch.rand(shape_a, generator=gen) * 5.0).to(dtype_a)
    b = (torch.rand(shape_b, generator=gen) * 10.0).to(dtype_b)
    return a, b


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("scale_result", [True, False])
@pytest.mark.parametrize("dtype", [E5, E4, "mixed"])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, "fp8"])
def test_reference_cases(oracle, dev, bias, scale_result, dtype, out_dtype):
    if scale_result and out_dtype != "fp8":
        pytest.skip("scale_result is applicable only for fp8 output (reference :126)")
    if out_dtype == "fp8" and bias:
        pytest.skip("bias is not supported for fp8 output (reference :130)")
    if out_dtype == "fp8" and not scale_result:
        pytest.skip("fp8 output is applicable only for all scales given (reference :132)")
    dtype_a, dtype_b = (E5, E4) if dtype == "mixed" else (dtype, dtype)
    out_t = dtype_a if out_dtype == "fp8" else out_dtype
    g = torch.Generator().manual_seed(7)
    a, b = operands((12, 16), (16, 24), dtype_a, dtype_b, g)
    sa, sb = torch.tensor(2.71), torch.tensor(3.14)
    sr = torch.tensor(0.05) if scale_result else None
    bias_t = (torch.randn(24, generator=g) * 50.0).to(torch.bfloat16 if out_t != torch.float32 else torch.float32) if bias else None
    out = torch.ops.mi355q.scaled_mm(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev),
                                     bias_t.to(dev) if bias else None, sr.to(dev) if scale_result else None, out_t)
    ref = oracle.torch_scaled_mm(a, b, sa, sb, bias_t, sr, out_t)
    assert out.dtype == out_t and tuple(out.shape) == (12, 24)
    if out_t in (E4, E5):
        # one code apart at most: the fp32 sums differ in their last bits only
        torch.testing.assert_close(out.cpu().float(), ref.float(), atol=1e-3, rtol=RTOL[out_t])
    else:
        torch.testing.assert_close(out.cpu().float(), ref.float(), atol=1e-3, rtol=RTOL[out_t])
        rel, ok = gemm_errors(out, ref)
        assert rel <= 1e-2 and ok


@pytest.mark.parametrize("mat2_layout", ["row_major", "column_major"])
@pytest.mark.parametrize("mat1_layout", ["row_major", "column_major"])
@pytest.mark.parametrize("rowwise", [False, True])
@pytest.mark.parametrize("M,K,N", [(256, 384, 512), (4000, 208, 4112), (48, 1024, 272)])
def test_mfma_kernels_layouts_and_rowwise_scales(oracle, dev, M, K, N, rowwise, mat1_layout, mat2_layout):
    g = torch.Generator().manual_seed(M + K + N)
    a = torch.randint(-4, 5, (M, K), generator=g).float().to(E4)
    b = torch.randint(-4, 5, (K, N), generator=g).float().to(E5)
    sa = (torch.rand(M, 1, generator=g) + 0.5) if rowwise else torch.tensor(0.5)
    sb = (torch.rand(1, N, generator=g) + 0.5) if rowwise else torch.tensor(0.25)
    bias = torch.randn(N, generator=g).bfloat16()
    ad = a.to(dev) if mat1_layout == "row_major" else a.t().contiguous().to(dev).t()
    bd = b.to(dev) if mat2_layout == "row_major" else b.t().contiguous().to(dev).t()
    out = torch.ops.mi355q.scaled_mm(ad, bd, sa.to(dev), sb.to(dev), bias.to(dev), None, torch.bfloat16)
    ref = oracle.torch_scaled_mm(a, b, sa, sb, bias, None, torch.float32)
    rel, ok = gemm_errors(out, ref)
    assert rel <= 1e-2 and ok
    if not rowwise:
        # small-integer operands: every partial sum is exact, so is the scaled result before rounding
        exact = ((a.float() @ b.float()) * 0.125 + bias.float()).bfloat16()
        assert torch.equal(out.cpu(), exact)


def test_fp8_output_saturates(oracle, dev):
    a = torch.full((32, 64), 16.0).to(E4)
    b = torch.full((64, 48), 16.0).to(E4)
    one = torch.tensor(1.0)
    out = torch.ops.mi355q.scaled_mm(a.to(dev), b.to(dev), one.to(dev), one.to(dev), None, None, E4)
    assert torch.equal(out.cpu().float(), torch.full((32, 48), 448.0))
    assert torch.equal(out.cpu().view(torch.uint8), oracle.torch_scaled_mm(a, b, one, one, None, None, E4).view(torch.uint8))


def test_default_out_dtype_is_mat1s(dev):
    a = torch.ones(16, 32).to(E5).to(dev)
    b = torch.ones(32, 16).to(E4).to(dev)
    one = torch.tensor(1.0, device=dev)
    assert torch.ops.mi355q.scaled_mm(a, b, one, one).dtype == E5


def test_errors(dev):
    a = torch.ones(16, 32).to(E4).to(dev)
    b = torch.ones(32, 16).to(E4).to(dev)
    one = torch.tensor(1.0, device=dev)
    with pytest.raises(RuntimeError, match="mat1 must be a matrix"):
        torch.ops.mi355q.scaled_mm(a[0], b, one, one)
    with pytest.raises(RuntimeError, match=r"mat1 and mat2 shapes cannot be multiplied \(16x32 and 16x32\)"):
        torch.ops.mi355q.scaled_mm(a, b.t(), one, one)
    with pytest.raises(RuntimeError, match="Bias must be size 16 but got 3"):
        torch.ops.mi355q.scaled_mm(a, b, one, one, torch.ones(3, device=dev).bfloat16(), None, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Expected mat1 to be Float8_e5m2 or Float8_e4m3fn matrix got"):
        torch.ops.mi355q.scaled_mm(a.float(), b, one, one)


def test_replaces_torch_scaled_mm_on_request(pkg, dev):
    """torch._scaled_mm lands on this package's kernel after use_for_aten_scaled_mm(), and on the
    library's again after use_for_aten_scaled_mm(False)."""
    g = torch.Generator().manual_seed(3)
    a = torch.randn(256, 512, generator=g).to(E4).to(dev)
    b = torch.randn(384, 512, generator=g).to(E4).to(dev).t()   # column-major, as the library wants it
    sa = torch.tensor(0.5, device=dev)
    sb = torch.tensor(2.0, device=dev)
    ours = torch.ops.mi355q.scaled_mm(a, b, sa, sb, None, None, torch.bfloat16)
    try:
        vendor = torch._scaled_mm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
    except RuntimeError:
        vendor = None
    pkg.use_for_aten_scaled_mm()
    try:
        routed = torch._scaled_mm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
        assert torch.equal(routed, ours)
    finally:
        pkg.use_for_aten_scaled_mm(False)
    if vendor is not None:
        again = torch._scaled_mm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
        assert torch.equal(again, vendor)
        rel, ok = gemm_errors(ours, vendor)
        assert rel <= 1e-2
