"""GPU parity of hpu::cast_to_fp8, hpu::fp8_gemm (the deprecated out-variants) and hpu::cast_to_fp8_hybrid, written after the
reference's own tests of them (tests/pytest_working/eager/test_hpu_fp8_ops.py:34-140)."""
import pytest
import torch

from helpers import E4, FP8_DTYPES, assert_bits_equal, assert_fp8_equal, gemm_errors

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu
FP8_MAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


@pytest.mark.parametrize("dtype", [torch.float, torch.bfloat16])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_cast_to_fp8(oracle, dev, dtype, out_dtype):
    """test_hpu_fp8_ops.py:34-61: cast into caller tensors, amax written in place, cast back exact."""
    g = torch.Generator().manual_seed(3)
    pos = torch.rand(64, 48, generator=g).to(dtype) * 30 + 10
    x = torch.cat((pos, -pos))
    scale = torch.tensor(1.3)
    casted = torch.empty(x.shape, dtype=out_dtype, device=dev)
    amax = torch.tensor(0, dtype=torch.float).to(dev)
    r = ops.cast_to_fp8(x.to(dev), scale.to(dev), False, casted, amax)
    assert r[0].data_ptr() == casted.data_ptr() and r[1].data_ptr() == amax.data_ptr()
    ref, _ = oracle.c_cast_to_fp8(x, scale, out_dtype)
    assert_fp8_equal(casted, ref, out_dtype)
    assert amax.cpu() == x.abs().max().float()
    back = ops.cast_from_fp8(casted, scale.reciprocal().to(dev), dtype)
    assert_bits_equal(back, oracle.c_cast_from_fp8(ref, scale.reciprocal(), dtype))
    # an empty amax tensor switches the reduction off (fp8_ops.cpp:138); no scale means 1
    none = torch.empty(0, device=dev)
    ops.cast_to_fp8(x.to(dev), None, False, casted, none)
    assert_fp8_equal(casted, oracle.c_cast_to_fp8(x, None, out_dtype)[0], out_dtype)
    # a non-contiguous out is filled through a copy
    wide = torch.zeros(x.shape[0], 2 * x.shape[1], dtype=out_dtype, device=dev)
    ops.cast_to_fp8(x.to(dev), scale.to(dev), False, wide[:, ::2], none)
    assert_fp8_equal(wide[:, ::2].contiguous(), ref, out_dtype)
    assert (wide[:, 1::2].view(torch.uint8) == 0).all()


def test_cast_to_fp8_errors(dev):
    x = torch.zeros(4, 4, device=dev)
    none = torch.empty(0, device=dev)
    with pytest.raises(RuntimeError, match="CastToFp8 input must be of float or bfloat16 dtype."):
        ops.cast_to_fp8(x.half(), None, False, torch.empty(4, 4, dtype=E4, device=dev), none)
    with pytest.raises(RuntimeError, match="Input and output must have the same shape"):
        ops.cast_to_fp8(x, None, False, torch.empty(4, 5, dtype=E4, device=dev), none)


@pytest.mark.parametrize("shapeA,shapeB", [((2, 3, 4, 2), (2, 3, 4, 8)), ((24, 12), (24, 36)), ((256, 192), (256, 320))])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("accumulate", [True, False])
@pytest.mark.parametrize("dtype", [torch.float, torch.bfloat16])
@pytest.mark.parametrize("fp8_dtype", FP8_DTYPES)
def test_fp8_gemm(oracle, dev, shapeA, shapeB, bias, accumulate, dtype, fp8_dtype):
    """test_hpu_fp8_ops.py:64-140: trans_A GEMM into `out`, which is also the accumulate input D."""
    g = torch.Generator().manual_seed(4)
    A = (torch.rand(shapeA, generator=g) * 10 + 30.0).to(dtype)
    B = (torch.rand(shapeB, generator=g) * 10 + 30.0).to(dtype)
    sA = FP8_MAX[fp8_dtype] / A.abs().max().float()
    sB = FP8_MAX[fp8_dtype] / B.abs().max().float()
    out_shape = shapeA[:-2] + (shapeA[-1], shapeB[-1])
    bias_t = (torch.rand(out_shape, generator=g) * 10 + 30.0).to(dtype)
    out0 = torch.full(out_shape, 1000.0, dtype=dtype)
    out = out0.to(dev)
    A8, _ = ops.cast_to_fp8_v2(A.to(dev), sA.to(dev), False, False, fp8_dtype)
    B8, _ = ops.cast_to_fp8_v2(B.to(dev), sB.to(dev), False, False, fp8_dtype)
    r = ops.fp8_gemm(A8, True, B8, False, out, dtype, sA.reciprocal().to(dev), sB.reciprocal().to(dev),
                     bias_t.to(dev) if bias else None, accumulate, out)
    assert r.data_ptr() == out.data_ptr()
    ref = oracle.torch_fp8_gemm(A8.cpu(), True, B8.cpu(), False, dtype, sA.reciprocal(), sB.reciprocal(),
                                bias=bias_t if bias else None, D=out0 if accumulate else None)
    rel, ok = gemm_errors(out, ref)
    assert rel <= 1e-2 and ok, rel  # tolerance of the GEMM parity bar: max|out-ref| / max|ref| <= 1e-2
    # and the reference's own, much looser bar against the unquantised product (<= 15 integer percent)
    full = torch.matmul(A.float().transpose(-2, -1), B.float())
    if bias:
        full = full + bias_t.float()
    if accumulate:
        full = full + out0.float()
    assert (((out.cpu().float() - full) / full) * 100).abs().to(torch.int).max() <= 15


@pytest.mark.parametrize("dtype", [torch.float, torch.bfloat16])
@pytest.mark.parametrize("stochastic", [True, False])
@pytest.mark.parametrize("is_amax", [True, False])
@pytest.mark.parametrize("shape,use_152,use_143", [((64, 48), True, True), ((16, 24, 8), True, False),
                                                   ((16, 24, 8), False, True), ((1031,), False, False)])
def test_cast_to_fp8_hybrid(oracle, dev, dtype, stochastic, is_amax, shape, use_152, use_143):
    """test_hpu_fp8_ops_any_mode.py:266-358: one input, an e5m2 and an e4m3fn output with their own scales.
    The e4m3fn output always rounds to nearest (bit-exact vs the oracle); so does the e5m2 output unless
    stochastic, where it must be one of the two neighbours and within the reference's rtol of 0.26."""
    g = torch.Generator().manual_seed(8)
    pos = torch.rand(shape, generator=g).to(dtype) * 30 + 10
    x = torch.cat((pos, -pos))
    s152 = torch.tensor(1.3) if use_152 else None
    s143 = torch.tensor(0.7) if use_143 else None
    torch.manual_seed(5)
    y5, y4, amax = ops.cast_to_fp8_hybrid(x.to(dev), s152.to(dev) if use_152 else None,
                                          s143.to(dev) if use_143 else None, stochastic, is_amax)
    ref4, _ = oracle.c_cast_to_fp8(x, s143, torch.float8_e4m3fn)
    ref5, _ = oracle.c_cast_to_fp8(x, s152, torch.float8_e5m2)
    assert_fp8_equal(y4, ref4, torch.float8_e4m3fn, "e4m3fn output")
    if stochastic:
        p = (x * s152.to(dtype)).float() if use_152 else x.float()
        codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).float()
        grid = torch.unique(codes[torch.isfinite(codes)])
        hi = torch.searchsorted(grid, p.contiguous()).clamp(max=grid.numel() - 1)
        lo = (hi - (grid[hi] != p).long()).clamp(min=0)
        yv = y5.cpu().float()
        assert ((yv == grid[lo]) | (yv == grid[hi])).all()
        assert not torch.equal(yv, ref5.float())
        assert torch.allclose(yv, ref5.float(), rtol=0.26, atol=0.0)
    else:
        assert_fp8_equal(y5, ref5, torch.float8_e5m2, "e5m2 output")
    if is_amax:
        assert amax.cpu() == x.abs().max().float() and amax.dim() == 0
    else:
        assert amax.numel() == 0
