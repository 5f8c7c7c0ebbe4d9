"""GPU parity: cast_to_fp8_v2 / cast_from_fp8 / amax against the CPU oracle, bit exact."""
import ctypes

import pytest
import torch

from helpers import E4, E5, FP8_DTYPES, assert_bits_equal, assert_fp8_equal, c1_input

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


def all_bf16_patterns():
    return (torch.arange(65536, dtype=torch.int32) << 16).view(torch.float32)


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
def test_exhaustive_bf16_patterns(oracle, dev, in_dtype, out_dtype):
    """All 65536 bf16 bit patterns (NaN, Inf, subnormals, both zeros included)."""
    x = all_bf16_patterns().to(in_dtype)
    for scale in (None, 1.0, 0.37, 3.0):
        got, _ = ops.cast_to_fp8_v2(x.to(dev), scale, False, False, out_dtype)
        ref, _ = oracle.c_cast_to_fp8(x, scale, out_dtype)
        assert_fp8_equal(got, ref, out_dtype, f"scale={scale}")


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_random_fp32_bit_patterns(oracle, dev, out_dtype):
    g = torch.Generator().manual_seed(11)
    x = torch.randint(-2 ** 31, 2 ** 31 - 1, ((1 << 20) + 5,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    x = torch.where(torch.isnan(x), torch.zeros_like(x), x)
    got, amax = ops.cast_to_fp8_v2(x.to(dev), torch.tensor(0.75).to(dev), False, True, out_dtype)
    ref, amax_ref = oracle.c_cast_to_fp8(x, 0.75, out_dtype, True)
    assert_fp8_equal(got, ref, out_dtype)
    assert amax.cpu().item() == amax_ref.item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("is_amax", [True, False])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_cast_to_fp8_v2_round_trip(oracle, dev, dtype, is_amax, out_dtype):
    """test_hpu_fp8_ops_any_mode.py:53-147 (RNE cases), shape (64, 48) doubled by the sign cat."""
    pos = torch.rand(64, 48).to(dtype) * 30 + 10
    x = torch.cat((pos, -pos))
    scale = torch.tensor(1.3)
    casted, amax = ops.cast_to_fp8_v2(x.to(dev), scale.to(dev), False, is_amax, out_dtype)
    uncasted = ops.cast_from_fp8(casted, scale.reciprocal().to(dev), dtype, None)
    ref8, ref_amax = oracle.c_cast_to_fp8(x, scale, out_dtype, is_amax)
    assert_fp8_equal(casted, ref8, out_dtype)
    assert_bits_equal(uncasted, oracle.c_cast_from_fp8(ref8, scale.reciprocal(), dtype), "round trip")
    if is_amax:
        assert amax.cpu() == torch.max(x.abs()) and amax.dim() == 0
    else:
        assert amax.numel() == 0 and tuple(amax.shape) == (0,)


@pytest.mark.parametrize("dtype", FP8_DTYPES)
@pytest.mark.parametrize("scale", [None, 1.0])
def test_cast_to_fp8_v2_from_fp8_is_identity(dev, dtype, scale):
    """test :150-176, plus all 256 codes."""
    pos = torch.rand(64, 48) * 30 + 10
    x = torch.cat((pos, -pos)).to(dtype)
    out, _ = ops.cast_to_fp8_v2(x.to(dev), scale, False, False, dtype)
    assert torch.equal(out.cpu().view(torch.uint8), x.view(torch.uint8))
    codes = torch.arange(256, dtype=torch.uint8).view(dtype)
    out, _ = ops.cast_to_fp8_v2(codes.to(dev), scale, False, False, dtype)
    assert torch.equal(out.cpu().view(torch.uint8), codes.view(torch.uint8))


@pytest.mark.parametrize("dtype", FP8_DTYPES)
@pytest.mark.parametrize("dst_dtype", FP8_DTYPES)
@pytest.mark.parametrize("is_amax", [False, True])
def test_cast_to_fp8_v2_from_fp8_exception(dev, dtype, dst_dtype, is_amax):
    """test :179-202."""
    x = torch.rand(16, 24, 8).to(dtype).to(dev)
    if is_amax:
        with pytest.raises(RuntimeError, match="CastToFp8V2 must have no amax for float8."):
            ops.cast_to_fp8_v2(x, None, False, is_amax, dst_dtype)
    elif dtype != dst_dtype:
        with pytest.raises(RuntimeError, match="CastToFp8V2 input and output must have the same dtype for float8, but are"):
            ops.cast_to_fp8_v2(x, 1.0, False, is_amax, dst_dtype)
    else:
        ops.cast_to_fp8_v2(x, 1.0, False, is_amax, dst_dtype)


@pytest.mark.parametrize("mode", ["scalar", "tensor_channel", "scalar_channel"])
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_cast_to_fp8_v2_scales(oracle, dev, mode, axis, out_dtype):
    """test :205-217: scalar, per-channel tensor and per-channel list scales on (16, 24, 8)."""
    pos = torch.rand(16, 24, 8).bfloat16() * 30 + 10
    x = torch.cat((pos, -pos))
    if mode == "scalar":
        s_cpu, s_arg, s_inv_arg, shape = 1.3, 1.3, 1 / 1.3, None
    else:
        vals = (torch.rand(x.shape[-1 - axis]) * 2.0 + 0.5)
        shape = list(vals.unsqueeze(axis).shape)
        s_cpu = vals
        if mode == "tensor_channel":
            s_arg, s_inv_arg = vals.to(dev), vals.reciprocal().to(dev)
        else:
            s_arg, s_inv_arg = vals.tolist(), vals.reciprocal().tolist()
    casted, amax = ops.cast_to_fp8_v2(x.to(dev), s_arg, False, True, out_dtype, shape)
    ref8, _ = oracle.c_cast_to_fp8(x, s_cpu, out_dtype, scale_shape=shape)
    assert_fp8_equal(casted, ref8, out_dtype)
    assert amax.cpu() == x.abs().max()
    back = ops.cast_from_fp8(casted, s_inv_arg, torch.bfloat16, shape)
    inv_cpu = (1 / 1.3) if mode == "scalar" else (vals.reciprocal() if mode == "tensor_channel" else torch.tensor(s_inv_arg))
    assert_bits_equal(back, oracle.c_cast_from_fp8(ref8, inv_cpu, torch.bfloat16, scale_shape=shape), "back")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("big_tensor", [True, False])
def test_cast_to_fp8_v2_out_of_range(dev, dtype, big_tensor):
    """test :220-243: saturation, never Inf/NaN."""
    for out_dtype, vals, mx in ((E5, [100000, 60000, -60000, -100000], 57344.0), (E4, [1000, 500, -500, -1000], 448.0)):
        x = torch.tensor(vals, dtype=dtype)
        expected = torch.tensor([mx, mx, -mx, -mx])
        if big_tensor:
            x = x.expand(800, 4).reshape(80, 40)
            expected = expected.expand(800, 4).reshape(80, 40)
        out, _ = ops.cast_to_fp8_v2(x.to(dev), torch.tensor(1.0).to(dev), False, False, out_dtype)
        assert torch.equal(out.cpu().float(), expected)


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("shape,scale_shape", [
    ((257, 1024), (257, 1)),      # per row, vector kernel
    ((64, 2048), (1, 2048)),      # per column, vector kernel
    ((33, 40), (33, 1)),          # per row, generic kernel
    ((33, 40), (1, 40)),          # per column, generic kernel
    ((3, 5, 64), (3, 1, 64)),     # two separate runs -> expanded to full
    ((6, 50), (6, 50)),           # elementwise
    ((3, 40984), (3, 1)),         # rows of 5123 vectors: several blocks per row, the last one ragged
    ((3, 40984), (1, 40984)),     # the same, per column
    ((3, 40984), (3, 40984)),     # the same, elementwise
    ((3, 40984), None),           # the same, one scale
    ((1031,), None),              # ragged flat tail
    ((0, 8), None),               # empty
])
def test_scale_broadcast_forms(oracle, dev, in_dtype, out_dtype, shape, scale_shape):
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(shape, generator=g) * 40).to(in_dtype)
    if scale_shape is None:
        s = torch.tensor(0.9)
    else:
        s = torch.rand(scale_shape, generator=g) * 2 + 0.25
    got, amax = ops.cast_to_fp8_v2(x.to(dev), s.to(dev), False, True, out_dtype, list(scale_shape) if scale_shape else None)
    ref, amax_ref = oracle.c_cast_to_fp8(x, s, out_dtype, True, scale_shape=list(scale_shape) if scale_shape else None)
    assert_fp8_equal(got, ref, out_dtype)
    assert amax.cpu().item() == amax_ref.item()
    for back_dtype in (torch.float32, torch.bfloat16):
        back = ops.cast_from_fp8(got, s.to(dev), back_dtype, list(scale_shape) if scale_shape else None)
        back_ref = oracle.c_cast_from_fp8(ref, s, back_dtype, scale_shape=list(scale_shape) if scale_shape else None)
        assert_bits_equal(back, back_ref, f"cast_from {back_dtype}")


@pytest.mark.parametrize("fmt", FP8_DTYPES)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_cast_from_fp8_all_codes(oracle, dev, fmt, out_dtype):
    codes = torch.arange(256, dtype=torch.uint8).repeat(37).view(fmt)  # 9472 = not a multiple of 16*256
    for scale in (None, 1.0, 0.3, 1.0 / 448 * 7.5):
        got = ops.cast_from_fp8(codes.to(dev), scale, out_dtype)
        assert_bits_equal(got, oracle.c_cast_from_fp8(codes, scale, out_dtype), f"scale={scale}")


def test_unaligned_views(oracle, dev):
    """A contiguous view that starts 2 bytes off a 16-byte boundary takes the generic kernels."""
    base = (torch.randn(4099) * 20).bfloat16()
    xd = base.to(dev)[1:]
    got, amax = ops.cast_to_fp8_v2(xd, 1.7, False, True, E4)
    ref, amax_ref = oracle.c_cast_to_fp8(base[1:], 1.7, E4, True)
    assert_fp8_equal(got, ref, E4)
    assert amax.cpu().item() == amax_ref.item()
    back = ops.cast_from_fp8(got[3:], 0.5, torch.bfloat16)
    assert_bits_equal(back, oracle.c_cast_from_fp8(ref[3:], 0.5, torch.bfloat16), "unaligned cast_from")


def test_amax_nan_propagates(dev):
    x = torch.randn(5000).bfloat16()
    x[1234] = float("nan")
    _, amax = ops.cast_to_fp8_v2(x.to(dev), None, False, True, E4)
    assert torch.isnan(amax.cpu())
    assert torch.isnan(torch.ops.mi355q.amax(x.float().to(dev)).cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_amax_ops(oracle, dev, dtype):
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(300, 1000, generator=g) * 7).to(dtype)
    assert torch.ops.mi355q.amax(x.to(dev)).cpu() == oracle.c_amax(x)
    assert torch.equal(torch.ops.mi355q.rowwise_amax(x.to(dev)).cpu(), oracle.c_amax(x, rowwise=True))
    y = x[:, :777].contiguous()
    assert torch.equal(torch.ops.mi355q.rowwise_amax(y.to(dev)).cpu(), oracle.c_amax(y, rowwise=True))
    assert torch.ops.mi355q.amax(y.to(dev)).cpu() == oracle.c_amax(y)


def test_config1_full_size(oracle, dev):
    """benchmark configuration 1 at full size: amax, scale = 448/amax, cast, cast back.
    Checked bit-exactly against the PyTorch-CPU twin (multi-threaded; the C
    oracle is pinned to it on smaller inputs) and on a 1/16 slice against C."""
    x = c1_input()
    xd = x.to(dev)
    amax = torch.ops.mi355q.amax(xd)
    assert amax.cpu() == x.abs().max().float()
    scale = (448.0 / amax.cpu()).reshape(())
    y, amax2 = ops.cast_to_fp8_v2(xd, scale.to(dev), False, True, E4)
    assert amax2.cpu() == amax.cpu()
    ref, _ = oracle.torch_cast_to_fp8(x, scale, E4)
    assert_fp8_equal(y, ref, E4, "full size vs torch twin")
    cref, _ = oracle.c_cast_to_fp8(x[:256], scale, E4)
    assert_fp8_equal(y[:256], cref, E4, "slice vs C oracle")
    back = ops.cast_from_fp8(y, scale.reciprocal().to(dev), torch.bfloat16)
    assert_bits_equal(back, oracle.torch_cast_from_fp8(ref, scale.reciprocal(), torch.bfloat16), "cast back")
    # saturation was exercised: the +-1e4 outliers sit at +-448
    assert (y.cpu().float().abs() == 448).sum().item() >= 16778


def test_c_abi_direct(oracle, pkg, dev):
    """Straight through the C ABI with raw device pointers, no torch op in between."""
    lib = pkg.capi()
    x = (torch.randn(128, 512) * 5).bfloat16()
    xd = x.to(dev)
    y = torch.empty(128, 512, dtype=torch.uint8, device=dev)
    amax = torch.full((1,), -1.0, device=dev)
    scale = torch.rand(128) + 0.5
    sd = scale.to(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = lib.mi355q_cast_to_fp8(xd.data_ptr(), pkg.BF16, y.data_ptr(), pkg.E4M3FN, sd.data_ptr(), 0.0,
                                pkg.SCALE_MID, 1, 128, 512, amax.data_ptr(), stream)
    assert st == 0
    torch.cuda.synchronize()
    ref, aref = oracle.c_cast_to_fp8(x, scale, E4, True, scale_shape=[128, 1])
    assert_fp8_equal(y.view(E4), ref, E4)
    assert amax.cpu().item() == aref.item()
    out = torch.empty(128, 512, dtype=torch.float32, device=dev)
    st = lib.mi355q_cast_from_fp8(y.data_ptr(), pkg.E4M3FN, out.data_ptr(), pkg.F32, sd.data_ptr(), 0.0,
                                  pkg.SCALE_MID, 1, 128, 512, stream)
    assert st == 0
    torch.cuda.synchronize()
    assert_bits_equal(out, oracle.c_cast_from_fp8(ref, scale, torch.float32, scale_shape=[128, 1]))
    ra = torch.empty(128, device=dev)
    assert lib.mi355q_rowwise_amax(xd.data_ptr(), pkg.BF16, 128, 512, ra.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(ra.cpu(), x.abs().amax(1).float())


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("dtype,shape", [
    (torch.bfloat16, (16, 8192)),        # decode-shaped activations
    (torch.bfloat16, (513, 4096)),
    (torch.bfloat16, (3, 5, 14336)),     # leading dims are rows
    (torch.bfloat16, (7, 16392)),        # row longer than the one-pass kernel holds: three-step route
    (torch.bfloat16, (9, 100)),          # not a multiple of 8: three-step route
    (torch.float32, (64, 1024)),
    (torch.float32, (5, 8196)),
])
def test_quantize_rows(oracle, pkg, dev, dtype, shape, out_dtype):
    """Dynamic per-row quantisation equals rowwise amax -> target / amax -> cast with per-row scales,
    bit for bit, both against the separate GPU ops and against the oracle."""
    g = torch.Generator().manual_seed(21)
    x = torch.randn(*shape, generator=g)
    x[..., ::97] *= 20
    x = x.to(dtype)
    target = 448.0 if out_dtype == E4 else 57344.0
    y, s_inv = torch.ops.mi355q.quantize_rows(x.to(dev), out_dtype)
    assert y.shape == x.shape and s_inv.shape == x.shape[:-1] + (1,) and s_inv.dtype == torch.float32
    amax = x.abs().amax(-1, keepdim=True).float()
    # tensor / tensor is an IEEE division; torch evaluates scalar / tensor as scalar * (1 / tensor)
    scale = torch.full_like(amax, target) / amax
    x2 = x.reshape(-1, shape[-1])
    ref, _ = oracle.c_cast_to_fp8(x2, scale.reshape(-1), out_dtype, scale_shape=[x2.shape[0], 1])
    assert_fp8_equal(y.reshape(x2.shape), ref, out_dtype, "vs oracle")
    assert torch.equal(s_inv.cpu(), torch.ones_like(scale) / scale)
    amax_d = torch.ops.mi355q.rowwise_amax(x.to(dev)).reshape(-1, 1)
    y3, _ = ops.cast_to_fp8_v2(x2.to(dev), torch.full_like(amax_d, target) / amax_d, False, False, out_dtype, [x2.shape[0], 1])
    assert_fp8_equal(y.reshape(x2.shape), y3.cpu(), out_dtype, "vs the three GPU steps")


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("dtype,cols", [
    (torch.bfloat16, 4096),    # the one-pass kernel
    (torch.bfloat16, 100),     # not whole vectors: rowwise_amax, the division and cast_to_fp8 with per-row scales
    (torch.float32, 1024),
    (torch.float32, 1022),
])
def test_quantize_rows_zero_and_tiny_rows(oracle, dev, dtype, cols, out_dtype):
    """Rows of zeros (padding tokens) among ordinary rows: zero codes and a finite 1 / scale, never the
    NaN codes of 0 * inf; a row whose amax makes fp8_max / amax overflow is quantised with the capped
    scale; both on the fused kernel and on the three-step route, bit for bit as the oracle."""
    g = torch.Generator().manual_seed(cols)
    x = torch.randn(12, cols, generator=g) * 2
    x[0] = 0
    x[5] = 0
    x[5, 3] = -0.0
    x[7] = 0
    x[7, 1] = 1e-38
    x[7, 9] = -3e-39
    x[11] = 0
    x = x.to(dtype)
    y, s_inv = torch.ops.mi355q.quantize_rows(x.to(dev), out_dtype)
    ref, s_ref = oracle.quantize_rows(x, out_dtype)
    assert_fp8_equal(y, ref, out_dtype)
    assert torch.equal(s_inv.cpu(), s_ref)
    assert torch.isfinite(s_inv).all() and not torch.isnan(y.float()).any()
    assert (y.cpu().view(torch.uint8)[[0, 5, 11]] & 0x7F).eq(0).all()
    # a GEMM fed with the zero rows gives zeros there, not NaN
    w = torch.randint(-3, 4, (cols // 16 * 16, 32), generator=g).float().to(E4)
    if cols % 16 == 0:
        out = ops.fp8_gemm_v2(y, False, w.to(dev), False, None, torch.bfloat16, s_inv)
        assert torch.isfinite(out.float()).all() and out[[0, 5, 11]].float().abs().max().item() == 0.0


def test_quantize_rows_c_abi(oracle, pkg, dev):
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x = (torch.randn(33, 2048, generator=torch.Generator().manual_seed(5)) * 3).bfloat16()
    xd = x.to(dev)
    y = torch.empty(x.shape, dtype=E4, device=dev)
    s = torch.empty(33, device=dev)
    si = torch.empty(33, device=dev)
    assert lib.mi355q_quantize_rows(xd.data_ptr(), pkg.BF16, 33, 2048, y.data_ptr(), pkg.E4M3FN, 448.0,
                                    s.data_ptr(), si.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    amax = x.abs().amax(1).float()
    scale = torch.full_like(amax, 448.0) / amax
    assert torch.equal(s.cpu(), scale) and torch.equal(si.cpu(), torch.ones_like(scale) / scale)
    ref, _ = oracle.c_cast_to_fp8(x, scale, E4, scale_shape=[33, 1])
    assert_fp8_equal(y, ref, E4)
    # rows that do not fit one workgroup's registers are refused, not mangled
    assert lib.mi355q_quantize_rows(xd.data_ptr(), pkg.BF16, 1, 33 * 2048, y.data_ptr(), pkg.E4M3FN, 448.0,
                                    None, None, stream) == 2
    assert lib.mi355q_quantize_rows(xd.data_ptr(), pkg.BF16, 0, 2048, y.data_ptr(), pkg.E4M3FN, 448.0,
                                    None, None, stream) == 0


def fp8_grid(dtype):
    """All finite values of an fp8 format, ascending."""
    codes = torch.arange(256, dtype=torch.uint8).view(dtype).float()
    return torch.unique(codes[torch.isfinite(codes)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("is_amax", [True, False])
def test_stochastic_rounding(oracle, dev, dtype, out_dtype, is_amax):
    """stochastic_rounding=True (test_hpu_fp8_ops_any_mode.py:124-128 and test_hpu_fp8_te.py:89-150):
    every output is one of the two fp8 neighbours of the exact scaled value, the result differs from
    round-to-nearest, the mean is preserved, amax is untouched by the rounding mode."""
    g = torch.Generator().manual_seed(31)
    pos = torch.rand(256, 333, generator=g).to(dtype) * 30 + 10
    x = torch.cat((pos, -pos))
    scale = torch.tensor(1.3)
    torch.manual_seed(1234)
    y, amax = ops.cast_to_fp8_v2(x.to(dev), scale.to(dev), True, is_amax, out_dtype)
    p = (x * scale.to(dtype)).float()            # the value that gets rounded (bf16 product for bf16 input)
    grid = fp8_grid(out_dtype)
    hi_i = torch.searchsorted(grid, p.contiguous()).clamp(max=grid.numel() - 1)
    lo_i = (hi_i - (grid[hi_i] != p).long()).clamp(min=0)
    yv = y.cpu().float()
    assert ((yv == grid[lo_i]) | (yv == grid[hi_i])).all()
    rne, _ = oracle.c_cast_to_fp8(x, scale, out_dtype)
    assert not torch.equal(yv, rne.float())
    back = ops.cast_from_fp8(y, scale.reciprocal().to(dev), dtype).cpu()
    ref_back = oracle.c_cast_from_fp8(rne, scale.reciprocal(), dtype)
    assert torch.allclose(back, ref_back, rtol=0.26, atol=0.0)      # the reference's own bound
    if is_amax:
        assert amax.cpu() == x.abs().max().float() and amax.dim() == 0
    else:
        assert amax.numel() == 0
    # reproducible under the torch seed, and successive calls draw fresh bits
    torch.manual_seed(1234)
    y2, _ = ops.cast_to_fp8_v2(x.to(dev), scale.to(dev), True, False, out_dtype)
    y3, _ = ops.cast_to_fp8_v2(x.to(dev), scale.to(dev), True, False, out_dtype)
    assert torch.equal(y2.view(torch.uint8), y.view(torch.uint8))
    assert not torch.equal(y3.view(torch.uint8), y.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt,lo,hi,max_diff", [(E4, 18.0, 20.0, 0.4), (E5, 16.0, 20.0, 0.8)])
def test_stochastic_rounding_is_unbiased(dev, dtype, fmt, lo, hi, max_diff):
    """test_hpu_fp8_te.py:105-150: 18.5 rounds to 18 / 20 (e4m3fn) or 16 / 20 (e5m2) with probabilities
    that keep the mean; here also checked as a rate on 2^18 draws (binomial sigma below 0.001)."""
    x = torch.full((1 << 18,), 18.5, dtype=dtype, device=dev)
    torch.manual_seed(7)
    y = ops.cast_to_fp8_v2(x, None, True, False, fmt)[0].float().cpu()
    assert set(y.unique().tolist()) == {lo, hi}
    assert abs(y[:1000].mean().item() - 18.5) < max_diff
    p_up = (18.5 - lo) / (hi - lo)
    assert abs((y == hi).float().mean().item() - p_up) < 0.01
    rne = ops.cast_to_fp8_v2(x, None, False, False, fmt)[0].float().cpu()
    assert (rne == (18.0 if fmt == E4 else 20.0)).all()
    # values on the fp8 grid are never moved, saturation still applies
    z = torch.tensor([448.0, -448.0, 1e6, -1e6, 0.0, 0.5], dtype=dtype, device=dev)
    zz = ops.cast_to_fp8_v2(z, None, True, False, E4)[0].float().cpu()
    assert zz.tolist() == [448.0, -448.0, 448.0, -448.0, 0.0, 0.5]


def test_stochastic_flush_to_zero(pkg, dev):
    """Round mode SFTZ (GetCastParams, hpu_ops/backend/fp8_ops.cpp:105-119; flag is_sr_sftz, default on:
    scripts/env_flags.yaml:753-758): from bfloat16 to e5m2 a scaled value below 2^-14, the smallest normal e5m2,
    gives a zero of its sign; at and above it the cast rounds stochastically as before.  Other type pairs keep plain
    stochastic rounding (subnormal results occur).  The C entry point takes the mode as an argument."""
    import ctypes
    tiny = torch.tensor([3e-5, -3e-5, 6.0e-5, -1.5e-5, 2.0 ** -14, -(2.0 ** -14), 7.0e-5, 1.0], dtype=torch.bfloat16)
    x = tiny.repeat(4096).to(dev)
    torch.manual_seed(5)
    y = ops.cast_to_fp8_v2(x, None, True, False, E5)[0].cpu().view(-1, 8)
    yf = y.float()
    assert (yf[:, :4] == 0).all() and (y.view(torch.uint8)[:, 1] == 0x80).all() and (y.view(torch.uint8)[:, 0] == 0).all()
    assert (yf[:, 4] == 2.0 ** -14).all() and (yf[:, 5] == -(2.0 ** -14)).all() and (yf[:, 7] == 1.0).all()
    assert set(yf[:, 6].unique().tolist()) == {2.0 ** -14, 2.0 ** -14 * 1.25}      # 7e-5 lies between two normal values
    # fp32 input (and an e4m3fn output) stay plain stochastic rounding: 3e-5 lands on the subnormals 1.5e-5 * {1, 2} ... or 0
    y32 = ops.cast_to_fp8_v2(x.float(), None, True, False, E5)[0].cpu().float().view(-1, 8)
    assert set(y32[:, 0].unique().tolist()) == {2.0 ** -15, 2.0 ** -16 * 3} or set(y32[:, 0].unique().tolist()) <= {2.0 ** -16, 2.0 ** -15, 2.0 ** -16 * 3}
    assert (y32[:, 0] != 0).any()
    # the C entry point: the same input with the mode switched off rounds among the subnormals
    lib = pkg.capi()
    out = torch.empty(x.shape, dtype=E5, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for flush, expect_zero in ((1, True), (0, False)):
        assert lib.mi355q_cast_to_fp8_sr(x.data_ptr(), pkg.BF16, out.data_ptr(), pkg.E5M2, None, 1.0, pkg.SCALE_NONE, x.numel(), 1, 1,
                                         None, 11, 0, flush, st) == 0
        first = out.cpu().float().view(-1, 8)[:, 0]
        assert bool((first == 0).all()) == expect_zero
    # the hybrid cast's e5m2 output follows the same rule for a bfloat16 input
    y5 = ops.cast_to_fp8_hybrid(x, None, None, True, False)[0].cpu().float().view(-1, 8)
    assert (y5[:, :4] == 0).all() and (y5[:, 4] == 2.0 ** -14).all()


def test_cast_more_than_2_31_elements(dev):
    """2^31 + 4104 bf16 elements in one call: indices are 64-bit throughout.  The whole-tensor
    result equals the results of two half-size calls, amax equals torch's, and the cast back
    reproduces the fp8 values."""
    n = 2 ** 31 + 4104
    x = torch.empty(n, dtype=torch.bfloat16, device=dev)
    half = n // 2
    g = torch.Generator(device=dev).manual_seed(3)
    x[:half].normal_(generator=g)
    x[half:].normal_(generator=g)
    x[-1] = 77.0
    scale = torch.tensor(3.0, device=dev)
    y, amax = ops.cast_to_fp8_v2(x, scale, False, True, E4)
    assert amax.item() == x.abs().max().float().item()
    y1, _ = ops.cast_to_fp8_v2(x[:half], scale, False, False, E4)
    y2, _ = ops.cast_to_fp8_v2(x[half:], scale, False, False, E4)
    assert torch.equal(y[:half].view(torch.uint8), y1.view(torch.uint8))
    assert torch.equal(y[half:].view(torch.uint8), y2.view(torch.uint8))
    assert y[-1].float().item() == 224.0  # 77 * 3 = 231 rounds to 224 in e4m3
    del y1, y2, x
    back = ops.cast_from_fp8(y, None, torch.bfloat16)
    assert torch.equal(back[-4096:].float(), y[-4096:].float()) and back.numel() == n
