"""Pins the CPU oracle's fp8 casts against the reference's own known answers,
against PyTorch's CPU float8 casts and against what the formats fix."""
import json
import os

import pytest
import torch

from helpers import E4, E5, FP8_DTYPES, assert_bits_equal, assert_fp8_equal

HERE = os.path.dirname(os.path.abspath(__file__))


def golden():
    with open(os.path.join(HERE, "golden", "oracle_vectors.json")) as f:
        return json.load(f)


def all_bf16_patterns():
    return (torch.arange(65536, dtype=torch.int32) << 16).view(torch.float32)


# The reference's test oracle (tests/pytest_working/fp8_utils.py:58-79): add
# "half ulp minus one" plus the odd bit of the kept mantissa, then mask.  Masks
# restated from :23-52.  Valid in the fp8 normal range without overflow.
def reference_closed_form(x, out_dtype):
    if x.dtype == torch.float32:
        it, excessive = torch.int32, (21 if out_dtype == E5 else 20)
        mask = 0x7FE00000 if out_dtype == E5 else 0x7FF00000
    else:
        it, excessive = torch.int16, (5 if out_dtype == E5 else 4)
        mask = 0x7FE0 if out_dtype == E5 else 0x7FF0
    mask_round = (1 << excessive) // 2 - 1
    signs = torch.where(x < 0, -1.0, 1.0).to(x.dtype)
    as_int = x.view(it).to(torch.int64)
    odd = (as_int >> excessive) & 1
    masked = (as_int + mask_round + odd) & mask
    return masked.to(it).view(x.dtype) * signs


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_encode_exhaustive_bf16_patterns_vs_torch_cpu(oracle, out_dtype):
    """any_mode/test_hpu_cast.py:35-55 takes PyTorch's CPU float8 cast as ground
    truth; with an explicit clamp it is the saturating cast."""
    x = all_bf16_patterns()
    got, _ = oracle.c_cast_to_fp8(x, None, out_dtype)
    ref, _ = oracle.torch_cast_to_fp8(x, None, out_dtype)
    assert_fp8_equal(got, ref, out_dtype, "oracle vs torch cpu")


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_encode_random_fp32_bit_patterns_vs_torch_cpu(oracle, out_dtype):
    g = torch.Generator().manual_seed(1)
    x = torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << 20,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    got, _ = oracle.c_cast_to_fp8(x, None, out_dtype)
    ref, _ = oracle.torch_cast_to_fp8(x, None, out_dtype)
    assert_fp8_equal(got, ref, out_dtype, "oracle vs torch cpu")


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_encode_ties_and_neighbours(oracle, out_dtype):
    """Every midpoint between adjacent fp8 values rounds to the even code, and
    one fp32 ulp either side rounds to the nearer one (brute force on the grid)."""
    codes = torch.arange(0, 0x7E if out_dtype == E4 else 0x7B, dtype=torch.uint8)
    lo = codes.view(out_dtype).float()
    hi = (codes + 1).view(out_dtype).float()
    mid = (lo.double() + hi.double()) / 2
    assert torch.equal(mid.float().double(), mid)  # midpoints are exact in fp32
    mid = mid.float()
    even = torch.where(codes % 2 == 0, codes, codes + 1)
    got, _ = oracle.c_cast_to_fp8(mid, None, out_dtype)
    assert torch.equal(got.view(torch.uint8), even)
    below = (mid.view(torch.int32) - 1).view(torch.float32)
    above = (mid.view(torch.int32) + 1).view(torch.float32)
    assert torch.equal(oracle.c_cast_to_fp8(below, None, out_dtype)[0].view(torch.uint8), codes)
    assert torch.equal(oracle.c_cast_to_fp8(above, None, out_dtype)[0].view(torch.uint8), codes + 1)
    # and negated
    assert torch.equal(oracle.c_cast_to_fp8(-mid, None, out_dtype)[0].view(torch.uint8), even | 0x80)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_encode_matches_reference_closed_form(oracle, dtype, out_dtype):
    """The input distribution and expectation of test_hpu_fp8_ops_any_mode.py:53-87."""
    pos = torch.rand(64, 48).to(dtype) * 30 + 10
    x = torch.cat((pos, -pos))
    for scale in (1.0, 1.3):
        st = torch.tensor(scale)
        expect = reference_closed_form(x * st.to(dtype), out_dtype)
        got8, _ = oracle.c_cast_to_fp8(x, st, out_dtype)
        assert torch.equal(got8.float(), expect.float())
        # and the round trip the reference asserts with torch.equal (:130)
        back = oracle.c_cast_from_fp8(got8, st.reciprocal(), dtype)
        assert_bits_equal(back, expect * st.reciprocal().to(dtype), "round trip")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_saturation_known_answers(oracle, dtype):
    """test_hpu_fp8_ops_any_mode.py:224-243, the non-Gaudi2 branch."""
    x = torch.tensor([1000, 500, -500, -1000], dtype=dtype)
    y, _ = oracle.c_cast_to_fp8(x, torch.tensor(1.0), E4)
    assert y.float().tolist() == [448.0, 448.0, -448.0, -448.0]
    x = torch.tensor([100000, 60000, -60000, -100000], dtype=dtype)
    y, _ = oracle.c_cast_to_fp8(x, torch.tensor(1.0), E5)
    assert y.float().tolist() == [57344.0, 57344.0, -57344.0, -57344.0]
    big = x.expand(800, 4).reshape(80, 40)
    y, _ = oracle.c_cast_to_fp8(big, torch.tensor(1.0), E5)
    assert torch.equal(y.float(), torch.tensor([57344.0, 57344.0, -57344.0, -57344.0]).expand(800, 4).reshape(80, 40))


def test_special_values(oracle):
    x = torch.tensor([float("inf"), float("-inf"), float("nan"), 0.0, -0.0, 2.0 ** -10, 2.0 ** -17])
    y4 = oracle.c_cast_to_fp8(x, None, E4)[0].view(torch.uint8).tolist()
    y5 = oracle.c_cast_to_fp8(x, None, E5)[0].view(torch.uint8).tolist()
    # Inf saturates, NaN stays NaN, signed zero kept, e4m3 min subnormal 2^-9:
    # 2^-10 is the tie with zero -> even (0); e5m2 min subnormal 2^-16: 2^-17 ties to 0
    assert y4 == [0x7E, 0xFE, 0x7F, 0x00, 0x80, 0x00, 0x00]
    assert y5 == [0x7B, 0xFB, 0x7F, 0x00, 0x80, 0x14, 0x00]


def test_bf16_input_rounds_scale_and_product_to_bf16(oracle):
    """test :86-87: expected = fp8(input * scale.to(bf16)) in bf16 arithmetic.
    The fp32 route gives different codes on a visible share of inputs, so a
    kernel that multiplies in fp32 only cannot pass."""
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(1 << 16, generator=g) * 3).bfloat16()
    s = torch.tensor(1.3)
    got, _ = oracle.c_cast_to_fp8(x, s, E4)
    twin, _ = oracle.torch_cast_to_fp8(x, s, E4)
    assert_fp8_equal(got, twin, E4, "C oracle vs torch twin")
    fp32_route = (x.float() * s).clamp(-448, 448).to(E4)
    differ = (fp32_route.view(torch.uint8) != got.view(torch.uint8)).float().mean().item()
    assert differ > 0.01, differ


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_amax(oracle, dtype):
    x = (torch.randn(64, 48) * 30).to(dtype)
    _, amax = oracle.c_cast_to_fp8(x, torch.tensor(1.3), E4, is_amax=True)
    assert amax.dim() == 0 and amax.dtype == torch.float32
    assert amax == torch.max(x.abs())  # test :132-134
    _, none = oracle.c_cast_to_fp8(x, None, E4, is_amax=False)
    assert none.numel() == 0 and tuple(none.shape) == (0,)  # fp8_ops.cpp:173-176
    assert torch.equal(oracle.c_amax(x), x.abs().max().float())
    assert torch.equal(oracle.c_amax(x, rowwise=True), x.abs().amax(dim=1).float())
    x[3, 5] = float("nan")
    assert torch.isnan(oracle.c_amax(x))


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_decode_tables(oracle, out_dtype):
    codes = torch.arange(256, dtype=torch.uint8).view(out_dtype)
    for dt in (torch.float32, torch.bfloat16):
        got = oracle.c_cast_from_fp8(codes, None, dt)
        assert_bits_equal(got, codes.to(dt), "decode vs torch cpu")
    # fp8 -> bf16 is exact: going through bf16 loses nothing
    assert_bits_equal(oracle.c_cast_from_fp8(codes, None, torch.bfloat16).float(),
                      oracle.c_cast_from_fp8(codes, None, torch.float32), "bf16 exactness")
    key = "decode_e4m3fn_bits" if out_dtype == E4 else "decode_e5m2_bits"
    gold = torch.tensor(golden()[key], dtype=torch.int64)
    got = oracle.c_cast_from_fp8(codes, None, torch.float32).view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    nan = torch.isnan(codes.float())
    assert torch.equal(got[~nan], gold[~nan])


def test_golden_encode_samples(oracle):
    gd = golden()
    bits = torch.tensor(gd["encode_sample_bf16_bits"], dtype=torch.int32)
    x = (bits << 16).view(torch.float32)
    for dt, key in ((E4, "encode_sample_e4m3fn"), (E5, "encode_sample_e5m2")):
        got, _ = oracle.c_cast_to_fp8(x, None, dt)
        assert_fp8_equal(got, torch.tensor(gd[key], dtype=torch.uint8).view(dt), dt, key)
    allb = all_bf16_patterns()
    finite = torch.isfinite(allb)
    for dt, key in ((E4, "encode_all_finite_bf16_digest_e4m3fn"), (E5, "encode_all_finite_bf16_digest_e5m2")):
        codes = oracle.c_cast_to_fp8(allb, None, dt)[0].view(torch.uint8)[finite].tolist()
        acc = 0
        for c in codes:
            acc = (acc * 257 + c + 1) % (2 ** 61 - 1)
        assert acc == gd[key]


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("axis", [0, 1])
def test_scale_forms_agree(oracle, out_dtype, axis):
    """test :64-83,205-217: tensor, float and float-list scales, per-tensor and per-channel."""
    pos = torch.rand(16, 24, 8).bfloat16() * 30 + 10
    x = torch.cat((pos, -pos))
    a, _ = oracle.c_cast_to_fp8(x, torch.tensor(1.3), out_dtype)
    b, _ = oracle.c_cast_to_fp8(x, 1.3, out_dtype)
    c, _ = oracle.c_cast_to_fp8(x, [1.3], out_dtype)
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert torch.equal(a.view(torch.uint8), c.view(torch.uint8))
    vals = (torch.rand(x.shape[-1 - axis]) * 2.0 + 0.5)
    shape = list(vals.unsqueeze(axis).shape)
    t, _ = oracle.c_cast_to_fp8(x, vals, out_dtype, scale_shape=shape)
    lst, _ = oracle.c_cast_to_fp8(x, vals.tolist(), out_dtype, scale_shape=shape)
    twin, _ = oracle.torch_cast_to_fp8(x, vals, out_dtype, scale_shape=shape)
    assert torch.equal(t.view(torch.uint8), lst.view(torch.uint8))
    assert_fp8_equal(t, twin, out_dtype, "per-channel vs torch twin")
    expect = reference_closed_form(x * vals.unsqueeze(axis).to(x.dtype), out_dtype)
    assert torch.equal(t.float(), expect.float())
    back = oracle.c_cast_from_fp8(t, vals.reciprocal(), torch.bfloat16, scale_shape=shape)
    assert_bits_equal(back, expect * vals.reciprocal().unsqueeze(axis).to(torch.bfloat16), "per-channel round trip")
    with pytest.raises(ValueError, match="is not equal to number of scale_shape elements"):
        oracle.c_cast_to_fp8(x, vals, out_dtype, scale_shape=[3, 1])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
def test_quantize_rows_of_zero_and_tiny_rows(oracle, dtype, out_dtype):
    """Dynamic per-row quantisation caps scale = fp8_max / amax at the largest finite bf16 value:
    a row of zeros gives zero codes (not the NaN of 0 * inf) and a finite, non-zero 1 / scale, a row
    whose amax is so small that the quotient overflows is quantised with the cap, every other row is
    untouched by the cap, and a row holding a NaN keeps a NaN scale."""
    x = torch.zeros(6, 64, dtype=dtype)
    x[1] = torch.linspace(-3, 3, 64).to(dtype)
    x[2, 5] = 1e-38            # 448 / 1e-38 overflows fp32
    x[2, 6] = -5e-39
    x[3, ::2] = 2.5
    x[4, 7] = float("nan")
    x[5, 0] = -0.0
    y, s_inv = oracle.quantize_rows(x, out_dtype)
    codes = y.view(torch.uint8)
    assert torch.equal(codes[0], torch.zeros(64, dtype=torch.uint8))
    assert (codes[5] & 0x7F).eq(0).all()
    cap = oracle.ROW_SCALE_CAP
    assert cap == torch.tensor([0x7F7F0000], dtype=torch.int32).view(torch.float32).item()
    assert torch.isfinite(s_inv[[0, 2, 5]]).all() and (s_inv[[0, 2, 5]] > 0).all()
    assert s_inv[0, 0].item() == (torch.ones(()) / torch.tensor(cap)).item()
    # the capped row: x * cap, saturating, with cast_to_fp8_v2's rounding
    ref2, _ = oracle.c_cast_to_fp8(x[2:3], torch.tensor(cap), out_dtype)
    assert_fp8_equal(y[2:3], ref2, out_dtype)
    assert not torch.isnan(y[2].float()).any() and y[2].float().abs().max() > 0
    # ordinary rows: exactly fp8_max / amax
    mx = oracle.FP8_MAX[out_dtype]
    for r in (1, 3):
        amax = x[r].abs().max().float()
        assert s_inv[r, 0].item() == (torch.ones(()) / (torch.tensor(mx) / amax)).item()
        assert y[r].float().abs().max().item() == mx
    assert torch.isnan(s_inv[4]).all()
