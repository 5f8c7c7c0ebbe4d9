"""Pins the oracle's 4-bit dequantisation: nibble order, sign, group layout."""
import json
import os

import pytest
import torch

from helpers import assert_bits_equal

HERE = os.path.dirname(os.path.abspath(__file__))


# test_hpu_convert_from_int4.py:41-49 packs by building a binary string with
# element 0 in the lowest 4 bits; restated with integer arithmetic.
def pack_like_reference(values):
    flat = [int(v) & 0xF for v in values]
    words = []
    for b in range(len(flat) // 8):
        w = 0
        for i in range(8):
            w |= flat[b * 8 + i] << (4 * i)
        words.append(w - (1 << 32) if w >= (1 << 31) else w)
    return words


def test_nibble_order_and_sign_brute_force(oracle):
    """Every nibble value in every one of the 8 positions."""
    for pos in range(8):
        for val in range(16):
            q = [0] * 8
            q[pos] = val
            packed = torch.tensor([pack_like_reference(q)], dtype=torch.int32)
            assert torch.equal(packed, oracle.pack_nibbles(torch.tensor([q])))
            s = torch.ones(1, 8)
            u = oracle.c_dequant_4bit(packed, s, None, torch.float32, signed=False)
            i = oracle.c_dequant_4bit(packed, s, None, torch.float32, signed=True)
            eu = [0.0] * 8
            eu[pos] = float(val)
            ei = [0.0] * 8
            ei[pos] = float(val - 16 if val > 7 else val)  # test :104-105
            assert u.tolist() == [eu] and i.tolist() == [ei]


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("zp", ["none", "packed", "float"])
@pytest.mark.parametrize("packed_shape", [(10,), (4, 6, 4)])
def test_elementwise_form_matches_reference_formula(oracle, out_dtype, signed, zp, packed_shape):
    """test_hpu_convert_from_int4.py:74-137: scale (and zero-point) shaped like the output."""
    real = list(packed_shape)
    real[-1] *= 8
    q = torch.randint(0, 16, real, dtype=torch.int32)
    packed = torch.tensor(pack_like_reference(q.flatten().tolist()), dtype=torch.int32).reshape(packed_shape)
    qv = torch.where(q > 7, q - 16, q) if signed else q
    scale = (torch.randn(real) * 50.0).to(out_dtype)
    if zp == "none":
        zt, sub = None, qv.to(out_dtype)
    elif zp == "packed":
        z = torch.randint(1, 5, real, dtype=torch.int32)
        if not signed:
            z = torch.where(z > qv, 0, z)
        zt = torch.tensor(pack_like_reference(z.flatten().tolist()), dtype=torch.int32).reshape(packed_shape)
        sub = (qv - z).to(out_dtype)
    else:
        zt = (torch.randn(real) * 5.0).to(out_dtype)
        sub = qv.to(out_dtype) - zt
    expect = sub * scale
    got = oracle.c_dequant_4bit(packed, scale, zt, out_dtype, signed)
    assert_bits_equal(got, expect, "C oracle vs reference formula")
    twin = oracle.torch_dequant_4bit(packed, scale, zt, out_dtype, signed)
    assert_bits_equal(twin, expect, "torch twin vs reference formula")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("input_values", ["0", "1", "7", "range", "normal"])
@pytest.mark.parametrize("zeros_values", ["none", "0", "1", "8", "range"])
@pytest.mark.parametrize("scale_values", ["1", "range", "range_int", "rand"])
def test_groupwise_form_closed_cases(oracle, out_dtype, input_values, zeros_values, scale_values):
    """The AutoGPTQ grid of test_hpu_convert_from_int4.py:398-476 (64x64, group 16):
    weight[k, n] = scale[k // g, n] * (q[k, n] - zero[k // g, n])  (:224-247)."""
    K = N = 64
    g = 16
    if input_values == "normal":
        q = torch.randint(0, 16, (K, N))
    elif input_values == "range":
        q = (torch.arange(K * N) % 16).reshape(K, N)
    else:
        q = torch.full((K, N), int(input_values))
    G = K // g
    if scale_values == "1":
        s = torch.ones(G, N)
    elif scale_values == "range":
        s = (torch.arange(G * N).reshape(G, N) % 16 + 1) / 10.0
    elif scale_values == "range_int":
        s = (torch.arange(G * N).reshape(G, N) % 16 + 1).float()
    else:
        s = torch.rand(G, N) * 0.02 + 0.001
    s = s.to(out_dtype)
    if zeros_values == "none":
        z, zp = None, None
    else:
        z = (torch.arange(G * N).reshape(G, N) % 16) if zeros_values == "range" else torch.full((G, N), int(zeros_values))
        zp = oracle.pack_nibbles(z)
    packed = oracle.pack_nibbles(q)
    qz = q if z is None else q - z.repeat_interleave(g, dim=0)
    expect = qz.to(out_dtype) * s.repeat_interleave(g, dim=0)
    got = oracle.c_dequant_4bit(packed, s, zp, out_dtype, signed=False)
    assert_bits_equal(got, expect, "group-wise")
    assert_bits_equal(oracle.torch_dequant_4bit(packed, s, zp, out_dtype, False), expect, "twin")
    if zeros_values != "none":
        zf = z.to(out_dtype)
        gotf = oracle.c_dequant_4bit(packed, s, zf, out_dtype, signed=False)
        expf = (q.to(out_dtype) - zf.repeat_interleave(g, dim=0)) * s.repeat_interleave(g, dim=0)
        assert_bits_equal(gotf, expf, "group-wise float zero-point")


def test_bf16_product_is_one_rounding(oracle):
    """(q - z) is a small integer, exact in bf16, so the result is the bf16
    rounding of the exact product: compare with a float64 product."""
    q = torch.randint(0, 16, (128, 64))
    z = torch.randint(0, 16, (1, 64))
    s = (torch.rand(1, 64) * 0.019 + 0.001).bfloat16()
    got = oracle.c_dequant_4bit(oracle.pack_nibbles(q), s, oracle.pack_nibbles(z), torch.bfloat16, False)
    exact = (q - z).double() * s.double()
    assert_bits_equal(got, exact.to(torch.bfloat16), "single rounding")


def test_golden_int4_case(oracle):
    with open(os.path.join(HERE, "golden", "oracle_vectors.json")) as f:
        gd = json.load(f)
    packed = torch.tensor(gd["int4_packed"], dtype=torch.int32)
    zp = torch.tensor(gd["int4_zp_packed"], dtype=torch.int32)
    s = torch.tensor(gd["int4_scale_bf16_bits"], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for key, signed, z in (("int4_uint4_out_bf16_bits", False, zp), ("int4_int4_out_bf16_bits", True, None)):
        exp = torch.tensor(gd[key], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        assert_bits_equal(oracle.c_dequant_4bit(packed, s, z, torch.bfloat16, signed), exp, key)
