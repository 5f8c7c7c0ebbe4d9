"""GPU parity: convert_from_int4 / convert_from_uint4 against the CPU oracle, bit exact."""
import pytest
import torch

from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


@pytest.mark.parametrize("packed_shape", [(10,), (4, 6, 4)])
@pytest.mark.parametrize("variant", ["int4", "uint4"])
@pytest.mark.parametrize("zp", ["packed", "float", "none"])
@pytest.mark.parametrize("is_scale", [True, False])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_convert_from_int4(oracle, dev, packed_shape, variant, zp, is_scale, out_dtype):
    """test_hpu_convert_from_int4.py:74-137."""
    fn = getattr(ops, "convert_from_" + variant)
    signed = variant == "int4"
    real = list(packed_shape)
    real[-1] *= 8
    q = torch.randint(0, 16, real, dtype=torch.int32)
    packed = oracle.pack_nibbles(q)
    qv = torch.where(q > 7, q - 16, q) if signed else q
    scale = (torch.randn(real) * 50.0).to(out_dtype) if is_scale else torch.ones(real).to(out_dtype)
    if zp == "packed":
        z = torch.randint(1, 5, real, dtype=torch.int32)
        if not signed:
            z = torch.where(z > qv, 0, z)
        zt = oracle.pack_nibbles(z)
        expect = (qv - z).to(out_dtype) * scale
    elif zp == "float":
        zt = (torch.randn(real) * 5.0).to(out_dtype)
        expect = (qv.to(out_dtype) - zt) * scale
    else:
        zt = None
        expect = qv.to(out_dtype) * scale
    got = fn(packed.to(dev), scale.to(dev), None if zt is None else zt.to(dev), out_dtype)
    assert_bits_equal(got, oracle.c_dequant_4bit(packed, scale, zt, out_dtype, signed), "vs C oracle")
    assert_bits_equal(got, expect, "vs reference formula")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("zeros_values", ["none", "0", "1", "8", "range"])
@pytest.mark.parametrize("scale_values", ["1", "range", "range_int", "rand"])
@pytest.mark.parametrize("input_values", ["0", "1", "7", "range", "normal"])
@pytest.mark.parametrize("packed_zp", [True, False])
def test_convert_from_uint4_groupwise(oracle, dev, out_dtype, zeros_values, scale_values, input_values, packed_zp):
    """The AutoGPTQ grid of test_hpu_convert_from_int4.py:398-476: 64x64, group 16."""
    K = N = 64
    g = 16
    G = K // g
    if input_values == "normal":
        q = torch.randint(0, 16, (K, N))
    elif input_values == "range":
        q = (torch.arange(K * N) % 16).reshape(K, N)
    else:
        q = torch.full((K, N), int(input_values))
    if scale_values == "1":
        s = torch.ones(G, N)
    elif scale_values == "range":
        s = (torch.arange(G * N).reshape(G, N) % 16 + 1) / 10.0
    elif scale_values == "range_int":
        s = (torch.arange(G * N).reshape(G, N) % 16 + 1).float()
    else:
        s = torch.rand(G, N) * 0.02 + 0.001
    s = s.to(out_dtype)
    packed = oracle.pack_nibbles(q)
    if zeros_values == "none":
        zt = None
    else:
        z = (torch.arange(G * N).reshape(G, N) % 16) if zeros_values == "range" else torch.full((G, N), int(zeros_values))
        zt = oracle.pack_nibbles(z) if packed_zp else z.to(out_dtype)
    got = ops.convert_from_uint4(packed.to(dev), s.to(dev), None if zt is None else zt.to(dev), out_dtype)
    assert_bits_equal(got, oracle.c_dequant_4bit(packed, s, zt, out_dtype, False), "group-wise")


@pytest.mark.parametrize("group", [128, 32, 24, 6, 1])
@pytest.mark.parametrize("variant", ["int4", "uint4"])
def test_group_sizes_and_ragged_rows(oracle, dev, group, variant):
    """Groups that are and are not multiples of the rows-per-thread count, rows
    that do not fill the last block."""
    signed = variant == "int4"
    rows = group * 7
    cols = 136 * 8
    g = torch.Generator().manual_seed(group)
    q = torch.randint(0, 16, (rows, cols), generator=g)
    packed = oracle.pack_nibbles(q)
    s = (torch.rand(rows // group, cols, generator=g) * 0.019 + 0.001).bfloat16()
    z = oracle.pack_nibbles(torch.randint(0, 16, (rows // group, cols), generator=g))
    fn = getattr(ops, "convert_from_" + variant)
    got = fn(packed.to(dev), s.to(dev), z.to(dev), torch.bfloat16)
    assert_bits_equal(got, oracle.c_dequant_4bit(packed, s, z, torch.bfloat16, signed), f"group {group}")


def test_config2_full_size(oracle, dev):
    """benchmark configuration 2: K = N = 4096, group 128, bf16 scales U(0.001, 0.02), packed uint4
    zero-points; then int4 with signed nibbles and no zero-point.  Bit exact."""
    g = torch.Generator().manual_seed(0xC001A1)
    K = N = 4096
    q = torch.randint(0, 16, (K, N), generator=g)
    packed = oracle.pack_nibbles(q)
    s = (torch.rand(K // 128, N, generator=g) * 0.019 + 0.001).bfloat16()
    z = torch.randint(0, 16, (K // 128, N), generator=g)
    zp = oracle.pack_nibbles(z)
    pd, sd, zd = packed.to(dev), s.to(dev), zp.to(dev)
    got = ops.convert_from_uint4(pd, sd, zd, torch.bfloat16)
    assert got.shape == (K, N) and got.dtype == torch.bfloat16
    assert_bits_equal(got, oracle.torch_dequant_4bit(packed, s, zp, torch.bfloat16, False), "uint4 vs twin")
    assert_bits_equal(got[:512], oracle.c_dequant_4bit(packed[:512], s[:4], zp[:4], torch.bfloat16, False), "uint4 slice vs C")
    got_i = ops.convert_from_int4(pd, sd, None, torch.bfloat16)
    assert_bits_equal(got_i, oracle.torch_dequant_4bit(packed, s, None, torch.bfloat16, True), "int4 vs twin")
    # size-independent property: out / scale recovers the integers q - z exactly
    rec = (got.cpu().float() / s.float().repeat_interleave(128, 0)).round().long()
    assert torch.equal(rec, q - z.repeat_interleave(128, 0))
