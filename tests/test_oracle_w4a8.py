"""Pins of the oracle's fused int4-dequant GEMM (oracle.torch_w4a8_gemm): it must be the composition of the
two reference-pinned pieces, convert_from_[u]int4 and the fp32-accumulated GEMM, and exact where the
arithmetic is exact."""
import pytest
import torch

from helpers import E4, E5


def problem(gen, M, K, N, group, signed, zp):
    lo, hi = (-8, 8) if signed else (0, 16)
    q = torch.randint(lo, hi, (K, N), generator=gen)
    z = torch.randint(lo, hi, (K // group, N), generator=gen) if zp else None
    return q, z


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("zp", [False, True])
def test_exact_integers_equal_integer_matmul(oracle, signed, zp):
    """Small-integer activations, power-of-two scales: every product and sum is an integer times a power of
    two, so the result is fixed by integer arithmetic alone (a wrong nibble order, sign rule, group index or
    a dropped zero-point would change it)."""
    gen = torch.Generator().manual_seed(5 + signed * 2 + zp)
    M, K, N, group = 9, 256, 64, 64
    q, z = problem(gen, M, K, N, group, signed, zp)
    a = torch.randint(-4, 5, (M, K), generator=gen)
    e = torch.randint(-3, 3, (K // group, N), generator=gen)
    s = torch.exp2(e.float())
    w_int = q - (z.repeat_interleave(group, 0) if zp else 0)                   # int64
    expect = ((a.double() @ (w_int.double() * s.double().repeat_interleave(group, 0))))
    out = oracle.torch_w4a8_gemm(a.float().to(E4), oracle.pack_nibbles(q), s.bfloat16(),
                                 oracle.pack_nibbles(z) if zp else None, signed, torch.float32)
    assert torch.equal(out.double(), expect)


@pytest.mark.parametrize("signed", [False, True])
def test_equals_dequant_then_gemm(oracle, signed):
    """Against the composition of the two pinned oracle functions: c_dequant_4bit to fp32 (exact there) and
    the fp32-accumulated GEMM of the dequantised operands, within fp32 accumulation error."""
    gen = torch.Generator().manual_seed(11)
    M, K, N, group = 17, 512, 96, 128
    q, z = problem(gen, M, K, N, group, signed, True)
    s = (torch.rand(K // group, N, generator=gen) * 0.019 + 0.001).bfloat16()
    a8 = (torch.randn(M, K, generator=gen) * 2).to(E5)
    sa = torch.rand(M, 1, generator=gen) + 0.5
    bias = torch.randn(N, generator=gen).bfloat16()
    w32 = oracle.c_dequant_4bit(oracle.pack_nibbles(q), s.float(), oracle.pack_nibbles(z), torch.float32, signed)
    ref = (a8.float() @ w32) * sa + bias.float()
    out = oracle.torch_w4a8_gemm(a8, oracle.pack_nibbles(q), s, oracle.pack_nibbles(z), signed, torch.float32, sa, bias)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-5 * ref.abs().max().item())
    out16 = oracle.torch_w4a8_gemm(a8, oracle.pack_nibbles(q), s, oracle.pack_nibbles(z), signed, torch.bfloat16, sa, bias)
    assert out16.dtype == torch.bfloat16 and torch.allclose(out16.float(), ref, rtol=1e-2, atol=1e-2 * ref.abs().max().item())


# ------------------------------------------------------------------ W4A16 (bf16 activations)

@pytest.mark.parametrize("signed", [False, True])
def test_w4a16_exact_integers_and_composition(oracle, signed):
    """torch_w4a16_gemm on small-integer bf16 activations equals the integer matmul, and on random ones the
    composition convert_from_[u]int4 (fp32, exact) -> matmul of the dequantised operands."""
    gen = torch.Generator().manual_seed(31 + signed)
    M, K, N, group = 9, 256, 64, 128
    q, z = problem(gen, M, K, N, group, signed, True)
    a = torch.randint(-100, 101, (M, K), generator=gen)
    s = torch.exp2(torch.randint(-3, 3, (K // group, N), generator=gen).float())
    expect = a.double() @ ((q - z.repeat_interleave(group, 0)).double() * s.double().repeat_interleave(group, 0))
    out = oracle.torch_w4a16_gemm(a.bfloat16(), oracle.pack_nibbles(q), s.bfloat16(), oracle.pack_nibbles(z), signed, torch.float32)
    assert torch.equal(out.double(), expect)
    s2 = (torch.rand(K // group, N, generator=gen) * 0.019 + 0.001).bfloat16()
    x = torch.randn(M, K, generator=gen).bfloat16()
    bias = torch.randn(N, generator=gen).bfloat16()
    w32 = oracle.c_dequant_4bit(oracle.pack_nibbles(q), s2.float(), oracle.pack_nibbles(z), torch.float32, signed)
    ref = x.float() @ w32 + bias.float()
    out = oracle.torch_w4a16_gemm(x, oracle.pack_nibbles(q), s2, oracle.pack_nibbles(z), signed, torch.float32, bias)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-5 * ref.abs().max().item())


def test_two_fp8_planes_hold_a_bf16_row(oracle):
    """oracle.split_rows_fp8x2: x s = hi + lo / 16 exactly wherever hi is a normal e4m3fn number (|x s| >= 2^-6: the
    remainder of an 8-bit significand after its leading 4 bits has at most 4), and to within 2^-14 otherwise; s is a
    power of two that puts the row's largest value in (224, 448]."""
    gen = torch.Generator().manual_seed(7)
    x = (torch.randn(6, 4096, generator=gen) * torch.tensor([1e-3, 1.0, 37.0, 1e4, 1e-20, 1.0]).reshape(-1, 1)).bfloat16()
    x[5] = 0
    x[1, :64] *= 1e-6          # elements far below the row's largest
    hi, lo, sinv = oracle.split_rows_fp8x2(x)
    s = 1.0 / sinv.double().reshape(-1, 1)
    p = x.double() * s
    rec = hi.double() + lo.double() / 16
    assert sinv[5] == 1.0 and torch.count_nonzero(hi[5].float()) == 0
    assert (torch.log2(s).round() == torch.log2(s)).all()
    amax = p.abs().amax(dim=1)
    assert ((amax[:5] > 224) & (amax[:5] <= 448)).all()
    normal = p.abs() >= 2.0 ** -6
    assert torch.equal(rec[normal], p[normal])
    assert ((rec - p).abs() <= 2.0 ** -14).all()
    # all 65536 bf16 patterns as one row scaled into range: finite ones are reproduced to the same bound
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    row = allv[torch.isfinite(allv.float()) & (allv.float().abs() <= 448)].reshape(1, -1)
    hi, lo, sinv = oracle.split_rows_fp8x2(row)
    assert sinv[0] == 1.0
    rec = hi.double() + lo.double() / 16
    assert ((rec - row.double()).abs() <= 2.0 ** -14).all()
    big = row.double().abs() >= 2.0 ** -6
    assert torch.equal(rec[big], row.double()[big])
