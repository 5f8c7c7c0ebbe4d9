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
