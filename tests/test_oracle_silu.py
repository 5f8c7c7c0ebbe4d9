"""Pins of the oracle's SiLU(gate) * up (ora_silu_mul_bf16): exhaustive over the 65536 bf16 inputs
against a double-precision evaluation and against PyTorch's CPU silu, known values, and the
composition with the row quantisation."""
import torch

ALL = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def test_silu_on_every_bf16_value(oracle):
    ones = torch.ones_like(ALL)
    h = oracle.c_silu_mul_bf16(ALL, ones)
    x = ALL.double()
    exact = (x / (1 + torch.exp(-x))).float().bfloat16()
    finite = torch.isfinite(x)
    differ = (h.view(torch.int16) != exact.view(torch.int16)) & finite
    # the spelled-out exp returns -0 where the true result is below 3.3e-37 in magnitude
    assert int(differ.sum()) == 18
    assert (ALL[differ].float() <= -88.5).all() and (h[differ].float() == 0).all()
    assert (exact[differ].float().abs() < 3.3e-37).all()
    # PyTorch's own CPU kernel (float exp from a vector library) agrees everywhere else
    theirs = torch.nn.functional.silu(ALL)
    d2 = (h.view(torch.int16) != theirs.view(torch.int16)) & finite
    assert int(d2.sum()) <= 18 and (ALL[d2].float() <= -88.5).all()
    # NaN in, NaN out; +inf -> +inf; -inf -> NaN (inf / inf), as the formula gives
    assert torch.isnan(h[torch.isnan(ALL.float())].float()).all()
    pinf = ALL.float() == float("inf")
    assert (h[pinf].float() == float("inf")).all()


def test_known_values_and_second_rounding(oracle):
    g = torch.tensor([0.0, 1.0, -1.0, 20.0, -20.0, 3.0]).bfloat16()
    u = torch.tensor([5.0, 2.0, 2.0, 0.5, 1.0, 1.0 / 3.0]).bfloat16()
    h = oracle.c_silu_mul_bf16(g, u).float()
    # silu(1) = 0.731058..., bf16 0.73046875; silu(-1) = -0.268941..., bf16 -0.26953125
    assert h[0] == 0.0 and h[1] == 2 * 0.73046875 and h[2] == 2 * -0.26953125
    assert h[3] == 10.0                        # silu(20) rounds to 20 in bf16
    assert abs(h[4] + 4.1223e-8) < 1e-10       # -20 * exp(-20) / (1 + exp(-20))
    # two roundings: bf16(silu(3)) = 2.859375, times bf16(1/3) = 0.333984375 -> 0.95498..., bf16 0.953125
    assert h[5] == 0.953125
    g2 = torch.randn(64, 257, generator=torch.Generator().manual_seed(3)).bfloat16() * 4
    u2 = torch.randn(64, 257, generator=torch.Generator().manual_seed(4)).bfloat16()
    mine = oracle.c_silu_mul_bf16(g2, u2)
    assert torch.equal(mine, torch.nn.functional.silu(g2) * u2)   # no input below -88 here


def test_quantize_rows_of_the_product(oracle):
    g = (torch.randn(7, 512, generator=torch.Generator().manual_seed(5)) * 3).bfloat16()
    u = torch.randn(7, 512, generator=torch.Generator().manual_seed(6)).bfloat16()
    h = oracle.c_silu_mul_bf16(g, u)
    y, s_inv = oracle.quantize_rows(h, torch.float8_e4m3fn)
    amax = h.float().abs().amax(1, keepdim=True)
    assert torch.allclose(s_inv, amax / 448.0, rtol=1e-6)
    back = y.float() * s_inv
    # e4m3 keeps 3 mantissa bits: half a step is 1/16 of the value (the bf16 rounding of the scaled
    # product adds a little), and 2^-9 in scaled units below the normal range
    assert ((back - h.float()).abs() <= h.float().abs() * 0.066 + amax / 448.0 * 2.0 ** -9).all()
    assert (y.float().abs().amax(1) == 448.0).all()                        # the row maximum maps onto the top code
