"""GPU parity of mi355q::silu_mul_quantize_rows (SiLU(gate) * up in bf16 fused with the dynamic
per-row quantisation) against the CPU oracle: bit-exact, the fp8 codes and the inverse scales."""
import ctypes

import pytest
import torch

from helpers import E4, E5, FP8_DTYPES

pytestmark = pytest.mark.gpu

ALL = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def same_codes(a, b):
    return torch.equal(a.cpu().view(torch.uint8), b.cpu().view(torch.uint8))


def test_silu_bits_on_every_bf16_value(oracle, pkg, dev):
    """h_out of the C entry point for all 65536 gate values (up = 1 and up = an odd constant)."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for upv in (1.0, -0.337890625):
        g = ALL.reshape(32, 2048)
        u = torch.full_like(g, upv)
        gd, ud = g.to(dev), u.to(dev)
        y = torch.empty(g.shape, dtype=E4, device=dev)
        h = torch.empty(g.shape, dtype=torch.bfloat16, device=dev)
        assert lib.mi355q_silu_mul_quantize_rows(gd.data_ptr(), 2048, ud.data_ptr(), 2048, 32, 2048, y.data_ptr(),
                                                 pkg.E4M3FN, 448.0, h.data_ptr(), None, None, stream) == 0
        torch.cuda.synchronize()
        ref = oracle.c_silu_mul_bf16(g, u)
        nan = torch.isnan(ref.float())
        assert torch.equal(torch.isnan(h.cpu().float()), nan)
        assert torch.equal(h.cpu().view(torch.int16)[~nan], ref.view(torch.int16)[~nan])


@pytest.mark.parametrize("cols", [2048, 8192])
def test_table_kernel_on_every_bf16_value(oracle, pkg, dev, cols):
    """From 2048 rows on, bf16(silu(gate)) comes from a table in LDS with range fix-ups outside it:
    every one of the 65536 gate values, in every lane position, against the oracle (h_out, codes and
    scales); rows of zeros and a ragged last workgroup share included."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rows = 2048 + 7
    gen = torch.Generator().manual_seed(cols)
    g = ALL[torch.randperm(65536, generator=gen)].repeat(-(-rows * cols // 65536))[: rows * cols].reshape(rows, cols).clone()
    # NaN, -inf and gates whose product overflows make a row's scale NaN: keep them to the first 64 rows
    bad = torch.isnan(g.float()) | torch.isinf(g.float()) | (g.float().abs() > 1e30)
    bad[:64] = False
    g[bad] = 0.75
    u = torch.randn(rows, cols, generator=gen).bfloat16()
    u[5] = 0
    u[:, ::3] = 1.0
    gd, ud = g.to(dev), u.to(dev)
    y = torch.empty(g.shape, dtype=E4, device=dev)
    h = torch.empty(g.shape, dtype=torch.bfloat16, device=dev)
    si = torch.empty(rows, device=dev)
    assert lib.mi355q_silu_mul_quantize_rows(gd.data_ptr(), cols, ud.data_ptr(), cols, rows, cols, y.data_ptr(),
                                             pkg.E4M3FN, 448.0, h.data_ptr(), None, si.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    ref = oracle.c_silu_mul_bf16(g, u)
    nan = torch.isnan(ref.float())
    assert torch.equal(torch.isnan(h.cpu().float()), nan)
    assert torch.equal(h.cpu().view(torch.int16)[~nan], ref.view(torch.int16)[~nan])
    # rows without a NaN: codes and scales as the oracle's
    clean = ~nan.any(dim=1)
    assert clean.sum() > 100
    ref_y, ref_s = oracle.quantize_rows(ref[clean], E4)
    assert same_codes(y.cpu()[clean], ref_y)
    assert torch.equal(si.cpu()[clean], ref_s.reshape(-1))


@pytest.mark.parametrize("out_dtype", FP8_DTYPES)
@pytest.mark.parametrize("shape", [(64, 1024), (33, 2048), (5, 14336), (3, 8), (16, 16384), (2050, 1032), (2048, 14336)])
def test_against_oracle(oracle, dev, shape, out_dtype):
    gen = torch.Generator().manual_seed(shape[0] * 131 + shape[1])
    g = (torch.randn(*shape, generator=gen) * 3).bfloat16()
    u = torch.randn(*shape, generator=gen).bfloat16()
    g[:, ::97] *= 10
    y, s_inv = torch.ops.mi355q.silu_mul_quantize_rows(g.to(dev), u.to(dev), out_dtype)
    assert y.shape == g.shape and y.dtype == out_dtype and s_inv.shape == (shape[0], 1)
    ref_y, ref_s = oracle.quantize_rows(oracle.c_silu_mul_bf16(g, u), out_dtype)
    assert same_codes(y, ref_y)
    assert torch.equal(s_inv.cpu(), ref_s)


def test_zero_rows(oracle, dev):
    """SiLU(gate) * up rows that are all zero (up = 0, or gate = 0) among ordinary rows: zero codes
    and a finite 1 / scale as the oracle gives them, no NaN."""
    gen = torch.Generator().manual_seed(4)
    g = (torch.randn(9, 2048, generator=gen) * 3).bfloat16()
    u = torch.randn(9, 2048, generator=gen).bfloat16()
    u[0] = 0
    g[4] = 0
    u[8] = 0
    for out_dtype in FP8_DTYPES:
        y, s_inv = torch.ops.mi355q.silu_mul_quantize_rows(g.to(dev), u.to(dev), out_dtype)
        ref_y, ref_s = oracle.quantize_rows(oracle.c_silu_mul_bf16(g, u), out_dtype)
        assert same_codes(y, ref_y) and torch.equal(s_inv.cpu(), ref_s)
        assert torch.isfinite(s_inv).all() and not torch.isnan(y.float()).any()
        assert (y.cpu().view(torch.uint8)[[0, 4, 8]] & 0x7F).eq(0).all()


def test_halves_of_one_wide_matrix(oracle, dev):
    """gate and up as column ranges of one [T, 2 ff] GEMM output (row pitch 2 ff)."""
    gen = torch.Generator().manual_seed(9)
    gu = (torch.randn(48, 2 * 1536, generator=gen) * 2).bfloat16()
    d = gu.to(dev)
    y, s_inv = torch.ops.mi355q.silu_mul_quantize_rows(d[:, :1536], d[:, 1536:], E4)
    ref_y, ref_s = oracle.quantize_rows(oracle.c_silu_mul_bf16(gu[:, :1536].contiguous(), gu[:, 1536:].contiguous()), E4)
    assert same_codes(y, ref_y) and torch.equal(s_inv.cpu(), ref_s)
    # equals the unfused route on the device, where aten's silu agrees with the oracle's
    h = torch.nn.functional.silu(d[:, :1536]) * d[:, 1536:]
    y2, s2 = torch.ops.mi355q.quantize_rows(h, E4)
    assert (y.view(torch.uint8) != y2.view(torch.uint8)).float().mean().item() < 1e-3


def test_shapes_the_kernel_refuses_take_the_aten_route(dev):
    g = torch.randn(4, 20, device=dev).bfloat16()        # 20 columns: not whole 16-byte vectors
    u = torch.randn(4, 20, device=dev).bfloat16()
    y, s_inv = torch.ops.mi355q.silu_mul_quantize_rows(g, u, E5)
    y2, s2 = torch.ops.mi355q.quantize_rows(torch.nn.functional.silu(g) * u, E5)
    assert same_codes(y, y2) and torch.equal(s_inv, s2)


def test_argument_checks(dev):
    g = torch.randn(4, 16, device=dev)
    with pytest.raises(RuntimeError, match="inputs must be bfloat16"):
        torch.ops.mi355q.silu_mul_quantize_rows(g, g, E4)
    b = g.bfloat16()
    with pytest.raises(RuntimeError, match="two matrices of the same shape"):
        torch.ops.mi355q.silu_mul_quantize_rows(b, b[:, :8], E4)
    with pytest.raises(RuntimeError, match="dtype must be float8_e4m3fn or float8_e5m2"):
        torch.ops.mi355q.silu_mul_quantize_rows(b, b, torch.bfloat16)
