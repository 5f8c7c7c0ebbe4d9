"""mi355q_sum_fp8_static, the entry point that allocates nothing: its partial sums live in a fixed buffer
inside the library's device image instead of a caller's workspace.  Same kernels as mi355q_sum_fp8, so
the outputs must agree bit for bit, also on a second, smaller call that reuses the buffer while it still
holds the first call's partial sums."""
import ctypes

import pytest
import torch

from helpers import E4, E5

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 2 << 20   # MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES


def both(pkg, dev, x8, fmt, outer, red, inner, out_dtype, torch_dtype):
    """(status, output) of mi355q_sum_fp8 with a torch-allocated workspace and of mi355q_sum_fp8_static."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.mi355q_sum_fp8_workspace_bytes(outer, red, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    a = torch.full((outer * inner,), -7.0, device=dev).to(torch_dtype)
    b = torch.full((outer * inner,), -9.0, device=dev).to(torch_dtype)
    st_a = lib.mi355q_sum_fp8(x8.data_ptr(), fmt, outer, red, inner, a.data_ptr(), out_dtype, ws.data_ptr() if need else None,
                              need, stream)
    st_b = lib.mi355q_sum_fp8_static(x8.data_ptr(), fmt, outer, red, inner, b.data_ptr(), out_dtype, stream)
    torch.cuda.synchronize()
    return need, st_a, a, st_b, b


def same_bits(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


def test_two_calls_in_a_row_the_second_smaller(pkg, dev):
    g = torch.Generator().manual_seed(11)
    # columns of [8192, 8192]: 64 slices, exactly 2 MiB of partial sums (the whole buffer)
    x = (torch.randn(8192, 8192, generator=g) * 4).to(E4).to(dev)
    need, st_a, a, st_b, b = both(pkg, dev, x, pkg.E4M3FN, 1, 8192, 8192, pkg.F32, torch.float32)
    assert need == SCRATCH_BYTES and st_a == 0 and st_b == 0
    assert same_bits(a, b)
    assert torch.allclose(b.cpu(), x.cpu().float().sum(0), rtol=1e-5, atol=1e-2)
    # second call, smaller, other format and output type: the buffer still holds the first call's sums
    x2 = (torch.randn(3, 1000, 1536, generator=g) * 2).to(E5).to(dev)
    need2, st_a, a2, st_b, b2 = both(pkg, dev, x2, pkg.E5M2, 3, 1000, 1536, pkg.BF16, torch.bfloat16)
    assert 0 < need2 < need and st_a == 0 and st_b == 0
    assert same_bits(a2, b2)
    assert torch.allclose(b2.cpu().float(), x2.cpu().float().sum(1).reshape(-1), rtol=1e-2, atol=0.5)
    # and the first problem again
    _, _, a3, st_b, b3 = both(pkg, dev, x, pkg.E4M3FN, 1, 8192, 8192, pkg.F32, torch.float32)
    assert st_b == 0 and same_bits(a3, b3) and same_bits(b3, b)


def test_rows_split_and_unsplit(pkg, dev):
    g = torch.Generator().manual_seed(12)
    # long rows: slices of a row, summed by the finish kernel
    x = (torch.randn(8, 1 << 20, generator=g) * 3).to(E4).to(dev)
    need, st_a, a, st_b, b = both(pkg, dev, x, pkg.E4M3FN, 8, 1 << 20, 1, pkg.F32, torch.float32)
    assert need > 0 and st_a == 0 and st_b == 0 and same_bits(a, b)
    # enough rows to fill the chip: no split, the buffer is not touched
    x = (torch.randn(2048, 512, generator=g)).to(E4).to(dev)
    need, st_a, a, st_b, b = both(pkg, dev, x, pkg.E4M3FN, 2048, 512, 1, pkg.E4M3FN, torch.float8_e4m3fn)
    assert need == 0 and st_a == 0 and st_b == 0 and same_bits(a, b)


def test_too_large_is_refused(pkg, dev):
    lib = pkg.capi()
    outer, red, inner = 1, 128, 511 * 1024      # two slices of 523 264 outputs: 4.2 MB of partial sums
    assert lib.mi355q_sum_fp8_workspace_bytes(outer, red, inner) > SCRATCH_BYTES
    x = torch.zeros(red, inner, dtype=torch.uint8, device=dev)
    out = torch.full((inner,), 5.0, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = lib.mi355q_sum_fp8_static(x.data_ptr(), pkg.E4M3FN, outer, red, inner, out.data_ptr(), pkg.F32, stream)
    assert st == 5 and b"scratch" in lib.mi355q_status_string(st)
    torch.cuda.synchronize()
    assert (out == 5.0).all()                   # nothing was launched
    assert lib.mi355q_sum_fp8_static(None, pkg.E4M3FN, 0, 5, 5, None, pkg.F32, stream) == 0
    assert lib.mi355q_sum_fp8_static(x.data_ptr(), 9, 1, 1, 1, out.data_ptr(), pkg.F32, stream) == 1
