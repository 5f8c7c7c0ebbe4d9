"""fp8_gemm_v2 on large products whose extents are not multiples of 16: the operator copies such
operands into zero-padded buffers so that the MFMA kernels serve them (the any-shape kernel runs
at a few TFLOP/s).  Operands are small integers, so the result is exact whatever the kernel."""
import pytest
import torch

from helpers import E4, E5

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


@pytest.mark.parametrize("M,K,N", [
    (1000, 1000, 500),    # K % 16 = 8, N % 16 = 4
    (301, 1001, 1003),    # nothing a multiple of 2
    (520, 1024, 1001),    # only N ragged
    (515, 1024, 1008),    # only M ragged
    (512, 1030, 512),     # only K ragged
    (70, 4100, 1999),     # few rows: the strip kernel
])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_ragged_large_products_are_exact(dev, M, K, N, ta, tb):
    g = torch.Generator().manual_seed(M + K + N)
    A = torch.randint(-4, 5, (K, M) if ta else (M, K), generator=g).float()
    B = torch.randint(-4, 5, (N, K) if tb else (K, N), generator=g).float()
    # the last k and the last m / n carry weight: a chunk dropped at an edge changes the result
    (A[-1] if ta else A[:, -1]).fill_(4.0)
    (B[:, -1] if tb else B[-1]).fill_(3.0)
    sa = (torch.randint(1, 5, (M, 1), generator=g).float() * 0.25)
    sb = (torch.randint(1, 5, (N,), generator=g).float() * 0.25)
    bias = torch.randint(-8, 9, (N,), generator=g).float()
    ref = ((A.t() if ta else A) @ (B.t() if tb else B)) * sa * sb + bias
    for out_dtype, fa, fb in ((torch.bfloat16, E4, E4), (torch.float32, E5, E4)):
        out = ops.fp8_gemm_v2(A.to(fa).to(dev), ta, B.to(fb).to(dev), tb, None, out_dtype, sa.to(dev), sb.to(dev),
                              bias.to(out_dtype).to(dev), False, [1, N])
        assert out.shape == (M, N) and out.dtype == out_dtype
        assert torch.equal(out.cpu().float(), ref.to(out_dtype).float()), (M, K, N, ta, tb, out_dtype)


def test_ragged_batched_and_accumulate(dev):
    g = torch.Generator().manual_seed(5)
    b, M, K, N = 3, 333, 777, 555
    A = torch.randint(-4, 5, (b, M, K), generator=g).float()
    B = torch.randint(-4, 5, (b, N, K), generator=g).float()
    D = torch.randint(-8, 9, (b, M, N), generator=g).float()
    ref = (A @ B.transpose(-1, -2)) * 0.5 + D
    out = ops.fp8_gemm_v2(A.to(E4).to(dev), False, B.to(E4).to(dev), True, D.bfloat16().to(dev), torch.bfloat16,
                          torch.tensor([0.5], device=dev), None, None, True)
    assert torch.equal(out.cpu().float(), ref.bfloat16().float())
    # a 16-byte misaligned view of an aligned shape
    K2 = 768
    flat = torch.randint(-4, 5, (M * K2 + 3,), generator=g).float()
    A2 = flat[3:].reshape(M, K2)
    B2 = torch.randint(-4, 5, (K2, 512), generator=g).float()
    out = ops.fp8_gemm_v2(flat.to(E4).to(dev)[3:].reshape(M, K2), False, B2.to(E4).to(dev), False, None, torch.float32)
    assert torch.equal(out.cpu(), A2 @ B2)

