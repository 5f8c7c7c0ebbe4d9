"""GPU parity of mi355q::w4a16_gemm (bf16 activations times packed 4-bit weights, the weights expanded inside the
GEMM) against the oracle: the split of the activations into two fp8 planes bit for bit; the product bit-exact where
the arithmetic is exact (integer activations, power-of-two scales) and within max|out - ref| / max|ref| <= 1e-2 of the
float64-accumulated reference otherwise (measured: 5e-5), and against the unfused route the reference takes,
convert_from_[u]int4 followed by a matmul."""
import ctypes

import pytest
import torch

from helpers import gemm_errors
from test_gpu_w4a8_gemm import weights

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("rows,cols,ld", [
    (37, 1000, 1008),      # one vector per thread, eight columns of padding
    (9, 1003, 1008),       # cols not a multiple of 8: the element-wise kernel
    (5, 8192, 8192),       # the benchmark's K: four vectors per thread
    (3, 16384, 16384),     # eight vectors per thread
    (2, 20000, 20000),     # longer than a workgroup's registers hold: the element-wise kernel
    (4, 2056, 2064),       # two vectors per thread
])
def test_split_rows_bit_exact(oracle, pkg, dev, rows, cols, ld):
    gen = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=gen) * torch.logspace(-6, 4, rows).reshape(-1, 1)).bfloat16()
    if rows > 5:
        x[3] = 0
        x[5, ::7] *= 1e-5
    x[0, ::5] *= 1e-4
    lib = pkg.capi()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    xd = x.to(dev)
    hi = torch.full((rows, ld), 0x7f, dtype=torch.uint8, device=dev)
    lo = torch.full((rows, ld), 0x7f, dtype=torch.uint8, device=dev)
    sinv = torch.empty(rows, device=dev)
    assert lib.mi355q_split_rows_fp8x2(xd.data_ptr(), pkg.BF16, cols, rows, cols, hi.data_ptr(), lo.data_ptr(), ld, sinv.data_ptr(), st) == 0
    rh, rl, rs = oracle.split_rows_fp8x2(x)
    assert torch.equal(hi.cpu()[:, :cols], rh.view(torch.uint8)) and torch.equal(lo.cpu()[:, :cols], rl.view(torch.uint8))
    assert torch.equal(sinv.cpu(), rs)
    assert torch.count_nonzero(hi.cpu()[:, cols:]) == 0 and torch.count_nonzero(lo.cpu()[:, cols:]) == 0


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("M,K,N", [
    (16, 512, 256),       # 16-row form
    (5, 1024, 160),       # ragged M, a last strip of 32 columns... (160 = 5 x 32)
    (32, 2048, 512),      # 32-row form, K in parts
    (48, 640, 4096),      # 64-row tile
    (300, 256, 288),      # five row blocks
    (64, 4096, 1056),     # K in four parts
    (7, 4224, 1056),      # uneven parts
    (3, 256, 32800),      # 129 strips
    (130, 1024, 8992),    # three row blocks, 36 strips
])
def test_exact(oracle, dev, M, K, N, signed, zp):
    """Integer activations up to 2^11 in magnitude with a spread of magnitudes inside a row (so that both planes carry
    bits), power-of-two scales: every partial sum is an integer times a power of two below 2^24."""
    gen = torch.Generator().manual_seed(M + K + N + signed * 7 + zp)
    q, z, s, pk, pz = weights(oracle, gen, K, N, 128, signed, zp, pow2=True)
    a = torch.randint(-255, 256, (M, K), generator=gen).float()
    a[:, ::3] = torch.randint(-7, 8, (M, (K + 2) // 3), generator=gen).float()
    a = a * torch.exp2(torch.randint(-2, 3, (M, 1), generator=gen).float())
    bias = torch.randint(-8, 9, (N,), generator=gen).float()
    w = (q - (z.repeat_interleave(128, 0) if zp else 0)).double() * s.double().repeat_interleave(128, 0)
    expect = a.double() @ w + bias.double()
    assert expect.abs().max() < 2 ** 24 and torch.equal(a.bfloat16().float(), a)
    out = torch.ops.mi355q.w4a16_gemm(a.bfloat16().to(dev), pk.to(dev), s.to(dev), pz.to(dev) if zp else None, signed,
                                      torch.float32, bias.to(dev))
    assert out.shape == (M, N) and torch.equal(out.cpu().double(), expect)
    out16 = torch.ops.mi355q.w4a16_gemm(a.bfloat16().to(dev), pk.to(dev), s.to(dev), pz.to(dev) if zp else None, signed,
                                        torch.bfloat16, bias.bfloat16().to(dev))
    assert torch.equal(out16.cpu(), expect.float().bfloat16())


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("M", [16, 64, 256])
def test_against_oracle_config2_weights(oracle, dev, M, signed):
    """Benchmark configuration 2's weights (K = N = 4096, group 128, scales U(0.001, 0.02), zero-points for uint4) with
    configuration 4's activations (N(0, 1) with heavy-tail channels), in bf16."""
    gen = torch.Generator().manual_seed(0xC001A1 + M)
    K = N = 4096
    q, z, s, pk, pz = weights(oracle, gen, K, N, 128, signed, not signed)
    x = torch.randn(M, K, generator=gen)
    x[:, torch.randperm(K, generator=gen)[:41]] *= 20
    x = x.bfloat16()
    bias = (torch.randn(N, generator=gen) * 0.01).bfloat16()
    out = torch.ops.mi355q.w4a16_gemm(x.to(dev), pk.to(dev), s.to(dev), pz.to(dev) if pz is not None else None, signed,
                                      torch.float32, bias.float().to(dev))
    ref = oracle.torch_w4a16_gemm(x, pk, s, pz, signed, torch.float32, bias)
    rel, ok = gemm_errors(out, ref)
    assert rel <= 2e-4 and ok, rel            # far inside the 1e-2 bar: fp32 sums of q a and z a, whose difference is the result
    out16 = torch.ops.mi355q.w4a16_gemm(x.to(dev), pk.to(dev), s.to(dev), pz.to(dev) if pz is not None else None, signed,
                                        torch.bfloat16, bias.to(dev))
    rel, ok = gemm_errors(out16, ref)
    assert rel <= TOL and ok, rel
    # the route the reference takes: convert_from_[u]int4 to bf16 on the GPU (bit-exact op), then a bf16 matmul
    conv = torch.ops.hpu.convert_from_int4 if signed else torch.ops.hpu.convert_from_uint4
    w16 = conv(pk.to(dev), s.to(dev), pz.to(dev) if pz is not None else None, torch.bfloat16).cpu()
    ref2 = x.float() @ w16.float() + bias.float()      # its weights are rounded to bf16: the 1e-2 bar on max |ref| only
    rel, _ = gemm_errors(out16, ref2)
    assert rel <= TOL, rel


@pytest.mark.parametrize("M", [16, 256])
def test_exact_at_the_benchmark_shape(oracle, dev, M):
    K, N, group = 8192, 28672, 128
    gen = torch.Generator().manual_seed(8192 + M)
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, False, True, pow2=True)
    a = torch.randint(-40, 41, (M, K), generator=gen).float()
    qd, zd, sd = q.to(dev).double(), z.to(dev).double(), s.to(dev).double()
    w = (qd - zd.repeat_interleave(group, 0)) * sd.repeat_interleave(group, 0)
    expect = (a.to(dev).double() @ w).cpu()
    assert expect.abs().max() < 2 ** 24
    del w, qd, zd, sd
    out = torch.ops.mi355q.w4a16_gemm(a.bfloat16().to(dev), pk.to(dev), s.to(dev), pz.to(dev), False, torch.float32, None)
    assert torch.equal(out.cpu().double(), expect)


def test_batched_activations_c_abi_and_errors(oracle, pkg, dev):
    gen = torch.Generator().manual_seed(3)
    K, N = 256, 320
    q, z, s, pk, pz = weights(oracle, gen, K, N, 128, False, True)
    a = (torch.randn(2, 3, 7, K, generator=gen) * 2).bfloat16()
    out = torch.ops.mi355q.w4a16_gemm(a.to(dev), pk.to(dev), s.to(dev), pz.to(dev), False, torch.float32, None)
    assert out.shape == (2, 3, 7, N)
    ref = oracle.torch_w4a16_gemm(a.reshape(-1, K), pk, s, pz, False, torch.float32).reshape(2, 3, 7, N)
    rel, ok = gemm_errors(out, ref)
    assert rel < 2e-4 and ok, rel
    # the C entry point: wider pitches of A and C, K in one piece and split, the counters left zero
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    M, K2, N2 = 20, 4096, 1024
    q, z, s, pk, pz = weights(oracle, gen, K2, N2, 128, True, False)
    A = torch.zeros(M, K2 + 64, dtype=torch.bfloat16)
    A[:, :K2] = torch.randn(M, K2, generator=gen).bfloat16()
    Ad, pkd, sd = A.to(dev), pk.to(dev), s.to(dev)
    nbytes = lib.mi355q_w4a16_gemm_workspace_bytes(M, N2, K2, 128, pkg.BF16)
    assert nbytes > 0
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    ref = oracle.torch_w4a16_gemm(A[:, :K2].contiguous(), pk, s, None, True, torch.float32)
    for split in (1, 0, 1):
        C = torch.full((M, N2 + 32), -5.0, device=dev)
        assert lib.mi355q_w4a16_gemm(Ad.data_ptr(), pkg.BF16, K2 + 64, pkd.data_ptr(), N2 // 8, sd.data_ptr(), pkg.BF16, None, 1, 128,
                                     C.data_ptr(), pkg.F32, N2 + 32, M, N2, K2, None, ws.data_ptr(), nbytes, split, stream) == 0
        torch.cuda.synchronize()
        rel, ok = gemm_errors(C[:, :N2], ref)
        assert rel < 2e-4 and ok, rel
        assert (C[:, N2:] == -5.0).all() and torch.count_nonzero(ws[:1024]) == 0
    assert lib.mi355q_w4a16_gemm(Ad.data_ptr(), pkg.BF16, K2 + 64, pkd.data_ptr(), N2 // 8, sd.data_ptr(), pkg.BF16, None, 1, 128,
                                 C.data_ptr(), pkg.F32, N2 + 32, M, N2, K2, None, ws.data_ptr(), nbytes - 1, 1, stream) == 4      # workspace too small
    assert lib.mi355q_w4a16_gemm(Ad.data_ptr(), pkg.BF16, K2 + 64, pkd.data_ptr(), N2 // 8, sd.data_ptr(), pkg.BF16, None, 1, 256,
                                 C.data_ptr(), pkg.F32, N2 + 32, M, N2, K2, None, ws.data_ptr(), nbytes, 1, stream) == 2          # group 256: unsupported
    with pytest.raises(RuntimeError, match="groups of 128"):
        torch.ops.mi355q.w4a16_gemm(Ad[:, :K2], pkd, s.float().to(dev), None, True, torch.float32, None)
    with pytest.raises(RuntimeError, match="must be bfloat16"):
        torch.ops.mi355q.w4a16_gemm(Ad[:, :K2].float(), pkd, sd, None, True, torch.float32, None)


def test_one_workspace_serves_shapes_with_and_without_a_split(oracle, pkg, dev):
    """A buffer that is passed to calls of several shapes (the torch layer keeps one per stream): a shape that walks K
    in one part leaves the first KiB alone, where a later shape that splits K keeps its arrival counters."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(21)
    shapes = [(16, 512, 256), (32, 2048, 512), (16, 512, 256), (8, 4096, 512)]     # K in one part, in two, in one, in four
    nbytes = max(lib.mi355q_w4a16_gemm_workspace_bytes(M, N, K, 128, pkg.BF16) for M, K, N in shapes)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    for M, K, N in shapes:
        q, z, s, pk, pz = weights(oracle, gen, K, N, 128, False, True, pow2=True)
        a = torch.randint(-255, 256, (M, K), generator=gen).float()
        expect = a.double() @ ((q - z.repeat_interleave(128, 0)).double() * s.double().repeat_interleave(128, 0))
        Ad, pkd, sd, pzd = a.bfloat16().to(dev), pk.to(dev), s.to(dev), pz.to(dev)
        C = torch.full((M, N), -5.0, device=dev)
        assert lib.mi355q_w4a16_gemm(Ad.data_ptr(), pkg.BF16, K, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, pzd.data_ptr(), 0, 128,
                                     C.data_ptr(), pkg.F32, N, M, N, K, None, ws.data_ptr(), nbytes, 1, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().double(), expect), (M, K, N)
        assert torch.count_nonzero(ws[:1024]) == 0
