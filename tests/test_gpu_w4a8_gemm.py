"""GPU parity of mi355q::w4a8_gemm (fp8 activations times packed 4-bit weights, dequantisation fused into
the GEMM) against the oracle: bit-exact where the arithmetic is exact (small-integer activations,
power-of-two scales), max|out - ref| / max|ref| <= 1e-2 against the float64-accumulated reference otherwise,
and against the unfused route convert_from_[u]int4 -> fp32 weights on the CPU."""
import ctypes

import pytest
import torch

from helpers import E4, E5, gemm_errors

pytestmark = pytest.mark.gpu
TOL = 1e-2


def weights(oracle, gen, K, N, group, signed, zp, scale_dtype=torch.bfloat16, pow2=False):
    lo, hi = (-8, 8) if signed else (0, 16)
    q = torch.randint(lo, hi, (K, N), generator=gen)
    z = torch.randint(lo, hi, (K // group, N), generator=gen) if zp else None
    if pow2:
        s = torch.exp2(torch.randint(-3, 3, (K // group, N), generator=gen).float()).to(scale_dtype)
    else:
        s = (torch.rand(K // group, N, generator=gen) * 0.019 + 0.001).to(scale_dtype)
    return q, z, s, oracle.pack_nibbles(q), (oracle.pack_nibbles(z) if zp else None)


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("M,K,N,group", [
    (16, 512, 256, 128),      # 32-row strip
    (5, 1024, 160, 256),      # ragged M, a strip with 32 columns, groups of two stages
    (48, 640, 4096, 128),     # 64-row strip, K not a multiple of the ring
    (100, 384, 1056, 384),    # 128-row strip, one group
    (300, 256, 288, 128),     # three row blocks
    (64, 4096, 128, 4096),    # per-channel scales, a ring walked several times
    (16, 2048, 512, 128),     # 256-column strips, K in two parts
    (7, 4224, 1056, 128),     # ... in four uneven parts (33 stages), the last strip 32 columns wide
    (32, 8192, 256, 128),     # ... one strip, K in eight parts
    (3, 256, 32800, 128),     # ... 129 strips, K in one part
    (64, 4096, 1056, 128),    # ... 64-row tiles, K in four parts
    (100, 2048, 512, 128),    # ... two row blocks (the second ragged), K in two parts
    (130, 256, 8992, 128),    # ... three row blocks, 36 strips, K in one part
])
def test_exact(oracle, dev, M, K, N, group, signed, zp):
    gen = torch.Generator().manual_seed(M * 3 + K + N + signed * 7 + zp)
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, signed, zp, pow2=True)
    a = torch.randint(-4, 5, (M, K), generator=gen).float()
    sa = torch.exp2(torch.randint(-2, 3, (M, 1), generator=gen).float())
    bias = torch.randint(-8, 9, (N,), generator=gen).float()
    w = (q - (z.repeat_interleave(group, 0) if zp else 0)).double() * s.double().repeat_interleave(group, 0)
    expect = ((a.double() @ w) * sa.double() + bias.double())                    # integers times powers of two: exact
    assert expect.abs().max() < 2 ** 24
    for fmt in (E4, E5):
        out = torch.ops.mi355q.w4a8_gemm(a.to(fmt).to(dev), pk.to(dev), s.to(dev), pz.to(dev) if zp else None, signed,
                                         torch.float32, sa.to(dev), bias.to(dev))
        assert out.shape == (M, N) and torch.equal(out.cpu().double(), expect), fmt
    out16 = torch.ops.mi355q.w4a8_gemm(a.to(E4).to(dev), pk.to(dev), s.to(dev), pz.to(dev) if zp else None, signed,
                                       torch.bfloat16, sa.to(dev), bias.bfloat16().to(dev))
    assert torch.equal(out16.cpu(), expect.float().bfloat16())


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("scale_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [16, 64, 256])
def test_against_oracle_config2_weights(oracle, dev, M, signed, scale_dtype):
    """Benchmark configuration 2's weights (K = N = 4096, group 128, scales U(0.001, 0.02), zero-points for
    uint4) with configuration 4's activations (per-token e4m3fn of N(0, 1) with heavy-tail channels)."""
    gen = torch.Generator().manual_seed(0xC001A1 + M)
    K = N = 4096
    q, z, s, pk, pz = weights(oracle, gen, K, N, 128, signed, not signed, scale_dtype)
    x = torch.randn(M, K, generator=gen)
    x[:, torch.randperm(K, generator=gen)[:41]] *= 20
    x8, sx = oracle.quantize_rows(x.bfloat16(), E4)
    bias = (torch.randn(N, generator=gen) * 0.01).bfloat16()
    out = torch.ops.mi355q.w4a8_gemm(x8.to(dev), pk.to(dev), s.to(dev), pz.to(dev) if pz is not None else None, signed,
                                     torch.bfloat16, sx.to(dev), bias.to(dev))
    ref = oracle.torch_w4a8_gemm(x8, pk, s, pz, signed, torch.float32, sx, bias)
    rel, ok = gemm_errors(out, ref)
    assert rel <= TOL and ok, rel
    # the unfused route: convert_from_[u]int4 to fp32 on the GPU (bit-exact op), product on the CPU
    conv = torch.ops.hpu.convert_from_int4 if signed else torch.ops.hpu.convert_from_uint4
    w32 = conv(pk.to(dev), s.float().to(dev), pz.to(dev) if pz is not None else None, torch.float32).cpu()
    ref2 = (x8.float() @ w32) * sx + bias.float()
    rel, ok = gemm_errors(out, ref2)
    assert rel <= TOL and ok, rel


def test_batched_activations_scalar_scale_and_c_abi(oracle, pkg, dev):
    gen = torch.Generator().manual_seed(3)
    K, N, group = 256, 320, 128
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, False, True)
    a8 = (torch.randn(2, 3, 7, K, generator=gen) * 2).to(E4)
    sa = torch.tensor(0.37)
    out = torch.ops.mi355q.w4a8_gemm(a8.to(dev), pk.to(dev), s.to(dev), pz.to(dev), False, torch.float32, sa.to(dev), None)
    assert out.shape == (2, 3, 7, N)
    ref = oracle.torch_w4a8_gemm(a8.reshape(-1, K), pk, s, pz, False, torch.float32, sa).reshape(2, 3, 7, N)
    rel, ok = gemm_errors(out, ref)
    assert rel < 1e-5 and ok, rel
    # the C entry point with a host scalar, wider row pitches of A and C
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    M = 40
    A = torch.zeros(M, K + 64, dtype=torch.uint8)
    A[:, :K] = (torch.randn(M, K, generator=gen)).to(E4).view(torch.uint8)
    Ad, pkd, sd, pzd = A.to(dev), pk.to(dev), s.to(dev), pz.to(dev)
    C = torch.full((M, N + 32), -5.0, device=dev)
    st = lib.mi355q_w4a8_gemm(Ad.data_ptr(), pkg.E4M3FN, K + 64, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, pzd.data_ptr(), 0,
                              group, C.data_ptr(), pkg.F32, N + 32, M, N, K, None, 0.5, pkg.GS_HOST, None, None, 0, stream)
    assert st == 0
    torch.cuda.synchronize()
    ref = oracle.torch_w4a8_gemm(A[:, :K].view(E4), pk, s, pz, False, torch.float32, 0.5)
    rel, ok = gemm_errors(C[:, :N], ref)
    assert rel < 1e-5 and ok, rel
    assert (C[:, N:] == -5.0).all()
    # refused shapes launch nothing: a group of 64, N not a multiple of 32
    assert lib.mi355q_w4a8_gemm(Ad.data_ptr(), pkg.E4M3FN, K + 64, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, None, 0,
                                64, C.data_ptr(), pkg.F32, N + 32, M, N, K, None, 1.0, pkg.GS_NONE, None, None, 0, stream) == 2
    assert lib.mi355q_w4a8_gemm(Ad.data_ptr(), pkg.E4M3FN, K + 64, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, None, 0,
                                128, C.data_ptr(), pkg.F32, N + 32, M, N - 8, K, None, 1.0, pkg.GS_NONE, None, None, 0, stream) == 2
    with pytest.raises(RuntimeError, match="multiples of 128"):
        torch.ops.mi355q.w4a8_gemm(a8.to(dev), pk.to(dev), s.repeat(2, 1).to(dev), None, False, torch.float32, None, None)


@pytest.mark.parametrize("seed", range(32))
def test_random_shapes_exact(oracle, dev, seed):
    """Shapes drawn at random across the kernels' regimes (rows up to 300, K up to 64 stages, strips of every width,
    groups of one or more stages, both scale types), small-integer values: every output exact."""
    gen = torch.Generator().manual_seed(1000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    M = [r(1, 16), r(17, 32), r(33, 64), r(65, 300)][seed % 4]
    stages = r(1, 64)
    per_group = [1, 1, 1, 2, stages][r(0, 4)]
    stages -= stages % per_group
    stages = max(stages, per_group)
    K, group = 128 * stages, 128 * per_group
    N = 32 * r(1, 80)
    signed, zp = bool(r(0, 1)), bool(r(0, 1))
    scale_dtype = torch.float32 if r(0, 5) == 0 else torch.bfloat16
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, signed, zp, scale_dtype, pow2=True)
    a = torch.randint(-3, 4, (M, K), generator=gen).float()
    sa = torch.exp2(torch.randint(-2, 3, (M, 1), generator=gen).float())
    bias = torch.randint(-8, 9, (N,), generator=gen).float()
    w = (q - (z.repeat_interleave(group, 0) if zp else 0)).double() * s.double().repeat_interleave(group, 0)
    expect = (a.double() @ w) * sa.double() + bias.double()
    assert expect.abs().max() < 2 ** 24
    fmt = E5 if r(0, 3) == 0 else E4
    out = torch.ops.mi355q.w4a8_gemm(a.to(fmt).to(dev), pk.to(dev), s.to(dev), pz.to(dev) if zp else None, signed,
                                     torch.float32, sa.to(dev), bias.to(dev))
    assert torch.equal(out.cpu().double(), expect), (M, K, N, group, signed, zp, scale_dtype, fmt)


def test_split_k_workspace_c_abi(oracle, pkg, dev):
    """The C entry point with and without the workspace of the split over K: the same exact result, arrival
    counters back at zero after every call, repeated calls bit-identical, sizes checked."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(11)
    M, K, N, group = 24, 4096, 1312, 128
    need = lib.mi355q_w4a8_gemm_workspace_bytes(M, N, K, group, pkg.BF16)
    strips = (N + 255) // 256
    assert need == 1024 + 4 * strips * 32 * 256 * 4                       # 1 KiB of counters; K / 128 / 8 = 4 parts
    assert lib.mi355q_w4a8_gemm_workspace_bytes(33, N, K, group, pkg.BF16) == 1024 + 4 * strips * 64 * 256 * 4   # 64-row tiles
    assert lib.mi355q_w4a8_gemm_workspace_bytes(130, N, K, group, pkg.BF16) == 1024 + 4 * strips * 2 * 128 * 256 * 4  # two row blocks of 128
    assert lib.mi355q_w4a8_gemm_workspace_bytes(M, N, K, 256, pkg.BF16) == 0       # groups of two stages
    assert lib.mi355q_w4a8_gemm_workspace_bytes(M, N, K, group, pkg.F32) == 0      # fp32 scales
    assert lib.mi355q_w4a8_gemm_workspace_bytes(M, N, 1024, group, pkg.BF16) == 0  # too few stages to split
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, False, True, pow2=True)
    a = torch.randint(-4, 5, (M, K), generator=gen).float()
    w = (q - z.repeat_interleave(group, 0)).double() * s.double().repeat_interleave(group, 0)
    expect = a.double() @ w
    Ad, pkd, sd, pzd = a.to(E4).to(dev), pk.to(dev), s.to(dev), pz.to(dev)
    ws = torch.zeros(need + 64, dtype=torch.uint8, device=dev)

    def call(C, Adev, workspace, nbytes):
        return lib.mi355q_w4a8_gemm(Adev.data_ptr(), pkg.E4M3FN, K, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, pzd.data_ptr(), 0,
                                    group, C.data_ptr(), pkg.F32, N, M, N, K, None, 1.0, pkg.GS_NONE, None,
                                    workspace.data_ptr() if workspace is not None else None, nbytes, stream)
    for workspace, nbytes in ((ws, need), (None, 0), (ws, need + 64)):
        C = torch.full((M, N), -5.0, device=dev)
        assert call(C, Ad, workspace, nbytes) == 0
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().double(), expect)
        assert int(ws[:1024].view(torch.int32).abs().sum()) == 0
    C = torch.full((M, N), -5.0, device=dev)
    assert call(C, Ad, ws, need - 1) == 4 and call(C, Ad, ws[1:], need) == 4      # too small, misaligned
    torch.cuda.synchronize()
    assert (C == -5.0).all()
    # values whose fp32 sums depend on the order: the parts are added in a fixed order
    x8 = torch.randn(M, K, generator=gen).to(E4).to(dev)
    outs = []
    for _ in range(4):
        C = torch.empty(M, N, device=dev)
        assert call(C, x8, ws, need) == 0
        outs.append(C)
    torch.cuda.synchronize()
    assert all(torch.equal(outs[0], o) for o in outs[1:])
    ref = oracle.torch_w4a8_gemm(x8.cpu(), pk, s, pz, False, torch.float32, None)
    rel, ok = gemm_errors(outs[0], ref)
    assert rel < 1e-5 and ok, rel
    # at most 16 rows (the 16x16x128 form): bf16 output whose rows start at odd element offsets, per-row scales, bias
    M2 = 10
    sa = torch.exp2(torch.randint(-2, 3, (M2,), generator=gen).float())
    bias = torch.randint(-8, 9, (N,), generator=gen).float()
    C = torch.full((M2, N + 2), -5.0, dtype=torch.bfloat16, device=dev)
    sad, biasd = sa.to(dev), bias.bfloat16().to(dev)
    assert lib.mi355q_w4a8_gemm(Ad.data_ptr(), pkg.E4M3FN, K, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, pzd.data_ptr(), 0,
                                group, C.data_ptr(), pkg.BF16, N + 2, M2, N, K, sad.data_ptr(), 1.0, pkg.GS_PER_ROW, biasd.data_ptr(),
                                ws.data_ptr(), need, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(C[:, :N].cpu(), (expect[:M2] * sa.double()[:, None] + bias.double()).float().bfloat16())
    assert (C[:, N:] == -5.0).all()


def test_one_workspace_for_problems_of_different_shapes(oracle, pkg, dev):
    """A workspace sized for the largest problem serves a narrow one (one strip) and then a wide one (many strips),
    and the narrow one again: the counters have a place of their own in front, which no shape's partial sums reach."""
    lib = pkg.capi()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(12)
    K, group = 4096, 128
    shapes = [(24, 256), (40, 2304), (24, 256), (16, 6400)]
    need = max(lib.mi355q_w4a8_gemm_workspace_bytes(M, N, K, group, pkg.BF16) for M, N in shapes)
    assert need > 0
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    for M, N in shapes:
        assert lib.mi355q_w4a8_gemm_workspace_bytes(M, N, K, group, pkg.BF16) > 0
        q, z, s, pk, pz = weights(oracle, gen, K, N, group, False, True, pow2=True)
        a = torch.randint(-4, 5, (M, K), generator=gen).float()
        expect = a.double() @ ((q - z.repeat_interleave(group, 0)).double() * s.double().repeat_interleave(group, 0))
        Ad, pkd, sd, pzd = a.to(E4).to(dev), pk.to(dev), s.to(dev), pz.to(dev)
        C = torch.full((M, N), -5.0, device=dev)
        assert lib.mi355q_w4a8_gemm(Ad.data_ptr(), pkg.E4M3FN, K, pkd.data_ptr(), N // 8, sd.data_ptr(), pkg.BF16, pzd.data_ptr(), 0,
                                    group, C.data_ptr(), pkg.F32, N, M, N, K, None, 1.0, pkg.GS_NONE, None, ws.data_ptr(), need,
                                    stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().double(), expect), (M, N)
        assert not ws[:1024].any()


def test_meta_and_checks(dev):
    a = torch.empty(4, 256, device="meta", dtype=E4)
    pk = torch.empty(256, 16, device="meta", dtype=torch.int32)
    s = torch.empty(2, 128, device="meta", dtype=torch.bfloat16)
    out = torch.ops.mi355q.w4a8_gemm(a, pk, s, None, True, torch.bfloat16, None, None)
    assert out.shape == (4, 128) and out.dtype == torch.bfloat16
    with pytest.raises(RuntimeError, match="Common dimension"):
        torch.ops.mi355q.w4a8_gemm(torch.empty(4, 128, device="meta", dtype=E4), pk, s, None, True, torch.bfloat16, None, None)
    with pytest.raises(RuntimeError, match="scale must be"):
        torch.ops.mi355q.w4a8_gemm(a, pk, torch.empty(3, 128, device="meta"), None, True, torch.bfloat16, None, None)


@pytest.mark.parametrize("M", [16, 64, 256])
def test_exact_at_the_benchmark_shape(oracle, dev, M):
    """K = 8192, N = 28672 (the shape bench.py times: 112 strips of 256 columns, K in two parts, one to four row
    blocks): small-integer activations, power-of-two group scales and zero-points make every partial sum exact, so
    the whole [M, N] output is compared bit for bit with an integer matmul."""
    K, N, group = 8192, 28672, 128
    gen = torch.Generator().manual_seed(8192 + M)
    q, z, s, pk, pz = weights(oracle, gen, K, N, group, False, True, pow2=True)
    a = torch.randint(-2, 3, (M, K), generator=gen).float()
    sa = torch.exp2(torch.randint(-2, 3, (M, 1), generator=gen).float())
    # (q - z) s group by group on the GPU in float64 (exact: integers below 2^5 times powers of two)
    qd, zd, sd = q.to(dev).double(), z.to(dev).double(), s.to(dev).double()
    w = (qd - zd.repeat_interleave(group, 0)) * sd.repeat_interleave(group, 0)
    expect = ((a.to(dev).double() @ w) * sa.to(dev).double()).cpu()
    assert expect.abs().max() < 2 ** 24
    del w, qd, zd, sd
    out = torch.ops.mi355q.w4a8_gemm(a.to(E4).to(dev), pk.to(dev), s.to(dev), pz.to(dev), False, torch.float32, sa.to(dev), None)
    assert torch.equal(out.cpu().double(), expect)
    out2 = torch.ops.mi355q.w4a8_gemm(a.to(E4).to(dev), pk.to(dev), s.to(dev), pz.to(dev), False, torch.float32, sa.to(dev), None)
    assert torch.equal(out2, out)
