"""GPU parity: fp8_gemm_v2 against the CPU oracle.

Two bars: bit-exact where the mathematics makes the answer unique (small-integer
operands keep every fp32 partial sum exact, whatever the accumulation order),
and max|out - ref| / max|ref| <= 1e-2 (plus the reference's allclose(atol=1e-3,
rtol=1e-2), atol scaled to the output magnitude) against the fp32-accumulated
CPU reference elsewhere.
"""
import ctypes

import pytest
import torch

from helpers import E4, E5, FP8_DTYPES, gemm_errors

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu
TOL = 1e-2


def small_int_fp8(shape, dtype, gen, lo=-4, hi=5):
    return torch.randint(lo, hi, shape, generator=gen).float().to(dtype)


def check(out, ref, what=""):
    rel, ok = gemm_errors(out, ref)
    assert rel <= TOL and ok, f"{what}: rel {rel}"


@pytest.mark.parametrize("fa", FP8_DTYPES)
@pytest.mark.parametrize("fb", FP8_DTYPES)
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 512, 1024), (272, 144, 384), (48, 80, 1024), (300, 260, 144)])
def test_exact_small_integers_tiled(dev, fa, fb, ta, tb, M, N, K):
    """Exercises every layout x format combination of the MFMA kernel, full and
    ragged tiles, the K tail (K % 128 != 0) and both tile sizes; exact."""
    if (ta and M % 16) or (not tb and N % 16):
        pytest.skip("contiguous dimension not a multiple of 16: covered by the simple-kernel tests")
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    A = small_int_fp8((K, M) if ta else (M, K), fa, g)
    B = small_int_fp8((N, K) if tb else (K, N), fb, g)
    a = A.float().t() if ta else A.float()
    b = B.float().t() if tb else B.float()
    expect = a @ b  # exact in fp32: |sum| <= 16 K
    out = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.float32)
    assert torch.equal(out.cpu(), expect)
    out16 = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.bfloat16)
    assert torch.equal(out16.cpu(), expect.bfloat16())


# One shape per kernel the dispatcher can pick (256 CUs): 256 x 256 tiles need at least 256 of them
# (a last pass that fills at most a quarter of the CUs is split off as columns of 256 x 128 tiles:
# 272 and 528 tiles do that, 464 do not);
# below that the eight-wave kernel runs with 256 x 128 tiles while those fill more than half the CUs
# (more, or fewer, tiles than CUs), else with 128 x 128 tiles, two workgroups per CU; the strip kernel
# has three row-tile heights, and 128 x 128 tiles also serve N <= 128 < M (fewer, or more, tiles than
# the 512 workgroup slots).  Edges are ragged in M, N and K.
KERNEL_SHAPES = {
    "tile256_one_pass_and_tail_columns": (4000, 4112, 208),
    "tile256_two_passes_and_tail_columns": (4000, 8208, 208),
    "tile256_two_passes_no_split": (4000, 7184, 144),
    "tile256_ten_k_stages": (4000, 4112, 1168),
    "tile256_whole_stage_pairs_and_tail_columns": (4000, 4112, 512),   # K % 256 == 0: the kernel without per-lane K tests
    "tile256_whole_stage_pairs_two_passes": (4000, 8208, 256),
    "tile256x128_more_tiles_than_cus": (1008, 12304, 208),
    "tile256x128_fewer_tiles_than_cus": (272, 10256, 272),
    "tile128_underfilled": (272, 4112, 400),
    "strip_32_rows": (16, 1040, 400),
    "strip_64_rows": (48, 1040, 400),
    "strip_128_rows": (112, 1040, 400),
    "tile128": (400, 112, 272),
    "tile128_more_tiles_than_slots": (66576, 112, 144),
}


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("kernel", sorted(KERNEL_SHAPES))
def test_every_kernel_path(oracle, dev, kernel, ta, tb):
    """Exact small-integer products through each kernel (fp32 output: general epilogue), then the
    same operands with per-row x per-column scales, a bias vector and bf16 output (fast epilogue)
    against the fp32-accumulated CPU reference, with and without an accumulate input."""
    M, N, K = KERNEL_SHAPES[kernel]
    g = torch.Generator().manual_seed(M + N + K)
    A = small_int_fp8((K, M) if ta else (M, K), E4, g)
    B = small_int_fp8((N, K) if tb else (K, N), E5, g)
    a = A.float().t() if ta else A.float()
    b = B.float().t() if tb else B.float()
    expect = a @ b
    out = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.float32)
    assert torch.equal(out.cpu(), expect)
    sa = torch.rand(M, 1, generator=g) + 0.5
    sb = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g).bfloat16()
    out16 = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.bfloat16, sa.to(dev), sb.to(dev), bias.to(dev), False, [1, N])
    ref = oracle.torch_fp8_gemm(A, ta, B, tb, torch.float32, sa, sb.reshape(1, N), bias=bias)
    check(out16, ref, kernel)
    # scalar scales fold into one factor in the fast epilogue
    out_s = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.bfloat16, 0.5, 0.25, bias.to(dev), False)
    assert torch.equal(out_s.cpu(), (expect * 0.125 + bias.float()).bfloat16())
    # accumulate input in the fast epilogue: added after the bias, in fp32
    D = torch.randint(-64, 65, (M, N), generator=g).bfloat16()
    out_d = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, D.to(dev), torch.bfloat16, 0.5, 0.25, bias.to(dev), True)
    assert torch.equal(out_d.cpu(), (expect * 0.125 + bias.float() + D.float()).bfloat16())
    out_d = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, D.to(dev), torch.bfloat16, sa.to(dev), sb.to(dev), None, True, [1, N])
    check(out_d, oracle.torch_fp8_gemm(A, ta, B, tb, torch.float32, sa, sb.reshape(1, N), D=D), kernel + " accumulate")


@pytest.mark.parametrize("shape", [(24, 12, 36), (22, 10, 34), (26, 16, 38), (1, 7, 3), (17, 1, 5), (33, 65, 129)])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_exact_small_integers_odd_shapes(dev, shape, ta, tb):
    """Shapes that break the 16-byte rules (the reference's own test sizes, :476-501)."""
    K, M, N = shape
    g = torch.Generator().manual_seed(K * 100 + M * 10 + N)
    A = small_int_fp8((K, M) if ta else (M, K), E5, g)
    B = small_int_fp8((N, K) if tb else (K, N), E4, g)
    a = A.float().t() if ta else A.float()
    b = B.float().t() if tb else B.float()
    out = ops.fp8_gemm_v2(A.to(dev), ta, B.to(dev), tb, None, torch.float32)
    assert torch.equal(out.cpu(), a @ b)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("accumulate", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fp8_dtype", FP8_DTYPES)
@pytest.mark.parametrize("shapes", [((24, 12), (24, 36)), ((22, 10), (22, 34)), ((26, 16), (26, 38)), ((256, 160), (256, 320))])
def test_fp8_gemm_v2(oracle, dev, bias, accumulate, dtype, fp8_dtype, shapes):
    """test_hpu_fp8_ops_any_mode.py:361-501: cast -> gemm with trans_A, full [M,N] bias,
    accumulate into a 1000-filled D; the reference allows 15 % against the unquantised
    matmul, the oracle comparison here is the 1e-2 bar."""
    shapeA, shapeB = shapes
    A = torch.rand(shapeA).to(dtype) * 10 + 30.0
    B = torch.rand(shapeB).to(dtype) * 10 + 30.0
    fmax = 57344 * 0.9 if fp8_dtype == E5 else 240 * 0.9  # FP8_MAX of fp8_utils.py:53-55
    sA = (fmax / A.abs().max().float())
    sB = (fmax / B.abs().max().float())
    A8, _ = ops.cast_to_fp8_v2(A.to(dev), sA.to(dev), False, False, fp8_dtype)
    B8, _ = ops.cast_to_fp8_v2(B.to(dev), sB.to(dev), False, False, fp8_dtype)
    M, N = shapeA[1], shapeB[1]
    bias_t = (torch.rand(M, N).to(dtype) * 10 + 30.0) if bias else None
    D = torch.full((M, N), 1000.0, dtype=dtype)
    out = ops.fp8_gemm_v2(A8, True, B8, False, D.to(dev), dtype, sA.reciprocal().to(dev), sB.reciprocal().to(dev),
                          bias_t.to(dev) if bias else None, accumulate)
    ref = oracle.torch_fp8_gemm(A8.cpu(), True, B8.cpu(), False, torch.float32, sA.reciprocal(), sB.reciprocal(),
                                bias=bias_t, D=D if accumulate else None)
    check(out, ref)
    # the reference's own criterion against the unquantised product (:471-473)
    full = torch.matmul(A.float().t(), B.float())
    if bias:
        full = full + bias_t.float()
    if accumulate:
        full = full + D.float()
    pct = (((out.cpu().float() - full) / full) * 100).to(torch.int).abs().max().item()
    assert pct <= 15


@pytest.mark.parametrize("shapeA, shapeB", [((2, 1, 4, 2), (1, 3, 4, 8)), ((2, 1, 4, 2), (4, 8)), ((4, 2), (3, 4, 8)),
                                            ((2, 3, 64, 32), (2, 3, 64, 48)), ((3, 128, 32), (128, 256))])
def test_fp8_gemm_v2_batch_shapes(oracle, dev, shapeA, shapeB):
    """test :504-514: batch broadcasting, trans_A."""
    g = torch.Generator().manual_seed(21)
    A = small_int_fp8(shapeA, E5, g)
    B = small_int_fp8(shapeB, E5, g)
    out = ops.fp8_gemm_v2(A.to(dev), True, B.to(dev), False, None, torch.float32)
    expect = torch.matmul(A.float().transpose(-2, -1), B.float())
    assert out.shape == expect.shape and torch.equal(out.cpu(), expect)


SCALE_MODES = [("tensor", None), ("scalar", "scalar"), ("scalar", None), (None, "tensor"), (None, "scalar"),
               (None, "tensor_channel"), (None, "scalar_channel"), (None, None)]


@pytest.mark.parametrize("scaleA, scaleB", SCALE_MODES)
def test_fp8_gemm_v2_scales(oracle, dev, scaleA, scaleB):
    """test :517-531: every mix of tensor / float / list scales, batched, bf16, with bias."""
    shapeA, shapeB = (2, 1, 4, 2), (1, 3, 4, 8)
    A = (torch.rand(shapeA).bfloat16() * 10 + 30.0).to(E4)
    B = (torch.rand(shapeB).bfloat16() * 10 + 30.0).to(E4)
    N = shapeB[-1]
    va, vb = 0.37, 0.21

    def make(mode, v):
        if mode is None:
            return None, None
        if mode == "tensor":
            return torch.tensor(v).to(dev), torch.tensor(v)
        if mode == "scalar":
            return v, v
        vec = torch.full((N,), v) * (torch.arange(N) + 1)
        if mode == "tensor_channel":
            return vec.to(dev), vec
        return vec.tolist(), vec

    a_arg, a_ref = make(scaleA, va)
    b_arg, b_ref = make(scaleB, vb)
    if scaleB == "scalar_channel" and a_arg is None:
        a_arg, a_ref = [1.0], 1.0
    if isinstance(b_arg, float) and a_arg is None:
        a_arg, a_ref = 1.0, 1.0
    if isinstance(a_arg, float) and b_arg is None:
        b_arg, b_ref = 1.0, 1.0
    bias = (torch.rand(2, 3, 2, 8).bfloat16() * 10 + 30.0)
    out = ops.fp8_gemm_v2(A.to(dev), True, B.to(dev), False, None, torch.bfloat16, a_arg, b_arg, bias.to(dev), False)
    ref = oracle.torch_fp8_gemm(A, True, B, False, torch.float32, a_ref, b_ref, bias=bias)
    check(out, ref)


@pytest.mark.parametrize("shape_a, shape_b", [((10,), (10,)), ((2, 10), (10,)), ((10,), (10, 2)), ((4, 8, 16), (16,)),
                                              ((8,), (2, 4, 8, 16))])
@pytest.mark.parametrize("transpose_a", [True, False])
@pytest.mark.parametrize("transpose_b", [True, False])
def test_fp8_gemm_v2_1d(dev, shape_a, shape_b, transpose_a, transpose_b):
    """test :534-596: 1-D operands, operands handed over already transposed, bf16 scale tensors."""
    def gen(shape, transpose):
        t = (torch.rand(shape).bfloat16() * 10 + 30.0).to(E5)
        if transpose:
            if len(shape) == 1:
                pytest.skip("Configuration not supported")
            return t.to(torch.bfloat16), t.transpose(-2, -1).contiguous().to(dev)
        return t.to(torch.bfloat16), t.to(dev)

    A, A_dev = gen(shape_a, transpose_a)
    B, B_dev = gen(shape_b, transpose_b)
    sA = torch.tensor(3.14, dtype=torch.bfloat16)
    sB = torch.tensor(0.75, dtype=torch.bfloat16)
    ref = torch.matmul(A.float(), B.float()) * (sA.float() * sB.float())
    out = ops.fp8_gemm_v2(A_dev, transpose_a, B_dev, transpose_b, None, torch.bfloat16, sA.to(dev), sB.to(dev), None, False)
    assert out.shape == ref.shape
    check(out, ref)


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("dims", [(12, 24, 36), (160, 256, 272)])
def test_fp8_gemm_v2_scale_shape(dev, axis, dims):
    """test :599-657: list scales, B scale broadcast as [M,1] (axis 1) or [1,N] (axis 0)."""
    M, K, N = dims
    A = (torch.rand(M, K).bfloat16() * 10 + 30.0).to(E4)
    B = (torch.rand(K, N).bfloat16() * 10 + 30.0).to(E4)
    sa = (torch.rand(1) * 100).tolist()
    sbv = torch.rand(M if axis == 1 else N) * 100
    sb_t = sbv.unsqueeze(axis)
    out = ops.fp8_gemm_v2(A.to(dev), False, B.to(dev), False, None, torch.bfloat16, sa, sbv.tolist(), None, False,
                          list(sb_t.shape))
    ref = torch.matmul(A.float(), B.float()) * (torch.tensor(sa) * sb_t)
    check(out, ref)


@pytest.mark.parametrize("scaleA", [16, 14])
@pytest.mark.parametrize("scaleB", [0.00390625, 0.23])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fp8_gemm_v2_scalar_scales(dev, scaleA, scaleB, dtype):
    """test :660-704: power-of-two and odd scalar scales behave alike."""
    A = (torch.rand(12, 24).to(dtype) * 10 + 30.0).to(E4)
    B = (torch.rand(24, 36).to(dtype) * 10 + 30.0).to(E4)
    out = ops.fp8_gemm_v2(A.to(dev), False, B.to(dev), False, None, dtype, scaleA, scaleB, None, False)
    ref = torch.matmul(A.float(), B.float()) * (scaleA * scaleB)
    check(out, ref)


@pytest.mark.parametrize("scale_a", [1.0, 0.0625, 7.5])
@pytest.mark.parametrize("scale_b", [16.0, 1.0, 0.23])
@pytest.mark.parametrize("scale_out", [16.0, 0.0625, 7.5])
def test_gemm_then_cast_tensor_vs_scalar_scales(dev, scale_a, scale_b, scale_out):
    """test :706-792: the gemm -> cast chain gives the same bits with tensor and scalar scales."""
    a = (torch.rand(4, 8) * 5).to(E4).to(dev)
    b = (torch.rand(8, 12) * 5).to(E4).to(dev)

    def fn(sa, sb, so):
        return ops.cast_to_fp8_v2(ops.fp8_gemm_v2(a, False, b, False, None, torch.bfloat16, sa, sb, None, False),
                                  so, False, False, E4)[0]

    t = fn(torch.tensor(scale_a).to(dev), torch.tensor(scale_b).to(dev), torch.tensor(scale_out).to(dev))
    s = fn(scale_a, scale_b, scale_out)
    assert torch.equal(t.cpu().view(torch.uint8), s.cpu().view(torch.uint8))


def quantize_rows(oracle, x, dim):
    amax = x.abs().amax(dim=dim, keepdim=True).float().clamp_min(1e-12)
    s = 448.0 / amax
    x8, _ = oracle.torch_cast_to_fp8(x, s, E4)
    return x8, (1.0 / s)


@pytest.mark.parametrize("M", [16, 64, 256])
def test_config4_decode_shapes_reduced(oracle, dev, M):
    """benchmark configuration 4 semantics (per-token x per-channel scales, heavy-tail channels) at
    K = 1024, N = 1536 so that the CPU reference finishes in seconds."""
    g = torch.Generator().manual_seed(M)
    K, N = 1024, 1536
    x = torch.randn(M, K, generator=g)
    cols = torch.randperm(K, generator=g)[: K // 100 + 1]
    x[:, cols] *= 20
    x = x.bfloat16()
    w = (torch.randn(K, N, generator=g) * 0.02).bfloat16()
    x8, sx = quantize_rows(oracle, x, 1)          # [M,1]
    w8, sw = quantize_rows(oracle, w, 0)          # [1,N]
    out = ops.fp8_gemm_v2(x8.to(dev), False, w8.to(dev), False, None, torch.bfloat16, sx.to(dev), sw.reshape(-1).to(dev),
                          None, False, [1, N])
    ref = oracle.torch_fp8_gemm(x8, False, w8, False, torch.float32, sx, sw)
    check(out, ref)
    # the GPU per-row cast feeding the GEMM gives the same bits as the oracle's
    amax = torch.ops.mi355q.rowwise_amax(x.to(dev))
    assert torch.equal(amax.cpu(), x.abs().amax(1).float())
    s = (448.0 / amax).reshape(M, 1)
    x8_gpu, _ = ops.cast_to_fp8_v2(x.to(dev), s, False, False, E4, [M, 1])
    assert torch.equal(x8_gpu.cpu().view(torch.uint8), oracle.c_cast_to_fp8(x, s.cpu(), E4, scale_shape=[M, 1])[0].view(torch.uint8))


def test_config3_shape_properties(oracle, dev):
    """benchmark configuration 3 at full size (8192 x 4096 x 14336, per-tensor scales, bias).
    The CPU reference covers a sampled block of rows and columns; the whole output is
    covered by linearity in the scale and by an exact small-integer run."""
    g = torch.Generator().manual_seed(0xC001A1)
    M, K, N = 8192, 4096, 14336
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(K, N, generator=g) * 0.02).bfloat16()
    sa = 448.0 / a.abs().max().float()
    sw = 448.0 / w.abs().max().float()
    a8, _ = ops.cast_to_fp8_v2(a.to(dev), sa.to(dev), False, False, E4)
    w8, _ = ops.cast_to_fp8_v2(w.to(dev), sw.to(dev), False, False, E4)
    bias = (torch.randn(N, generator=g) * 0.01).bfloat16()
    out = ops.fp8_gemm_v2(a8, False, w8, False, None, torch.bfloat16, (1 / sa).to(dev), (1 / sw).to(dev), bias.to(dev), False)
    assert out.shape == (M, N)
    rows = torch.cat([torch.arange(0, 64), torch.arange(4000, 4064), torch.arange(M - 64, M)])
    colsel = torch.cat([torch.arange(0, 128), torch.arange(7000, 7128), torch.arange(N - 128, N)])
    a8c, w8c = a8.cpu(), w8.cpu()
    ref = oracle.torch_fp8_gemm(a8c[rows], False, w8c[:, colsel], False, torch.float32, 1 / sa, 1 / sw, bias=bias[colsel])
    check(out.cpu()[rows][:, colsel], ref, "sampled block")
    # linearity: doubling A's scale doubles (out - bias) exactly (power of two)
    out2 = ops.fp8_gemm_v2(a8, False, w8, False, None, torch.float32, (2 / sa).to(dev), (1 / sw).to(dev), None, False)
    out1 = ops.fp8_gemm_v2(a8, False, w8, False, None, torch.float32, (1 / sa).to(dev), (1 / sw).to(dev), None, False)
    assert torch.equal(out2, out1 * 2)
    del out, out1, out2
    # exactness at full size: small integers, K = 4096 keeps |sum| < 2^24
    gi = torch.Generator().manual_seed(5)
    Ai = torch.randint(-2, 3, (M, K), generator=gi).float().to(E4)
    Bi = torch.randint(-2, 3, (K, N), generator=gi).float().to(E4)
    got = ops.fp8_gemm_v2(Ai.to(dev), False, Bi.to(dev), False, None, torch.float32)
    expect = torch.matmul(Ai.to(dev).float(), Bi.to(dev).float())  # integers: exact in any order
    assert torch.equal(got, expect)


def test_c_abi_direct(oracle, pkg, dev):
    lib = pkg.capi()
    g = torch.Generator().manual_seed(77)
    M, K, N = 192, 256, 320
    A = small_int_fp8((M, K), E4, g)
    B = small_int_fp8((N, K), E5, g)          # trans_b: [N, K]
    sa = torch.rand(M, generator=g) + 0.5
    sb = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g)
    Ad, Bd, sad, sbd, bd = A.to(dev), B.to(dev), sa.to(dev), sb.to(dev), bias.to(dev)
    C = torch.empty(M, N, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = lib.mi355q_fp8_gemm(Ad.data_ptr(), pkg.E4M3FN, 0, K, Bd.data_ptr(), pkg.E5M2, 1, K, C.data_ptr(), pkg.F32, N,
                             M, N, K, sad.data_ptr(), 1.0, pkg.GS_PER_ROW, sbd.data_ptr(), 1.0, pkg.GS_PER_COL,
                             bd.data_ptr(), pkg.BIAS_ROW_VECTOR, 0, None, 0, 1, 0, 0, 0, 0, 0, stream)
    assert st == 0
    torch.cuda.synchronize()
    ref = oracle.c_fp8_gemm(A, False, B, True, torch.float32, sa.reshape(M, 1), sb, bias=bias, B_scale_shape=[1, N])
    rel, ok = gemm_errors(C, ref)
    assert rel < 1e-5 and ok, rel


@pytest.mark.parametrize("M", [32, 512])
def test_operand_larger_than_2_gib(dev, M):
    """B of 16384 x 131200 bytes (2.0 GiB + 2 MiB): the descriptors walk along K, so no offset
    inside the kernels depends on the size of the matrix.  Exact small-integer products; the
    columns checked include the last ones, whose high-k rows lie beyond 2 GiB."""
    K, N = 16384, 131200
    g = torch.Generator(device=dev).manual_seed(M)
    B = torch.randint(-4, 5, (K, N), generator=g, device=dev, dtype=torch.int8).to(torch.float16).to(E4)
    A = torch.randint(-4, 5, (M, K), generator=g, device=dev, dtype=torch.int8).to(torch.float16).to(E4)
    assert B.numel() > 2 ** 31
    out = ops.fp8_gemm_v2(A, False, B, False, None, torch.float32)
    a32 = A.float()
    for c0 in (0, 65536, N - 256):
        expect = a32 @ B[:, c0:c0 + 256].float()   # |sum| <= 16 K < 2^24: exact in any order
        assert torch.equal(out[:, c0:c0 + 256], expect), c0
