"""GPU parity at the full sizes of benchmark configurations 4 and 5, against the CPU oracle.

Configuration 4 (decode-shaped GEMM, K = 8192, N = 28672, M in {16, 64, 256}, per-token x
per-channel scales) is compared over the whole output: the CPU reference of an [M, 8192] x
[8192, 28672] product takes seconds.  Configuration 5 (the decoder MLP block, 4096 tokens, d = 4096,
ff = 14336) runs on the GPU exactly as the benchmark runs it and is compared stage by stage on a
sample of token rows (rows are independent): the fp8 codes and scales of both quantisations bit
for bit, the GEMM outputs within 1e-2 of the fp32-accumulated reference.
"""
import pytest
import torch

from helpers import E4, assert_fp8_equal, gemm_errors

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu
TOL = 1e-2   # max|out - ref| / max|ref| against the fp32-accumulated CPU reference of the dequantised operands


def per_channel_weights(dev, k, n, gen):
    """N(0, 0.02) bf16 weights [k, n] quantised per output channel on the GPU: (w bf16 cpu, w8 dev, 1/scale dev)."""
    w = (torch.randn(k, n, generator=gen) * 0.02).bfloat16()
    wd = w.to(dev)
    s = 448.0 / wd.abs().amax(dim=0).float()
    w8 = ops.cast_to_fp8_v2(wd, s, False, False, E4, [1, n])[0]
    return w, w8, (1.0 / s).contiguous()


@pytest.fixture(scope="module")
def c4_weights(dev, oracle):
    gen = torch.Generator().manual_seed(0xC001A1)
    K, N = 8192, 28672
    w, w8, sw_inv = per_channel_weights(dev, K, N, gen)
    w8c = w8.cpu()
    # the weight codes the GPU cast produced are the oracle's (first, middle and last 128 channels)
    s = (1.0 / sw_inv).cpu()
    for c0 in (0, 14336, N - 128):
        ref, _ = oracle.c_cast_to_fp8(w[:, c0:c0 + 128].contiguous(), s[c0:c0 + 128], E4, scale_shape=[1, 128])
        assert_fp8_equal(w8c[:, c0:c0 + 128], ref, E4, f"weights, channels {c0}..")
    return {"w8": w8, "w8_t": w8.t().contiguous(), "sw_inv": sw_inv, "w32": w8c.float(), "sw_inv_cpu": sw_inv.cpu()}


@pytest.mark.parametrize("M", [16, 64, 256])
def test_config4_full_size(oracle, pkg, dev, c4_weights, M):
    """K = 8192, N = 28672 with the benchmark's input recipe, the whole [M, N] output against the
    reference, for weights stored [K, N] and [N, K] (trans_B)."""
    K, N = 8192, 28672
    gen = torch.Generator().manual_seed(1000 + M)
    cols = torch.randperm(K, generator=gen)[:82]          # 1 % heavy-tail channels
    x = torch.randn(M, K, generator=gen)
    x[:, cols] *= 20
    x = x.bfloat16()
    x8, sx_inv = torch.ops.mi355q.quantize_rows(x.to(dev), E4)
    x8_ref, sx_ref = oracle.quantize_rows(x, E4)
    assert_fp8_equal(x8, x8_ref, E4, "activations")
    assert torch.equal(sx_inv.cpu(), sx_ref)
    ref = (x8_ref.float() @ c4_weights["w32"]) * sx_ref * c4_weights["sw_inv_cpu"]
    lib = pkg.capi()
    for trans_b, w8 in ((False, c4_weights["w8"]), (True, c4_weights["w8_t"])):
        variant = lib.mi355q_fp8_gemm_variant(0, K, int(trans_b), K if trans_b else N, M, N, K).decode()
        assert "simple" not in variant
        out = ops.fp8_gemm_v2(x8, False, w8, trans_b, None, torch.bfloat16, sx_inv, c4_weights["sw_inv"], None, False, [1, N])
        rel, ok = gemm_errors(out, ref)
        assert rel <= TOL and ok, f"M={M} trans_B={trans_b} ({variant}): rel {rel}"


@pytest.mark.parametrize("M", [16, 64, 128, 256])
def test_config4_full_size_exact(dev, M):
    """Small-integer operands at K = 8192, N = 28672 (|sum| <= 4 * 8192 < 2^24, so any accumulation
    order gives the same fp32 bits), power-of-two per-row and per-column scales: the bf16 output is
    determined bit for bit, every column of every strip and tile."""
    K, N = 8192, 28672
    g = torch.Generator(device=dev).manual_seed(M)
    A = torch.randint(-2, 3, (M, K), generator=g, device=dev, dtype=torch.int8).to(torch.float16).to(E4)
    B = torch.randint(-2, 3, (K, N), generator=g, device=dev, dtype=torch.int8).to(torch.float16).to(E4)
    sa = torch.exp2(torch.randint(-3, 4, (M, 1), generator=g, device=dev).float())
    sb = torch.exp2(torch.randint(-3, 4, (N,), generator=g, device=dev).float())
    expect = (torch.matmul(A.float(), B.float()) * sa * sb)     # integers times powers of two: exact
    out = ops.fp8_gemm_v2(A, False, B, False, None, torch.bfloat16, sa, sb, None, False, [1, N])
    assert torch.equal(out, expect.bfloat16())
    out_t = ops.fp8_gemm_v2(A, False, B.t().contiguous(), True, None, torch.float32, sa, sb, None, False, [1, N])
    assert torch.equal(out_t, expect)


def test_config5_mlp_block_pipeline(oracle, dev):
    """The block as the benchmark runs it: quantize_rows(x) -> one GEMM over the [d, 2 ff] gate / up
    weights -> silu_mul_quantize_rows on the two column ranges of its output -> down GEMM.  Every stage
    of the GPU run is checked on sampled token rows against the oracle applied to that stage's GPU input
    (quantisations: codes and scales bit for bit; GEMMs: 1e-2), and the block's output against the oracle
    chain run end to end on the CPU."""
    gen = torch.Generator().manual_seed(0xC001A1)
    T, d, ff = 4096, 4096, 14336
    _, wg8, sg = per_channel_weights(dev, d, ff, gen)
    _, wu8, su = per_channel_weights(dev, d, ff, gen)
    _, wd8, sdn = per_channel_weights(dev, ff, d, gen)
    wgu8 = torch.cat([wg8, wu8], dim=1).contiguous()
    sgu = torch.cat([sg, su]).contiguous()
    x = torch.randn(T, d, generator=gen).bfloat16()

    xd = x.to(dev)
    x8, sx = torch.ops.mi355q.quantize_rows(xd, E4)
    gu = ops.fp8_gemm_v2(x8, False, wgu8, False, None, torch.bfloat16, sx, sgu, None, False, [1, 2 * ff])
    h8, sh = torch.ops.mi355q.silu_mul_quantize_rows(gu[:, :ff], gu[:, ff:], E4)
    y = ops.fp8_gemm_v2(h8, False, wd8, False, None, torch.bfloat16, sh, sdn, None, False, [1, d])
    assert y.shape == (T, d)

    rows = torch.cat([torch.arange(0, 16), torch.arange(248, 264), torch.arange(2040, 2056), torch.arange(T - 16, T)])
    wgu32, wd32 = wgu8.cpu().float(), wd8.cpu().float()
    sgu_c, sdn_c = sgu.cpu(), sdn.cpu()

    # stage 1: dynamic per-token quantisation of x
    x8_ref, sx_ref = oracle.quantize_rows(x[rows], E4)
    assert_fp8_equal(x8.cpu()[rows], x8_ref, E4, "x8")
    assert torch.equal(sx.cpu()[rows], sx_ref)
    # stage 2: gate / up projection
    gu_ref = (x8_ref.float() @ wgu32) * sx_ref * sgu_c
    gu_gpu = gu.cpu()[rows]
    rel, ok = gemm_errors(gu_gpu, gu_ref)
    assert rel <= TOL and ok, f"gate / up GEMM: rel {rel}"
    # stage 3: bf16 SiLU(gate) * up and re-quantisation, from the GPU's own gate / up values
    h_ref = oracle.c_silu_mul_bf16(gu_gpu[:, :ff].contiguous(), gu_gpu[:, ff:].contiguous())
    h8_ref, sh_ref = oracle.quantize_rows(h_ref, E4)
    assert_fp8_equal(h8.cpu()[rows], h8_ref, E4, "h8")
    assert torch.equal(sh.cpu()[rows], sh_ref)
    # stage 4: down projection
    y_ref = (h8_ref.float() @ wd32) * sh_ref * sdn_c
    rel, ok = gemm_errors(y.cpu()[rows], y_ref)
    assert rel <= TOL and ok, f"down GEMM: rel {rel}"

    # end to end on the CPU: quantize_rows -> GEMM -> silu * up -> quantize_rows -> GEMM, nothing from the GPU
    gu_cpu = gu_ref.bfloat16()
    h8_cpu, sh_cpu = oracle.quantize_rows(oracle.c_silu_mul_bf16(gu_cpu[:, :ff].contiguous(), gu_cpu[:, ff:].contiguous()), E4)
    y_cpu = (h8_cpu.float() @ wd32) * sh_cpu * sdn_c
    rel, _ = gemm_errors(y.cpu()[rows], y_cpu)
    assert rel <= TOL, f"block output against the CPU chain: rel {rel}"


def test_batched_activation_times_one_weight_matrix(oracle, pkg, dev):
    """A [batch, M, K] activation times a 2-D weight matrix is one product over batch * M rows (the
    form aten.linear lowers to); per-token scales shaped [batch, M, 1], as quantize_rows returns
    them, a bias vector, a full bias and an accumulate input all follow the flattening."""
    g = torch.Generator().manual_seed(3)
    batch, M, K, N = 6, 5, 512, 384
    x = (torch.randn(batch, M, K, generator=g) * 2).bfloat16()
    w = (torch.randn(K, N, generator=g) * 0.05).bfloat16()
    x8, sx = torch.ops.mi355q.quantize_rows(x.to(dev), E4)
    assert sx.shape == (batch, M, 1)
    sw = 448.0 / w.abs().amax(dim=0).float()
    w8, _ = oracle.c_cast_to_fp8(w, sw, E4, scale_shape=[1, N])
    bias = torch.randn(N, generator=g).bfloat16()
    full = torch.randn(batch, M, N, generator=g).bfloat16()
    x8c, sxc = x8.cpu(), sx.cpu()
    for b_, d_ in ((None, None), (bias, None), (full, None), (bias, full)):
        out = ops.fp8_gemm_v2(x8, False, w8.to(dev), False, None if d_ is None else d_.to(dev), torch.bfloat16, sx,
                              (1 / sw).to(dev), None if b_ is None else b_.to(dev), d_ is not None, [1, N])
        assert out.shape == (batch, M, N)
        ref = oracle.torch_fp8_gemm(x8c, False, w8, False, torch.float32, sxc, 1 / sw, bias=b_, D=d_, B_scale_shape=[1, N])
        rel, ok = gemm_errors(out, ref)
        assert rel <= TOL and ok, rel
    # scales of shape [M, 1] shared by the batch elements, exact operands
    A = torch.randint(-3, 4, (batch, M, K), generator=g).float().to(E4)
    B = torch.randint(-3, 4, (K, N), generator=g).float().to(E4)
    sa = torch.exp2(torch.randint(-2, 3, (M, 1), generator=g).float())
    out = ops.fp8_gemm_v2(A.to(dev), False, B.to(dev), False, None, torch.float32, sa.to(dev))
    assert torch.equal(out.cpu(), torch.matmul(A.float(), B.float()) * sa)
    # the decode form [64, 1, K] x [K, N] is one 64-row strip, not 64 one-row products
    xs = torch.randint(-3, 4, (64, 1, K), generator=g).float().to(E4)
    out = ops.fp8_gemm_v2(xs.to(dev), False, B.to(dev), False, None, torch.float32)
    assert torch.equal(out.cpu(), torch.matmul(xs.float(), B.float()))
