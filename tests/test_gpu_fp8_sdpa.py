"""GPU parity of hpu::fp8_sdpa_recomp_fwd (inference forward, fp8 q / k / v) against the CPU oracle.

Floating point, so a tolerance, stated here once.  The oracle follows the kernel's own schedule (online
softmax over blocks of 64 keys, probabilities rounded to fp8 before the second product) in float64; the
device accumulates in fp32 and uses the hardware exp2, so two things separate them: the final rounding
of an output that sits near a rounding boundary (one bf16 step = 2^-8 relative, one e4m3 step = 2^-3),
and a probability that sits near an fp8 rounding boundary and falls to the other side (one e4m3 step on
one of kv_len terms: about one probability in 10^4 does, and it moves the 'head_dim_v' outputs of its row
by up to 2^-3 p_j / l |v_j|).  Bound used for a bf16 output: |out - ref| <= 2^-7 |ref| + 4e-3 max|ref| for
all but 0.5 % of the values, and <= that + 2^-3 max|v d_scale_v| for every value; for an fp8 output at
least 97 % of the codes are equal and the values obey the same two bounds with 2^-3 |ref| for 2^-7 |ref|.  The reference's own test
compares the device with plain bf16 attention at atol 0.4 / rtol 1e-3 (fp8 run) -- that looser check is
run as well (tests/pytest_working/any_mode/FusedSDPA/test_hpu_sdpa_fp8.py:1046-1052).
"""
import ctypes
import math

import pytest
import torch

from helpers import E4, E5

pytestmark = pytest.mark.gpu

NONE6 = (None,) * 6


def make_qkv(gen, qshape, kshape, vshape, fmt=E4, spread=1.0):
    q = (torch.randn(*qshape, generator=gen) * spread).to(fmt)
    k = (torch.randn(*kshape, generator=gen) * spread).to(fmt)
    v = torch.randn(*vshape, generator=gen).to(fmt)
    return q, k, v


def run_op(dev, q, k, v, mask=None, scale=None, causal=False, scales=NONE6, amax_s=False, amax_o=False, scalar=False):
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    if scalar:
        sc = [0.0 if s is None else float(s) for s in scales]
        op = torch.ops.hpu.fp8_sdpa_recomp_fwd.scalar
    else:
        sc = [None if s is None else torch.tensor([float(s)], device=dev) for s in scales]
        op = torch.ops.hpu.fp8_sdpa_recomp_fwd
    return op(q.to(dev), k.to(dev), v.to(dev), None if mask is None else mask.to(dev), 0.0, scale, causal, False, "None",
              *sc, amax_s, amax_o, None, "left")


def key_walk(pkg, q, k, v, workspace=True):
    """How the device walks the keys of this problem (None: block after block): asked of the library with the
    description the torch layer builds (batch extents right-aligned to three, stride 0 where k / v are broadcast)."""
    nb = q.dim() - 2
    bshape = list(torch.broadcast_shapes(q.shape[:-2], k.shape[:-2], v.shape[:-2]))
    batch = [1] * (3 - nb) + bshape

    def strides(t):
        st = [0] * (3 - nb) + [0 if t.shape[i] == 1 else t.stride(i) for i in range(nb)]
        return st
    desc = (ctypes.c_int64 * 29)(*batch, *strides(q), *strides(k), *strides(v), 0, 0, 0, 0, 0, 0,
                                 q.shape[-2], k.shape[-2], q.shape[-1], v.shape[-1],
                                 q.stride(-2), k.stride(-2), v.stride(-2), 0, v.shape[-1])
    per = ctypes.c_int64(0)
    n = pkg.capi().mi355q_fp8_sdpa_key_splits(desc, ctypes.byref(per))
    if n == 0:
        return None
    if not workspace:
        return (1, -(-k.shape[-2] // 64), 4)
    return (n, per.value, 4)


def check_bf16(out, ref, what="", vmax=None):
    """vmax: max |v * d_scale_v| (the largest value an output can take); max |ref| stands in when not given."""
    out, ref = out.cpu().float(), ref.float()
    assert out.shape == ref.shape, what
    tol = ref.abs() * 2.0 ** -7 + 4e-3 * ref.abs().max()
    err = (out - ref).abs()
    bad = err > tol
    assert float(bad.float().mean()) <= 5e-3, f"{what}: {int(bad.sum())} of {bad.numel()} outside the tight bound"
    loose = tol + 2.0 ** -3 * (float(ref.abs().max()) if vmax is None else vmax)
    assert not (err > loose).any(), f"{what}: worst {float((err - loose).max())} beyond one flipped probability"


def check_fp8(out, ref, what=""):
    """Codes equal for at least 97 % of the values; the others within one e4m3 step of the reference's
    magnitude plus the absolute term of the bf16 bound (values near zero have tiny steps)."""
    a, b = out.cpu().float(), ref.float()
    same = out.cpu().view(torch.uint8) == ref.view(torch.uint8)
    assert float(same.float().mean()) >= 0.97, f"{what}: only {float(same.float().mean()):.4f} of the codes agree"
    tol = b.abs() * 2.0 ** -3 + 4e-3 * b.abs().max()
    err = (a - b).abs()
    assert float((err > tol).float().mean()) <= 5e-3, f"{what}: {int((err > tol).sum())} values beyond one step"
    loose = tol + 2.0 ** -3 * b.abs().max()          # one flipped probability, as for a bf16 output
    assert not (err > loose).any(), f"{what}: worst {float((err - loose).max())} beyond one flipped probability"


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [
    # (batch, q_heads, kv_heads, q_len, kv_len, head_dim_qk, head_dim_v)
    (3, 4, 4, 16, 32, 8, 8),        # the reference test's own case (test_hpu_sdpa_fp8.py:454-476)
    (2, 3, 3, 128, 128, 64, 64),
    (1, 2, 2, 200, 333, 128, 128),
    (2, 2, 2, 257, 257, 128, 128),
    (1, 2, 2, 130, 190, 256, 256),
    (1, 2, 2, 96, 160, 72, 40),     # head dimensions that are no multiple of 16, and differ
    (1, 1, 1, 1, 700, 128, 128),    # one query (decoding)
    (1, 2, 2, 300, 1500, 64, 64),   # many blocks: the ring of K / V stages in steady state, 64-byte K rows
    (1, 2, 1, 260, 1100, 128, 128),
    (1, 1, 1, 140, 900, 256, 256),
    (1, 1, 1, 200, 1000, 96, 48),
    (2, 1, 1, 3, 64, 64, 128),
])
def test_against_oracle(oracle, pkg, dev, shape, causal):
    B, H, HK, L, S, DK, DV = shape
    gen = torch.Generator().manual_seed(L * 1000 + S + DK)
    q, k, v = make_qkv(gen, (B, H, L, DK), (B, HK, S, DK), (B, HK, S, DV))
    scales = (0.5, 2.0, 0.25, 128.0, None, 1.0 / 128.0)
    out, m, linv, seed, amax_s, amax_o = run_op(dev, q, k, v, causal=causal, scales=scales, amax_s=True, amax_o=True)
    assert out.dtype == torch.bfloat16 and m.shape == (1,) and linv.shape == (1,) and seed.dtype == torch.int32
    ref, ref_as, ref_ao = oracle.torch_fp8_sdpa(q, k, v, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0, d_scale_v=0.25,
                                                q_scale_s=128.0, d_scale_s=1.0 / 128.0, key_streams=key_walk(pkg, q, k, v))
    check_bf16(out, ref, str(shape))
    assert abs(float(amax_s.cpu()) - float(ref_as)) <= 1e-4 * float(ref_as)
    assert abs(float(amax_o.cpu()) - float(ref_ao)) <= 2e-3 * float(ref_ao)
    # the reference test's own check: plain attention on the dequantised inputs, atol 0.4 / rtol 1e-3
    keep = torch.ones(L, S, dtype=torch.bool).tril() if causal else None
    plain = torch.nn.functional.scaled_dot_product_attention(q.float() * 0.5, k.float() * 2.0, v.float() * 0.25, attn_mask=keep)
    assert torch.allclose(out.cpu().float(), plain, atol=0.4, rtol=1e-3)


@pytest.mark.parametrize("scalar", [False, True])
@pytest.mark.parametrize("causal", [False, True])
def test_fp8_output(oracle, dev, causal, scalar):
    """q_scale_o given: the output is e4m3fn holding out * q_scale_o (sdpa_gen.cpp:922-934)."""
    gen = torch.Generator().manual_seed(5)
    q, k, v = make_qkv(gen, (2, 4, 150, 128), (2, 4, 210, 128), (2, 4, 210, 128))
    scales = (1.0, 1.0, 1.0, 128.0, 64.0, 1.0 / 128.0)
    out = run_op(dev, q, k, v, causal=causal, scales=scales, scalar=scalar)[0]
    assert out.dtype == E4
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=causal, q_scale_s=128.0, q_scale_o=64.0, d_scale_s=1.0 / 128.0)
    check_fp8(out, ref)
    plain = torch.nn.functional.scaled_dot_product_attention(
        q.float(), k.float(), v.float(), attn_mask=torch.ones(150, 210, dtype=torch.bool).tril() if causal else None)
    assert torch.allclose(out.cpu().float() / 64.0, plain, atol=0.4, rtol=1e-3)


def test_defaults_without_scales(oracle, dev):
    """No scale given: all are 1, d_scale_s = 1 / q_scale_s = 1."""
    gen = torch.Generator().manual_seed(6)
    q, k, v = make_qkv(gen, (2, 100, 64), (2, 90, 64), (2, 90, 64))         # rank 3
    out = run_op(dev, q, k, v)[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v)
    check_bf16(out, ref)
    # q_scale_s alone: d_scale_s defaults to its inverse
    out = run_op(dev, q, k, v, scales=(None, None, None, 100.0, None, None))[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=100.0)
    check_bf16(out, ref)


@pytest.mark.parametrize("kind", ["bool", "bf16", "f32"])
@pytest.mark.parametrize("mshape", ["Bx1x1xN", "BxHxLxN", "LxN", "1x1xLx1"])
def test_attention_masks(oracle, dev, kind, mshape):
    B, H, L, S, D = 2, 3, 70, 150, 64
    gen = torch.Generator().manual_seed(7)
    q, k, v = make_qkv(gen, (B, H, L, D), (B, H, S, D), (B, H, S, D))
    shp = {"Bx1x1xN": (B, 1, 1, S), "BxHxLxN": (B, H, L, S), "LxN": (L, S), "1x1xLx1": (1, 1, L, 1)}[mshape]
    keep = torch.rand(*shp, generator=gen) > 0.3
    if mshape != "1x1xLx1":
        keep[..., 0] = True
    elif kind != "bool":
        # a float mask that is -1e9 for every key of a row leaves fp32 no bits for the scores themselves
        keep[...] = True
    if kind == "bool":
        mask = keep
    else:
        # the reference's float mask holds 0 and a large negative number (test_hpu_sdpa_fp8.py:272-276)
        mask = torch.where(keep, 0.0, -1e9) + torch.where(keep, torch.randn(*shp, generator=gen) * 0.5, 0.0)
        mask = mask.to(torch.bfloat16 if kind == "bf16" else torch.float32)
    out = run_op(dev, q, k, v, mask=mask, scales=(None, None, None, 128.0, None, 1 / 128.0))[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=mask, q_scale_s=128.0, d_scale_s=1 / 128.0)
    check_bf16(out, ref, f"{kind} {mshape}")


def test_rows_with_every_key_masked_give_zero(oracle, dev):
    gen = torch.Generator().manual_seed(8)
    q, k, v = make_qkv(gen, (1, 2, 40, 64), (1, 2, 100, 64), (1, 2, 100, 64))
    keep = torch.rand(1, 1, 40, 100, generator=gen) > 0.5
    keep[:, :, 5] = False
    keep[:, :, 33] = False
    out, _, _, _, amax_s, _ = run_op(dev, q, k, v, mask=keep, amax_s=True)
    ref, ref_as, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=keep)
    assert (out.cpu()[:, :, [5, 33]] == 0).all()
    check_bf16(out, ref)
    assert abs(float(amax_s.cpu()) - float(ref_as)) <= 1e-4 * float(ref_as)


def test_grouped_query_layout(oracle, dev):
    """The 5-d views the reference's wrapper builds for grouped-query attention: q [B, G, H/G, L, D], k and
    v [B, G, 1, S, D], mask [B, 1, 1, L, S] (Fp8FusedSDPA.py:49-77); and multi-query, kv_heads == 1."""
    B, G, HG, L, S, D = 2, 2, 4, 90, 130, 128
    gen = torch.Generator().manual_seed(9)
    q, k, v = make_qkv(gen, (B, G, HG, L, D), (B, G, 1, S, D), (B, G, 1, S, D))
    mask = torch.where(torch.rand(B, 1, 1, L, S, generator=gen) > 0.2, 0.0, -1e9).to(torch.bfloat16)
    out = run_op(dev, q, k, v, mask=mask, scales=(None, None, None, 128.0, None, 1 / 128.0))[0]
    assert out.shape == (B, G, HG, L, D)
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=mask, q_scale_s=128.0, d_scale_s=1 / 128.0)
    check_bf16(out, ref)
    q4, k4, v4 = make_qkv(gen, (B, 8, L, D), (B, 1, S, D), (B, 1, S, D))
    out = run_op(dev, q4, k4, v4, causal=True)[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q4, k4, v4, is_causal=True)
    check_bf16(out, ref)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_e5m2_inputs(oracle, dev, D):
    gen = torch.Generator().manual_seed(10 + D)
    q, k, v = make_qkv(gen, (2, 2, 100, D), (2, 2, 140, D), (2, 2, 140, D), fmt=E5)
    out = run_op(dev, q, k, v, causal=True, scales=(None, None, None, 1024.0, None, 1 / 1024.0))[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, q_scale_s=1024.0, d_scale_s=1 / 1024.0)
    # e5m2 probabilities have a 2-bit mantissa: one flipped rounding weighs four times an e4m3 one
    out, ref = out.cpu().float(), ref.float()
    assert ((out - ref).abs() <= ref.abs() * 2.0 ** -7 + 1.5e-2 * ref.abs().max()).all()


@pytest.mark.parametrize("D", [64, 128])
def test_q_scale_s_beyond_the_fp8_range_saturates(oracle, dev, D):
    gen = torch.Generator().manual_seed(11)
    q, k, v = make_qkv(gen, (1, 2, 64, D), (1, 2, 64, D), (1, 2, 64, D), spread=3.0)
    out = run_op(dev, q, k, v, scales=(None, None, None, 1000.0, None, 1e-3))[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=1000.0, d_scale_s=1e-3)
    check_bf16(out, ref)


def test_views_into_a_packed_projection(oracle, dev):
    """q, k, v as strided views of one [B, L, 3, H, D] buffer (row pitch 3 H D), transposed to heads first."""
    B, L, H, D = 2, 160, 4, 128
    gen = torch.Generator().manual_seed(12)
    qkv = torch.randn(B, L, 3, H, D, generator=gen).to(E4).to(dev)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    assert not q.is_contiguous()
    scale = 1.0 / math.sqrt(D)
    out = torch.ops.hpu.fp8_sdpa_recomp_fwd(q, k, v, None, 0.0, scale, True, False, "fast", None, None, None, None, None, None,
                                            False, False, None, "left")[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    check_bf16(out, ref)


def test_long_sequence_properties(oracle, dev):
    """At a size the CPU oracle does not finish in seconds: properties that fix the result.  With v = 1
    everywhere every output is exactly d_scale_s q_scale_s-consistent 1 (a convex combination), rows of a
    causal run equal the rows of the same keys without the later ones, and sampled rows match the oracle."""
    B, H, L, D = 1, 4, 4096, 128
    gen = torch.Generator().manual_seed(13)
    q, k, v = make_qkv(gen, (B, H, L, D), (B, H, L, D), (B, H, L, D))
    sc = (None, None, None, 128.0, None, 1 / 128.0)
    out = run_op(dev, q, k, v, causal=True, scales=sc)[0].cpu()
    # sampled rows against the oracle: row i of a causal run only sees keys <= i
    for i in (0, 63, 64, 1000, 4095):
        # the oracle's blocks must start where the device's do, so give it all keys up to the block's end
        ref, _, _ = oracle.torch_fp8_sdpa(q[:, :, i:i + 1], k[:, :, :i + 1], v[:, :, :i + 1], q_scale_s=128.0, d_scale_s=1 / 128.0)
        check_bf16(out[:, :, i:i + 1], ref, f"row {i}")
    ones = torch.ones_like(v.float()).to(E4)
    o1 = run_op(dev, q, k, ones, causal=True, scales=sc)[0].cpu().float()
    # sum of fp8-rounded probabilities over the sum of unrounded ones: within the fp8 rounding, 2^-4
    assert (o1 - 1.0).abs().max() <= 2.0 ** -4


@pytest.mark.parametrize("D", [128, 256])
def test_prefill_at_the_benchmark_shape(oracle, dev, D):
    """32 query / 8 kv heads, q_len = kv_len = 8192, head_dim 128 or 256, causal, in the wrapper's grouped layout (what
    bench.py times as fp8_sdpa_B1_L8192 and fp8_sdpa_B1_L8192_D256: 64 query blocks x 32 heads, kv broadcast along the
    heads of a group; at 256 two workgroups share a CU and the ring of two stages wraps 64 times):
    sampled rows of sampled heads against the oracle, every row of one head against the property that v = 1 gives 1."""
    G, HG, L = 8, 4, 8192
    gen = torch.Generator().manual_seed(8192 + D)
    q, k, v = make_qkv(gen, (1, G, HG, L, D), (1, G, 1, L, D), (1, G, 1, L, D))
    sc = (None, None, None, 128.0, None, 1 / 128.0)
    out = run_op(dev, q, k, v, causal=True, scales=sc)[0].cpu()
    assert out.shape == (1, G, HG, L, D)
    rows = [0, 1, 63, 64, 127, 128, 4095, 4096, 5000, 8063, 8064, 8191]
    for g, h in ((0, 0), (3, 2), (7, 3)):
        # the rows of a head are judged together: the bound allows 0.5 % of the values one flipped fp8 rounding
        refs = [oracle.torch_fp8_sdpa(q[0, g, h, i:i + 1], k[0, g, 0, :i + 1], v[0, g, 0, :i + 1], q_scale_s=128.0, d_scale_s=1 / 128.0)[0]
                for i in rows]
        check_bf16(out[0, g, h, rows], torch.cat(refs), f"group {g} head {h}", vmax=float(v.float().abs().max()))
    # heads of one group differ (their queries do), groups read their own k / v
    assert not torch.equal(out[0, 0, 0], out[0, 0, 1]) and not torch.equal(out[0, 0, 0], out[0, 1, 0])
    o1 = run_op(dev, q, k, torch.ones_like(v.float()).to(E4), causal=True, scales=sc)[0].cpu().float()
    assert (o1 - 1.0).abs().max() <= 2.0 ** -4


@pytest.mark.parametrize("case", [
    # (batch, kv heads, query heads per kv head, q_len, kv_len, head_dim, causal, mask)
    (2, 2, 4, 1, 1000, 128, False, None),        # grouped-query decoding, keys split over workgroups
    (1, 1, 8, 4, 4096, 128, False, "bf16"),      # 32 rows: 8 heads x 4 queries, float mask
    (3, 2, 4, 1, 700, 64, False, "bool"),        # head dimension 64, ragged last block, bool mask
    (2, 3, 1, 5, 900, 128, True, None),          # no sharing (one query head per kv head), causal from the top left
    (1, 2, 4, 2, 8192, 128, False, None),        # long cache
    (16, 8, 4, 1, 2048, 128, False, None),       # many groups: no split, one workgroup each
    (1, 1, 4, 1, 520, 80, False, None),          # head dimension 80 (padded to 128 in LDS)
])
def test_few_queries_against_many_keys(oracle, pkg, dev, case):
    """Decoding shapes take the kernel that packs the queries sharing a k / v into one tile and splits the keys:
    same results as the oracle, in the reference wrapper's grouped layout, with and without fp8 output and amax."""
    B, G, HG, L, S, D, causal, mk = case
    gen = torch.Generator().manual_seed(S + D + L)
    q, k, v = make_qkv(gen, (B, G, HG, L, D), (B, G, 1, S, D), (B, G, 1, S, D))
    mask = None
    if mk is not None:
        keep = torch.rand(B, 1, 1, L, S, generator=gen) > 0.3
        keep[..., 0] = True
        mask = keep if mk == "bool" else torch.where(keep, 0.0, -1e9).to(torch.bfloat16)
    sc = (0.5, 2.0, 0.25, 128.0, None, 1 / 128.0)
    out, _, _, _, amax_s, amax_o = run_op(dev, q, k, v, mask=mask, causal=causal, scales=sc, amax_s=True, amax_o=True)
    walk = key_walk(pkg, q, k, v)
    assert walk is not None
    ref, ref_as, ref_ao = oracle.torch_fp8_sdpa(q, k, v, attn_mask=mask, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0,
                                                d_scale_v=0.25, q_scale_s=128.0, d_scale_s=1 / 128.0, key_streams=walk)
    check_bf16(out, ref, str(case))
    assert abs(float(amax_s.cpu()) - float(ref_as)) <= 1e-4 * float(ref_as)
    assert abs(float(amax_o.cpu()) - float(ref_ao)) <= 2e-3 * float(ref_ao)
    out8 = run_op(dev, q, k, v, mask=mask, causal=causal, scales=(0.5, 2.0, 0.25, 128.0, 32.0, 1 / 128.0))[0]
    ref8, _, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=mask, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0, d_scale_v=0.25,
                                       q_scale_s=128.0, q_scale_o=32.0, d_scale_s=1 / 128.0, key_streams=walk)
    check_fp8(out8, ref8, str(case))


def test_few_queries_without_a_workspace(oracle, pkg, dev):
    """The C entry point without the workspace it asks for: one workgroup per group walks all the keys."""
    gen = torch.Generator().manual_seed(21)
    B, G, HG, S, D = 1, 2, 4, 3000, 128
    q, k, v = make_qkv(gen, (B, G, HG, 1, D), (B, G, 1, S, D), (B, G, 1, S, D))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = torch.empty(B, G, HG, 1, D, dtype=torch.bfloat16, device=dev)
    lib = pkg.capi()
    desc = (ctypes.c_int64 * 29)(B, G, HG, 0, HG * D, D, 0, S * D, 0, 0, S * D, 0, 0, 0, 0, 0, HG * D, D, 1, S, D, D, D, D, D, 0, D)
    assert lib.mi355q_fp8_sdpa_workspace_bytes(desc) > 0
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.mi355q_fp8_sdpa_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16, desc,
                                   1 / math.sqrt(D), 0, None, None, None, None, None, 0, st) == 0
    torch.cuda.synchronize()
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, key_streams=key_walk(pkg, q, k, v, workspace=False))
    check_bf16(out, ref)


def test_few_queries_with_the_callers_workspace(oracle, pkg, dev):
    """The C entry point with a workspace the caller zero-filled once: the splits' last workgroup merges them
    and returns the arrival counters to zero, so a second call (other data, the same workspace) and a third
    (the first data again) need nothing in between.  Same bits as the torch op, which runs the same kernel."""
    gen = torch.Generator().manual_seed(22)
    B, G, HG, S, D = 1, 2, 4, 3000, 128
    lib = pkg.capi()
    desc = (ctypes.c_int64 * 29)(B, G, HG, 0, HG * D, D, 0, S * D, 0, 0, S * D, 0, 0, 0, 0, 0, HG * D, D, 1, S, D, D, D, D, D, 0, D)
    nbytes = lib.mi355q_fp8_sdpa_workspace_bytes(desc)
    assert nbytes > 0 and lib.mi355q_fp8_sdpa_key_splits(desc, None) > 1
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    data = [make_qkv(gen, (B, G, HG, 1, D), (B, G, 1, S, D), (B, G, 1, S, D)) for _ in range(2)]
    for q, k, v in (data[0], data[1], data[0]):
        qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
        out = torch.empty(B, G, HG, 1, D, dtype=torch.bfloat16, device=dev)
        assert lib.mi355q_fp8_sdpa_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16, desc,
                                       1 / math.sqrt(D), 0, None, None, None, None, ws.data_ptr(), nbytes, st) == 0
        torch.cuda.synchronize()
        ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, key_streams=key_walk(pkg, q, k, v))
        check_bf16(out, ref)
        assert torch.equal(out, run_op(dev, q, k, v)[0])
    # the counters (the first KiB) are back at zero; the partial results behind them are not
    assert not ws[:1024].any() and ws[1024:].any()


def test_argument_checks(dev):
    q = torch.zeros(1, 2, 16, 64, device=dev).to(E4)
    args = (None, 0.0, 0.125, False, False, "None", None, None, None, None, None, None, False, False, None, "left")
    op = torch.ops.hpu.fp8_sdpa_recomp_fwd
    with pytest.raises(RuntimeError, match="requires_backward"):
        op(q, q, q, None, 0.0, 0.125, False, True, *args[5:])
    with pytest.raises(RuntimeError, match="dropout"):
        op(q, q, q, None, 0.1, *args[2:])
    with pytest.raises(RuntimeError, match="valid_seq_len"):
        op(q, q, q, *args[:14], torch.zeros(1, device=dev, dtype=torch.int32), "left")
    with pytest.raises(RuntimeError, match="exclude each other"):
        op(q, q, q, torch.ones(16, 16, device=dev, dtype=torch.bool), 0.0, 0.125, True, *args[4:])
    with pytest.raises(RuntimeError, match="same head dimension"):
        op(q, q[..., :32], q, *args)
    big = torch.zeros(1, 1, 4, 320, device=dev).to(E4)
    with pytest.raises(RuntimeError, match="up to 256"):
        op(big, big, big, *args)


def test_measurement_pass_with_bf16_inputs(dev):
    """bf16 q, k, v with is_amax_s: the pass that measures max softmax probability before an fp8 run
    (test_hpu_sdpa_fp8.py tc_list1).  No fp8 is involved; the device's own matmul and softmax run."""
    gen = torch.Generator().manual_seed(14)
    q = torch.randn(3, 4, 16, 8, generator=gen).bfloat16()
    k = torch.randn(3, 4, 32, 8, generator=gen).bfloat16()
    v = torch.randn(3, 4, 32, 8, generator=gen).bfloat16()
    out, _, _, _, amax_s, _ = torch.ops.hpu.fp8_sdpa_recomp_fwd(
        q.to(dev), k.to(dev), v.to(dev), None, 0.0, 1 / math.sqrt(8), True, False, "fast", None, None, None, None, None, None,
        True, False, None, "left")
    keep = torch.ones(16, 32, dtype=torch.bool).tril()
    s = (q.float() @ k.float().transpose(-2, -1)) / math.sqrt(8)
    p = torch.softmax(s.masked_fill(~keep, float("-inf")), -1)
    assert out.dtype == torch.bfloat16
    assert torch.allclose(out.cpu().float(), p @ v.float(), atol=0.08, rtol=1e-3)
    assert abs(float(amax_s.cpu()) - float(p.max())) <= 0.05


@pytest.mark.parametrize("mask_kind", ["none", "bool_rows", "float_one_row"])
def test_measurement_pass_walks_long_prompts_in_pieces(dev, monkeypatch, mask_kind):
    """The bf16 measurement pass holds fp32 scores [batch, L, S]; beyond a fixed number of elements it walks the queries
    in pieces.  With the limit forced down to 37 rows at a time the result equals the one-piece result (the triangle and
    a per-query mask are shifted with the piece)."""
    gen = torch.Generator().manual_seed(15)
    B, H, L, S, D = 2, 3, 150, 200, 16
    q = torch.randn(B, H, L, D, generator=gen).bfloat16().to(dev)
    k = torch.randn(B, H, S, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, H, S, D, generator=gen).bfloat16().to(dev)
    causal = mask_kind == "none"
    mask = None
    if mask_kind == "bool_rows":
        mask = (torch.rand(B, 1, L, S, generator=gen) > 0.3)
        mask[..., 0] = True
        mask = mask.to(dev)
    elif mask_kind == "float_one_row":
        mask = (torch.randn(1, 1, 1, S, generator=gen)).bfloat16().to(dev)

    def run():
        out, _, _, _, amax_s, amax_o = torch.ops.hpu.fp8_sdpa_recomp_fwd(
            q, k, v, mask, 0.0, 0.25, causal, False, "None", None, None, None, None, None, None, True, True, None, "left")
        return out.cpu().float(), float(amax_s.cpu()), float(amax_o.cpu())

    monkeypatch.delenv("MI355Q_SDPA_MEASURE_SCORE_ELEMENTS", raising=False)
    whole = run()
    monkeypatch.setenv("MI355Q_SDPA_MEASURE_SCORE_ELEMENTS", str(B * H * S * 37))
    pieces = run()
    assert torch.allclose(whole[0], pieces[0], atol=2e-2, rtol=1e-2)
    assert abs(whole[1] - pieces[1]) <= 1e-3 and abs(whole[2] - pieces[2]) <= 2e-2
    # and against plain attention
    s = (q.cpu().float() @ k.cpu().float().transpose(-2, -1)) * 0.25
    if causal:
        s = s.masked_fill(~torch.ones(L, S, dtype=torch.bool).tril(), float("-inf"))
    if mask_kind == "bool_rows":
        s = s.masked_fill(~mask.cpu(), float("-inf"))
    elif mask_kind == "float_one_row":
        s = s + mask.cpu().float()
    ref = torch.softmax(s, -1) @ v.cpu().float()
    assert torch.allclose(pieces[0], ref, atol=0.08, rtol=1e-2)


def test_c_entry_point_rejects_bad_arguments(pkg, dev):
    lib = pkg.capi()
    q = torch.zeros(16, 64, device=dev).to(E4)
    out = torch.zeros(16, 64, device=dev, dtype=torch.bfloat16)
    desc = (ctypes.c_int64 * 29)(*([1, 1, 1] + [0] * 15 + [16, 16, 64, 64] + [64, 64, 64, 0, 64]))
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ok = lib.mi355q_fp8_sdpa_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16,
                                 desc, 0.125, 0, None, None, None, None, None, 0, st)
    assert ok == 0
    torch.cuda.synchronize()
    assert (out == 0).all()          # v = 0
    assert lib.mi355q_fp8_sdpa_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), pkg.BF16, None, 0, out.data_ptr(), pkg.BF16,
                                   desc, 0.125, 0, None, None, None, None, None, 0, st) == 1
    assert lib.mi355q_fp8_sdpa_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), pkg.E4M3FN, None, 2, out.data_ptr(), pkg.BF16,
                                   desc, 0.125, 0, None, None, None, None, None, 0, st) == 1     # mask kind without a mask
    desc[20] = 300                   # head_dim_qk
    assert lib.mi355q_fp8_sdpa_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16,
                                   desc, 0.125, 0, None, None, None, None, None, 0, st) == 2


# ------------------------------------------------------------------ valid_seq_len / seq_padding_type

def run_valid(dev, op, q, k, v, valid, pad, scales=(None, None, None, 128.0, None, 1.0 / 128.0), scalar=False):
    scale = 1.0 / math.sqrt(q.shape[-1])
    sc = [0.0 if s is None else float(s) for s in scales] if scalar else [None if s is None else torch.tensor([float(s)], device=dev) for s in scales]
    return op(q.to(dev), k.to(dev), v.to(dev), None, 0.0, scale, True, False, "None", *sc, False, False, valid.to(dev), pad)


@pytest.mark.parametrize("pad", ["left", "right"])
@pytest.mark.parametrize("layout", ["bhld", "gqa5d", "bld"])
@pytest.mark.parametrize("S,D", [(200, 64), (333, 128), (130, 256)])
def test_valid_seq_len(oracle, dev, pad, layout, S, D):
    """The per-batch key window of the inference forward (sdpa_gen.cpp:849-851, 902-904; Fp8FusedSDPA.py:123-126),
    incl. the wrapper's 5-d grouped-query layout; counts of 0, 1, kv_len, beyond kv_len, and off the 64-key blocks."""
    gen = torch.Generator().manual_seed(S + D)
    B = 6
    if layout == "bhld":
        q, k, v = make_qkv(gen, (B, 2, S, D), (B, 2, S, D), (B, 2, S, D))
    elif layout == "gqa5d":
        q, k, v = make_qkv(gen, (B, 2, 2, S, D), (B, 2, 1, S, D), (B, 2, 1, S, D))
    else:
        q, k, v = make_qkv(gen, (B, S, D), (B, S, D), (B, S, D))
    valid = torch.tensor([S, 0, 1, S + 50, 64, S - 71], dtype=torch.int32)
    out = run_valid(dev, torch.ops.hpu.fp8_sdpa_recomp_fwd, q, k, v, valid, pad)[0]
    ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, q_scale_s=128.0, d_scale_s=1 / 128.0, valid_seq_len=valid,
                                      seq_padding_type=pad)
    check_bf16(out, ref, f"{pad} {layout} {S} {D}", vmax=float(v.float().abs().max()))
    # rows that see no key are exactly zero; an int64 tensor is taken as well, and so is the alias with .scalar
    o = out.cpu().float()
    assert torch.count_nonzero(o[1]) == 0
    if pad == "left":
        assert torch.count_nonzero(o[2][..., : S - 1, :]) == 0
    out2 = run_valid(dev, torch.ops.hpu.fp8_sdpa_recomp_fwd_non_dropout.scalar, q, k, v, valid.long(), pad, scalar=True)[0]
    assert torch.equal(out2.cpu().view(torch.int16), out.cpu().view(torch.int16))


def test_valid_seq_len_through_the_c_abi(oracle, pkg, dev):
    lib = pkg.capi()
    gen = torch.Generator().manual_seed(77)
    B, H, S, D = 3, 2, 300, 128
    q, k, v = make_qkv(gen, (B, H, S, D), (B, H, S, D), (B, H, S, D))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    valid = torch.tensor([300, 129, 7], dtype=torch.int32)
    vd_len = valid.to(dev)
    out = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    host = (ctypes.c_float * 6)(0, 0, 0, 128.0, 0, 1 / 128.0)
    for pad_left in (1, 0):
        desc = (ctypes.c_int64 * 29)(1, B, H, 0, H * S * D, S * D, 0, H * S * D, S * D, 0, H * S * D, S * D, 0, 0, 0, 0, H * S * D, S * D,
                                     S, S, D, D, D, D, D, 0, D, vd_len.data_ptr(), 1 | (pad_left << 32))
        assert lib.mi355q_fp8_sdpa_workspace_bytes(desc) == 0
        assert lib.mi355q_fp8_sdpa_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16, desc,
                                       1.0 / math.sqrt(D), 1, None, host, None, None, None, 0, st) == 0
        ref, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, q_scale_s=128.0, d_scale_s=1 / 128.0, valid_seq_len=valid,
                                          seq_padding_type="left" if pad_left else "right")
        check_bf16(out, ref, f"c abi pad_left={pad_left}", vmax=float(v.float().abs().max()))
    desc[28] = 3      # a batch dimension that does not exist
    assert lib.mi355q_fp8_sdpa_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), pkg.E4M3FN, None, 0, out.data_ptr(), pkg.BF16, desc,
                                   0.1, 1, None, host, None, None, None, 0, st) == 1


def test_valid_seq_len_needs_the_causal_mask(dev):
    q = torch.zeros(2, 2, 8, 16, device=dev).to(E4)
    valid = torch.tensor([8, 4], dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="valid_seq_len is supported only"):
        torch.ops.hpu.fp8_sdpa_recomp_fwd(q, q, q, None, 0.0, 0.25, False, False, "None", *NONE6, False, False, valid, "left")
    with pytest.raises(RuntimeError, match="one value per batch entry"):
        torch.ops.hpu.fp8_sdpa_recomp_fwd(q, q, q, None, 0.0, 0.25, True, False, "None", *NONE6, False, False, valid[:1], "left")
    with pytest.raises(RuntimeError, match="seq_padding_type"):
        torch.ops.hpu.fp8_sdpa_recomp_fwd(q, q, q, None, 0.0, 0.25, True, False, "None", *NONE6, False, False, valid, "middle")


def test_valid_seq_len_measurement_pass_in_bf16(oracle, dev):
    """bf16 q, k, v (the pass that measures amax_s): the same window."""
    gen = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, 2, 70, 32, generator=gen).bfloat16() for _ in range(3))
    valid = torch.tensor([70, 20], dtype=torch.int32)
    out = torch.ops.hpu.fp8_sdpa_recomp_fwd(q.to(dev), k.to(dev), v.to(dev), None, 0.0, 0.2, True, False, "None", *NONE6, True, False,
                                            valid.to(dev), "right")[0]
    for b, n in enumerate([70, 20]):
        ref = torch.nn.functional.scaled_dot_product_attention(q[b, :, :n].float(), k[b, :, :n].float(), v[b, :, :n].float(), is_causal=True, scale=0.2)
        assert torch.allclose(out[b, :, :n].cpu().float(), ref, atol=2e-2, rtol=2e-2)


# ------------------------------------------------------------------ fp8_sdpa_fwd: the forward that keeps P

@pytest.mark.parametrize("op_name", ["fp8_sdpa_fwd", "fp8_sdpa_fwd_non_dropout"])
@pytest.mark.parametrize("case", ["plain", "causal", "bool_mask", "float_mask", "gqa5d", "window_left", "fp8_out", "e5m2"])
def test_fp8_sdpa_fwd(oracle, dev, op_name, case):
    """out, P, the dropout-mask placeholder and amax_s of the forward without recomputation against
    oracle.torch_fp8_sdpa_unfused (Fp8SDPAFwd::AddNode, sdpa_gen.cpp:340-437).  P's codes are compared bit for bit
    apart from the few entries where the device's exp and the CPU's put a bf16 probability on the other side of a
    rounding step; out within the GEMM bar of 1e-2 of max |ref| plus what those entries can move."""
    gen = torch.Generator().manual_seed(len(case))
    fmt = E5 if case == "e5m2" else E4
    B, H, L, S, D = 2, 4, 96, 160, 64
    if case == "gqa5d":
        q, k, v = make_qkv(gen, (B, 2, 2, L, D), (B, 2, 1, S, D), (B, 2, 1, S, D), fmt)
    else:
        q, k, v = make_qkv(gen, (B, H, L, D), (B, H, S, D), (B, H, S, D), fmt)
    if case == "window_left":
        q = q[..., :S, :] if L >= S else torch.cat([q, q], -2)[..., :S, :].contiguous()
    mask, valid, causal = None, None, case in ("causal", "window_left", "gqa5d")
    if case == "bool_mask":
        mask = torch.rand(B, 1, L, S, generator=gen) > 0.3
        mask[..., 0] = True
    if case == "float_mask":
        mask = (torch.randn(1, 1, L, S, generator=gen)).bfloat16()
    if case == "window_left":
        valid = torch.tensor([S, 45], dtype=torch.int32)
    qo = 32.0 if case == "fp8_out" else None
    t = lambda x: None if x is None else torch.tensor([float(x)], device=dev)
    op = getattr(torch.ops.hpu, op_name)
    out, P, dm, amax_s = op(q.to(dev), k.to(dev), v.to(dev), None if mask is None else mask.to(dev), 0.0, 0.125, causal, "None",
                            t(0.5), t(2.0), t(0.25), t(128.0), t(qo), t(1 / 128.0), case == "plain",
                            None if valid is None else valid.to(dev), "left")
    ref, Pref, ref_as = oracle.torch_fp8_sdpa_unfused(q, k, v, attn_mask=mask, scale=0.125, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0,
                                                      d_scale_v=0.25, q_scale_s=128.0, q_scale_o=qo, d_scale_s=1 / 128.0,
                                                      valid_seq_len=valid, seq_padding_type="left")
    assert P.dtype == fmt and tuple(P.shape) == tuple(Pref.shape) and tuple(dm.shape) == (1,) and dm.dtype == torch.int8
    assert amax_s.dtype == torch.float32 and tuple(amax_s.shape) == (1,)
    assert out.dtype == (fmt if qo is not None else torch.bfloat16) and tuple(out.shape) == tuple(ref.shape)
    same = P.cpu().view(torch.uint8) == Pref.view(torch.uint8)
    assert float(same.float().mean()) >= 0.98, f"{case}: only {float(same.float().mean()):.4f} of the probability codes agree"
    step = Pref.float().abs() * (2.0 ** -2 if fmt == E5 else 2.0 ** -3) + 2.0 ** -6
    assert ((P.cpu().float() - Pref.float()).abs() <= step).all()
    err = (out.cpu().float() - ref.float()).abs().max() / ref.float().abs().max()
    assert float(err) <= (0.13 if qo is not None or fmt == E5 else 2e-2), f"{case}: {float(err)}"
    if case == "plain":
        assert abs(float(amax_s.cpu()) - float(ref_as)) <= 2.0 ** -7 * float(ref_as)


def test_fp8_sdpa_fwd_measurement_pass_and_checks(dev):
    gen = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(2, 2, 40, 32, generator=gen).bfloat16().to(dev) for _ in range(3))
    out, P, dm, amax_s = torch.ops.hpu.fp8_sdpa_fwd(q, k, v, None, 0.0, 0.2, True, "None", *NONE6, True, None, "left")
    w = torch.softmax((q.float() @ k.float().transpose(-2, -1) * 0.2).masked_fill(~torch.ones(40, 40, dtype=torch.bool, device=dev).tril(), float("-inf")), -1)
    assert P.dtype == torch.bfloat16 and torch.allclose(P.float(), w, atol=1e-2)
    assert torch.allclose(out.float(), w @ v.float(), atol=3e-2) and abs(float(amax_s) - float(w.max())) < 1e-3
    with pytest.raises(RuntimeError, match="dropout is not implemented"):
        torch.ops.hpu.fp8_sdpa_fwd(q, k, v, None, 0.1, 0.2, True, "None", *NONE6, False, None, "left")
