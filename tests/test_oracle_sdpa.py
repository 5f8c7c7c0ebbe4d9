"""Pins of the CPU oracle of hpu::fp8_sdpa_recomp_fwd (oracle.torch_fp8_sdpa).

The arithmetic of that op is not in the reference tree (a closed kernel library runs it), so the oracle
restates the published online-softmax algorithm; what fixes it here: PyTorch's own attention on the
dequantised inputs (with the fp8 rounding of the probabilities switched off the two must agree to
float64 accuracy, whatever the block size), closed forms (uniform scores, a one-hot row), the bound the
fp8 rounding puts on the difference, and the reference test's own case, scales and tolerances
(tests/pytest_working/any_mode/FusedSDPA/test_hpu_sdpa_fp8.py:137-180, 454-476, 1046-1052).
"""
import math

import pytest
import torch

from helpers import E4, E5


def plain(q, k, v, mask=None, causal=False, scale=None):
    """The reference test's vanilla attention (test_hpu_sdpa_fp8.py:292-320) in float64."""
    q, k, v = q.double(), k.double(), v.double()
    s = q @ k.transpose(-2, -1) * (1 / math.sqrt(q.shape[-1]) if scale is None else scale)
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf")) if mask.dtype == torch.bool else s + mask.double()
    if causal:
        s = s.masked_fill(~torch.ones(s.shape[-2:], dtype=torch.bool).tril(), float("-inf"))
    w = torch.softmax(s, -1)
    return w @ v, w


@pytest.mark.parametrize("block", [None, 64, 16])
@pytest.mark.parametrize("causal", [False, True])
def test_without_rounding_it_is_plain_attention(oracle, block, causal):
    gen = torch.Generator().manual_seed(1)
    q = torch.randn(2, 3, 50, 24, generator=gen).to(E4)
    k = torch.randn(2, 3, 150, 24, generator=gen).to(E4)
    v = torch.randn(2, 3, 150, 40, generator=gen).to(E4)
    ref, w = plain(q.float() * 0.5, k.float() * 2.0, v.float() * 0.25, causal=causal, scale=0.3)
    out, amax_s, amax_o = oracle.torch_fp8_sdpa(q, k, v, scale=0.3, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0,
                                                d_scale_v=0.25, q_scale_s=128.0, d_scale_s=1 / 128.0, block=block,
                                                quantize_p=False)
    # the only rounding left is the final one to bf16
    assert torch.equal(out, ref.float().to(torch.bfloat16))
    assert abs(float(amax_s) - float(w.max())) < 1e-6
    assert abs(float(amax_o) - float(ref.abs().max())) < 1e-6


def test_the_walk_over_the_keys_does_not_matter_without_rounding(oracle):
    """key_streams (several streams of blocks, each with its own running maximum, merged at the end) is the same
    function as one pass when the probabilities are not rounded; with rounding it moves the result by no more than
    the rounding does."""
    gen = torch.Generator().manual_seed(11)
    q = torch.randn(2, 3, 64, generator=gen).to(E4)
    k = torch.randn(2, 1000, 64, generator=gen).to(E4)
    v = torch.randn(2, 1000, 64, generator=gen).to(E4)
    ref, w = plain(q.float(), k.float(), v.float())
    for walk in ((1, 16, 4), (3, 6, 4), (16, 1, 4), (2, 8, 1)):
        out, amax_s, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=128.0, quantize_p=False, key_streams=walk)
        assert torch.equal(out, ref.float().to(torch.bfloat16))
        assert abs(float(amax_s) - float(w.max())) < 1e-6
        rounded, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=128.0, key_streams=walk)
        assert (rounded.float() - ref.float()).abs().max() <= 2.0 ** -4 * v.float().abs().max()


@pytest.mark.parametrize("kind", ["bool", "float"])
def test_masks_and_broadcast_batches(oracle, kind):
    gen = torch.Generator().manual_seed(2)
    q = torch.randn(2, 2, 3, 20, 16, generator=gen).to(E4)          # grouped-query layout
    k = torch.randn(2, 2, 1, 70, 16, generator=gen).to(E4)
    v = torch.randn(2, 2, 1, 70, 16, generator=gen).to(E4)
    keep = torch.rand(2, 1, 1, 20, 70, generator=gen) > 0.4
    keep[..., 0] = True
    mask = keep if kind == "bool" else torch.where(keep, 0.0, -1e9) + 0.25
    ref, _ = plain(q.float(), k.float(), v.float(), mask=mask)
    out, _, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=mask, block=64, quantize_p=False)
    assert out.shape == (2, 2, 3, 20, 16)
    assert torch.equal(out, ref.float().to(torch.bfloat16))


def test_causal_mask_is_aligned_top_left(oracle):
    """Row i sees keys j <= i also when there are more keys than queries (test_hpu_sdpa_fp8.py:311-315)."""
    gen = torch.Generator().manual_seed(3)
    q = torch.randn(1, 4, 8, generator=gen).to(E4)
    k = torch.randn(1, 9, 8, generator=gen).to(E4)
    v = torch.randn(1, 9, 8, generator=gen).to(E4)
    out, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, quantize_p=False)
    assert torch.equal(out[0, 0], v[0, 0].to(torch.bfloat16))       # the first query sees the first key only
    only4, _, _ = oracle.torch_fp8_sdpa(q, k[:, :4], v[:, :4], is_causal=True, quantize_p=False)
    assert torch.equal(out, only4)


def test_uniform_scores_give_the_mean_exactly(oracle):
    """q = 0: every probability is 1 before normalisation, 128 = q_scale_s is an fp8 number, so nothing is
    rounded and the result is the mean of v times d_scale_v, for any block size."""
    gen = torch.Generator().manual_seed(4)
    q = torch.zeros(2, 5, 32).to(E4)
    k = torch.randn(2, 256, 32, generator=gen).to(E4)
    v = torch.randn(2, 256, 48, generator=gen).to(E4)
    for block in (None, 64):
        out, amax_s, _ = oracle.torch_fp8_sdpa(q, k, v, d_scale_v=0.5, q_scale_s=128.0, d_scale_s=1 / 128.0, block=block)
        mean = (v.double().mean(dim=-2, keepdim=True) * 0.5).expand(2, 5, 48)
        assert torch.equal(out, mean.float().to(torch.bfloat16))
        assert float(amax_s) == 1 / 256


def test_one_dominant_key_selects_its_row(oracle):
    q = torch.zeros(1, 3, 16)
    q[:, :, 0] = 16.0
    k = torch.zeros(1, 100, 16)
    k[0, 17, 0] = 16.0                                                # score 256 * scale on key 17, 0 elsewhere
    gen = torch.Generator().manual_seed(5)
    v = torch.randn(1, 100, 16, generator=gen).to(E4)
    out, amax_s, _ = oracle.torch_fp8_sdpa(q.to(E4), k.to(E4), v, scale=1.0, q_scale_s=128.0)
    assert torch.equal(out[0, 1], v[0, 17].to(torch.bfloat16))
    assert float(amax_s) == 1.0


def test_rounding_of_the_probabilities_is_bounded(oracle):
    """fp8(p q_scale_s) is within 2^-4 relative of p q_scale_s (e4m3, normal range), so the output moves by at
    most 2^-4 of sum p |v| / sum p <= 2^-4 max|v|; far less on average."""
    gen = torch.Generator().manual_seed(6)
    q = torch.randn(2, 60, 64, generator=gen).to(E4)
    k = torch.randn(2, 300, 64, generator=gen).to(E4)
    v = torch.randn(2, 300, 64, generator=gen).to(E4)
    exact, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=128.0, quantize_p=False)
    for block in (None, 64):
        rounded, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=128.0, block=block)
        d = (rounded.float() - exact.float()).abs()
        assert d.max() <= 2.0 ** -4 * v.float().abs().max()
        assert 0 < d.mean() < 0.01


def test_output_scale_and_formats(oracle):
    gen = torch.Generator().manual_seed(7)
    q = torch.randn(1, 2, 30, 16, generator=gen).to(E5)
    k = torch.randn(1, 2, 40, 16, generator=gen).to(E5)
    v = torch.randn(1, 2, 40, 16, generator=gen).to(E5)
    o16, _, amax_o = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=64.0)
    o8, _, amax_o8 = oracle.torch_fp8_sdpa(q, k, v, q_scale_s=64.0, q_scale_o=32.0)
    assert o16.dtype == torch.bfloat16 and o8.dtype == E4 and float(amax_o) == float(amax_o8)
    assert torch.allclose(o8.float() / 32.0, o16.float(), rtol=2.0 ** -3, atol=2.0 ** -9 / 32)
    huge, _, _ = oracle.torch_fp8_sdpa(q, k, v, q_scale_o=1e6)
    assert huge.float().abs().max() == 448.0                         # saturates, no NaN


def test_rows_with_every_key_masked(oracle):
    gen = torch.Generator().manual_seed(8)
    q = torch.randn(1, 6, 16, generator=gen).to(E4)
    k = torch.randn(1, 80, 16, generator=gen).to(E4)
    v = torch.randn(1, 80, 16, generator=gen).to(E4)
    keep = torch.ones(1, 6, 80, dtype=torch.bool)
    keep[0, 2] = False
    keep[0, 4, :70] = False            # the first block of row 4 is empty, the second is not
    out, amax_s, _ = oracle.torch_fp8_sdpa(q, k, v, attn_mask=keep)
    assert (out[0, 2] == 0).all() and not torch.isnan(out.float()).any()
    ref, w = plain(q.float(), k.float(), v.float(), mask=keep)
    assert torch.allclose(out[0, 4].float(), ref[0, 4].float(), atol=0.05)
    assert abs(float(amax_s) - float(torch.nan_to_num(w, 0.0).max())) < 1e-6


@pytest.mark.parametrize("causal,use_mask,out8", [(True, False, True), (True, False, False), (False, True, True), (False, True, False)])
def test_reference_test_case_within_its_tolerances(oracle, causal, use_mask, out8):
    """The reference's tc_list2 / tc_list4 (batch 3, 4 heads, 16 queries, 32 keys, head dimension 8), its seed,
    its power-of-two scales (get_scale_values on Gaudi3: 2^floor(log2(0.9 * 240 / amax)), q_scale_s fixed to
    128) and its tolerances for an fp8 run: atol 0.4, rtol 1e-3 against bf16 attention."""
    torch.manual_seed(1234567)
    q, k, v = torch.randn(3, 4, 16, 8).bfloat16(), torch.randn(3, 4, 32, 8).bfloat16(), torch.randn(3, 4, 32, 8).bfloat16()
    mask = None
    if use_mask:
        m = torch.randint(0, 2, (32,)).float()
        mask = m.masked_fill(m == 0, -1e9).masked_fill(m == 1, 0.0).bfloat16().expand(3, 1, 1, 32)
    ref, _ = plain(q.float(), k.float(), v.float(), mask=mask, causal=causal)

    def pow2_scale(t):
        return 2.0 ** int(math.log2(240 * 0.9 / t.abs().max().item()))
    sq, sk, sv = pow2_scale(q), pow2_scale(k), pow2_scale(v)
    q8 = (q.float() * sq).clamp(-448, 448).to(E4)
    k8 = (k.float() * sk).clamp(-448, 448).to(E4)
    v8 = (v.float() * sv).clamp(-448, 448).to(E4)
    so = pow2_scale(ref) if out8 else None
    out, _, _ = oracle.torch_fp8_sdpa(q8, k8, v8, attn_mask=mask, is_causal=causal, d_scale_q=1 / sq, d_scale_k=1 / sk,
                                      d_scale_v=1 / sv, q_scale_s=128.0, q_scale_o=so, d_scale_s=1 / 128.0)
    got = out.float() / so if out8 else out.float()
    assert torch.allclose(got, ref.float(), atol=0.4, rtol=1e-3)
    assert (got - ref.float()).abs().max() < 0.2        # in fact far inside the reference's bound
