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


# ------------------------------------------------------------------ valid_seq_len / seq_padding_type

@pytest.mark.parametrize("pad", ["left", "right"])
@pytest.mark.parametrize("gqa", [False, True])
def test_a_key_window_is_plain_causal_attention_on_the_valid_slice(oracle, pad, gqa):
    """Entry b attends to valid_seq_len[b] keys (the last ones for left padding, the first ones for right
    padding) under the triangular mask: its valid rows equal causal attention on the slice that holds only
    the valid positions.  Exactly so with the whole row taken at once (block=None), where the rounding of the
    probabilities does not depend on where the blocks fall."""
    gen = torch.Generator().manual_seed(11)
    S = 90
    if gqa:   # the wrapper's grouped-query view [B, G, H / G, L, D] against [B, G, 1, S, D]
        q = torch.randn(3, 2, 2, S, 16, generator=gen).to(E4)
        k = torch.randn(3, 2, 1, S, 16, generator=gen).to(E4)
        v = torch.randn(3, 2, 1, S, 24, generator=gen).to(E4)
    else:
        q = torch.randn(3, 2, S, 16, generator=gen).to(E4)
        k = torch.randn(3, 2, S, 16, generator=gen).to(E4)
        v = torch.randn(3, 2, S, 24, generator=gen).to(E4)
    valid = torch.tensor([90, 37, 1], dtype=torch.int32)
    out, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, q_scale_s=128.0, d_scale_s=1 / 128.0, block=None,
                                      valid_seq_len=valid, seq_padding_type=pad)
    for b, n in enumerate(valid.tolist()):
        sl = slice(S - n, S) if pad == "left" else slice(0, n)
        part, _, _ = oracle.torch_fp8_sdpa(q[b][..., sl, :], k[b][..., sl, :], v[b][..., sl, :], is_causal=True, q_scale_s=128.0,
                                           d_scale_s=1 / 128.0, block=None)
        assert torch.equal(out[b][..., sl, :].view(torch.int16), part.view(torch.int16)), (pad, b)
        # and against float64 attention with the rounding of the probabilities switched off
        exact, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, quantize_p=False, valid_seq_len=valid, seq_padding_type=pad)
        ref, _ = plain(q[b][..., sl, :].float(), k[b][..., sl, :].float(), v[b][..., sl, :].float(), causal=True)
        assert torch.equal(exact[b][..., sl, :].view(torch.int16), ref.float().to(torch.bfloat16).expand_as(exact[b][..., sl, :]).contiguous().view(torch.int16))


def test_rows_in_front_of_a_left_padded_window_are_zero_and_counts_are_clamped(oracle):
    gen = torch.Generator().manual_seed(12)
    q, k, v = (torch.randn(2, 1, 40, 16, generator=gen).to(E4) for _ in range(3))
    out, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, valid_seq_len=torch.tensor([10, 1000]), seq_padding_type="left")
    assert torch.count_nonzero(out[0, :, :30].float()) == 0 and torch.count_nonzero(out[0, :, 30:].float()) > 0
    full, _, _ = oracle.torch_fp8_sdpa(q[1:], k[1:], v[1:], is_causal=True)
    assert torch.equal(out[1:].view(torch.int16), full.view(torch.int16))          # a count beyond kv_len means all keys
    none, _, _ = oracle.torch_fp8_sdpa(q, k, v, is_causal=True, valid_seq_len=torch.tensor([0, 0]), seq_padding_type="right")
    assert torch.count_nonzero(none.float()) == 0


# ------------------------------------------------------------------ the forward that keeps P (fp8_sdpa_fwd)

@pytest.mark.parametrize("causal", [False, True])
def test_unfused_forward_is_plain_attention_within_its_roundings(oracle, causal):
    """out and P of oracle.torch_fp8_sdpa_unfused against float64 attention: P / q_scale_s is the softmax to
    one e4m3 step (2^-4 relative, plus bf16's 2^-9), rows of P sum to q_scale_s within that, and out is within
    the bound those steps allow (max |v| 2^-4 plus the bf16 steps of scores and output)."""
    gen = torch.Generator().manual_seed(21)
    q = torch.randn(2, 3, 48, 32, generator=gen).to(E4)
    k = torch.randn(2, 3, 80, 32, generator=gen).to(E4)
    v = torch.randn(2, 3, 80, 16, generator=gen).to(E4)
    out, P, amax_s = oracle.torch_fp8_sdpa_unfused(q, k, v, is_causal=causal, d_scale_q=0.5, d_scale_k=2.0, d_scale_v=0.25,
                                                   q_scale_s=128.0, d_scale_s=1 / 128.0)
    ref, w = plain(q.float() * 0.5, k.float() * 2.0, v.float() * 0.25, causal=causal)
    assert P.dtype == E4 and P.shape == (2, 3, 48, 80) and out.dtype == torch.bfloat16
    p = P.double() / 128.0
    # bf16 scores move a probability by up to exp(2^-9 |s|) - 1; the test's scores stay below 16 in magnitude
    assert ((p - w).abs() <= w * 2.0 ** -3 + 1e-3).all()
    assert ((p.sum(-1) - 1).abs() <= 0.08).all()
    assert ((out.double() - ref).abs() <= 0.13 * v.float().abs().max() * 0.25 + 1e-2).all()
    assert abs(float(amax_s) - float(w.max())) <= 0.07 * float(w.max()) + 1e-3
    if causal:
        assert torch.count_nonzero(P.float().triu(1)) == 0        # masked entries are exactly zero


def test_unfused_forward_is_composed_of_the_family_ops(oracle):
    """The same numbers out of the oracles of fp8_gemm_v2, softmax_fp8 and fp8_gemm_v2 chained by hand."""
    gen = torch.Generator().manual_seed(22)
    q = torch.randn(2, 40, 32, generator=gen).to(E4)
    k = torch.randn(2, 56, 32, generator=gen).to(E4)
    v = torch.randn(2, 56, 16, generator=gen).to(E4)
    out, P, _ = oracle.torch_fp8_sdpa_unfused(q, k, v, scale=0.2, d_scale_q=0.5, d_scale_k=2.0, d_scale_v=0.25, q_scale_s=64.0)
    for b in range(2):
        sc = oracle.torch_fp8_gemm(q[b], False, k[b], True, torch.bfloat16, 0.5, 2.0)
        Pb = oracle.torch_softmax_fp8(sc, -1, 0.2, 64.0)
        ob = oracle.torch_fp8_gemm(Pb, False, v[b], False, torch.bfloat16, 1.0 / 64.0, 0.25)
        assert torch.equal(P[b].view(torch.uint8), Pb.view(torch.uint8))
        assert torch.equal(out[b].view(torch.int16), ob.view(torch.int16))
