"""Pins of the oracle's sum_fp8 and softmax_fp8 (CPU only): the formulas of the reference's tests,
closed forms, invariants."""
import pytest
import torch

from helpers import E4, E5


@pytest.mark.parametrize("dim", [0, 1, 2, (0, 1), None])
@pytest.mark.parametrize("keep_dim", [True, False])
@pytest.mark.parametrize("dtype", [E5, E4])
def test_sum_matches_the_reference_tests_formula(oracle, dim, keep_dim, dtype):
    """any_mode/test_hpu_sum_fp8.py:36-47 with out_dtype=float: torch.sum of the values as fp32, no tolerance."""
    x = (torch.randn((10, 20, 30)) * 10.0).to(dtype)
    got = oracle.torch_sum_fp8(x, dim, keep_dim, torch.float)
    dims = dim if dim is not None else [0, 1, 2]
    want = torch.sum(x.to(torch.float), dims, keep_dim)
    assert got.dtype == torch.float and torch.equal(got, want)


def test_sum_closed_forms(oracle):
    x = torch.full((7, 300, 5), 1.5).to(E4)
    assert torch.equal(oracle.torch_sum_fp8(x, [1], False, torch.float), torch.full((7, 5), 450.0))
    # the fp8 result saturates: 7 * 300 * 5 * 1.5 = 15750 > 448
    assert oracle.torch_sum_fp8(x).float().item() == 448.0 and oracle.torch_sum_fp8(x).dtype == E4
    assert oracle.torch_sum_fp8(x.view(torch.uint8).view(E4)[:1, :2, :1]).float().item() == 3.0
    # cancellation that an fp32 running sum in the wrong order would lose
    y = torch.tensor([57344.0, 2.0 ** -16, -57344.0]).to(E5)
    assert oracle.torch_sum_fp8(y, None, False, torch.float).item() == 2.0 ** -16
    assert oracle.torch_sum_fp8(torch.zeros(0, 4).to(E4), [0], False, torch.float).tolist() == [0.0] * 4


@pytest.mark.parametrize("is_scale,input_dtype", [(True, torch.bfloat16), (True, E4), (False, torch.bfloat16)])
@pytest.mark.parametrize("is_inv_attn_heads", [True, False])
@pytest.mark.parametrize("fused_add_shape", [None, (5, 4, 4, 6), (5, 1, 1, 6)])
def test_softmax_within_the_reference_tests_tolerance(oracle, is_scale, input_dtype, is_inv_attn_heads, fused_add_shape):
    """any_mode/test_hpu_fp8_ops_any_mode.py:998-1045: the test's own arithmetic (every step rounded to
    bf16) against the oracle (fp32 up to the rounding of the softmax), atol 1e-2, rtol 0.1251."""
    x = torch.rand((5, 4, 4, 6), dtype=torch.bfloat16) * 4.0
    xin = x.to(input_dtype)
    s_in, s_out = (torch.tensor(0.05), torch.tensor(2.5)) if is_scale else (None, None)
    inv = torch.tensor(0.1) if is_inv_attn_heads else None
    add = torch.rand(fused_add_shape, dtype=torch.bfloat16) if (fused_add_shape and is_scale) else None
    got = oracle.torch_softmax_fp8(xin, -1, s_in, s_out, inv, add)
    ref = x
    if inv is not None:
        ref = ref * inv
    if is_scale:
        ref = ref * s_in
        if add is not None:
            ref = ref + add
    ref = torch.softmax(ref, -1).to(torch.bfloat16)
    if is_scale:
        ref = (ref * s_out).to(E4)
        assert got.dtype == E4
    else:
        assert got.dtype == torch.bfloat16
    assert torch.allclose(got.float(), ref.float(), atol=1e-2, rtol=0.1251)


def test_softmax_closed_forms(oracle):
    # equal inputs: 1 / L exactly representable for L a power of two
    x = torch.full((3, 64), 2.0, dtype=torch.bfloat16)
    assert torch.equal(oracle.torch_softmax_fp8(x).float(), torch.full((3, 64), 1.0 / 64))
    # with scales: bf16(1/64) * 128 = 2.0 in e4m3
    y = oracle.torch_softmax_fp8(x, -1, 0.5, 128.0)
    assert y.dtype == E4 and torch.equal(y.float(), torch.full((3, 64), 2.0))
    # one dominant entry -> 1, the rest underflow to 0; output_scale saturates at 448
    z = torch.zeros(2, 16, dtype=torch.bfloat16)
    z[:, 3] = 200.0
    out = oracle.torch_softmax_fp8(z, -1, 1.0, 1000.0).float()
    assert out[:, 3].tolist() == [448.0, 448.0] and out.sum().item() == 896.0
    # a shift of the row (here through fused_add) leaves the result alone
    r = torch.randn(4, 32).bfloat16()
    a = oracle.torch_softmax_fp8(r, -1, 1.0, 64.0)
    b = oracle.torch_softmax_fp8(r, -1, 1.0, 64.0, None, torch.full((4, 32), 8.0).bfloat16())
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    # rows sum to one to bf16 precision
    assert torch.allclose(oracle.torch_softmax_fp8(r).float().sum(-1), torch.ones(4), atol=2e-2)
