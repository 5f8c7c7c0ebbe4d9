"""GPU parity of hpu::sum_fp8 and hpu::softmax_fp8 against the oracle (the cases of the reference's
any_mode/test_hpu_sum_fp8.py and any_mode/test_hpu_fp8_ops_any_mode.py:991-1084, then the shapes that
reach every kernel variant)."""
import ctypes

import pytest
import torch

from helpers import E4, E5

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


# ----------------------------------------------------------------------------- sum_fp8

@pytest.mark.parametrize("dim", [0, 1, 2, (0, 1), None])
@pytest.mark.parametrize("keep_dim", [True, False])
@pytest.mark.parametrize("dtype", [E5, E4])
@pytest.mark.parametrize("out_dtype", [None, torch.float])
def test_sum_fp8(oracle, dev, dim, keep_dim, dtype, out_dtype):
    """test_hpu_sum_fp8.py:28-47, atol = rtol = 0."""
    x = (torch.randn((10, 20, 30)) * 10.0).to(dtype)
    got = ops.sum_fp8(x.to(dev), dim, keep_dim, out_dtype)
    want = oracle.torch_sum_fp8(x, dim, keep_dim, out_dtype)
    assert got.dtype == (out_dtype or dtype) and got.shape == want.shape
    assert torch.equal(got.cpu().float(), want.float())


@pytest.mark.parametrize("shape,dim", [
    ((64, 4096), [1]),            # rows, 16-byte vectors, one slice
    ((3, 1 << 20), [1]),          # rows split into slices, partial sums
    ((1 << 22,), None),           # everything into one value
    ((5, 1000), [1]),             # rows that do not start 16-byte aligned
    ((8, 1000, 256), [1]),        # columns, 16 per thread
    ((2, 5000, 20), [1]),         # columns, 4 per thread, split
    ((3, 700, 30), [1]),          # columns, 1 per thread
    ((70000, 3, 8), [1]),         # more outer positions than one grid dimension holds
    ((6, 7, 8, 9), [0, 2]),       # dimensions that are not adjacent
    ((6, 7, 8, 9), [1, 2]),       # adjacent, in the middle
    ((4, 0, 5), [1]),             # empty reduction: zeros
    ((0, 5), [1]),                # empty output
    ((), None),                   # 0-dim
])
@pytest.mark.parametrize("dtype", [E4, E5])
def test_sum_fp8_every_kernel_exact(oracle, dev, shape, dim, dtype):
    """Small-integer values: every fp32 partial sum is exact, so the result is the same in any order."""
    g = torch.Generator().manual_seed(11)
    x = torch.randint(-8, 9, shape, generator=g).float().to(dtype)
    for out_dtype in (torch.float, torch.bfloat16, None):
        got = ops.sum_fp8(x.to(dev), dim, False, out_dtype)
        want = oracle.torch_sum_fp8(x, dim, False, out_dtype)
        assert got.shape == want.shape and got.dtype == want.dtype
        assert torch.equal(got.cpu().float(), want.float()), (shape, dim, out_dtype)


def test_sum_fp8_general_values_and_repeatability(oracle, dev):
    x = (torch.randn(7, 100000) * 30).to(E5)
    a = ops.sum_fp8(x.to(dev), [1], False, torch.float)
    b = ops.sum_fp8(x.to(dev), [1], False, torch.float)
    assert torch.equal(a, b)                       # fixed summation order
    want = oracle.torch_sum_fp8(x, [1], False, torch.float)
    scale = x.float().abs().sum(1)
    assert ((a.cpu() - want).abs() <= 1e-6 * scale).all()
    with pytest.raises(RuntimeError, match="sum_fp8 input must be float8"):
        ops.sum_fp8(torch.zeros(4, device=dev), None, False, None)
    with pytest.raises(RuntimeError, match="appears multiple times"):
        ops.sum_fp8(x.to(dev), [1, -1], False, None)


def test_sum_fp8_meta():
    x = torch.empty(10, 20, 30, dtype=E4, device="meta")
    assert ops.sum_fp8(x, [0, 1], True, None).shape == (1, 1, 30) and ops.sum_fp8(x, [0, 1], True, None).dtype == E4
    assert ops.sum_fp8(x, None, False, torch.float).shape == () and ops.sum_fp8(x, [2], False, torch.float).dtype == torch.float


# ------------------------------------------------------------------------- softmax_fp8

def close_enough(got, want):
    """Equal up to one step of the output format on a few elements (the device's exp and the CPU's differ in
    the last place, which now and then moves a value across a rounding boundary); the reference's own bar
    (test_hpu_fp8_ops_any_mode.py:1045) is atol 1e-2, rtol 0.1251 for every element."""
    g, w = got.float().cpu(), want.float()
    assert got.dtype == want.dtype and g.shape == w.shape
    step = 0.1251 if want.dtype == E4 else 2.0 ** -7
    assert torch.allclose(g, w, atol=2e-3 if want.dtype == E4 else 1e-6, rtol=step)
    assert (g != w).float().mean().item() < 0.02


@pytest.mark.parametrize("is_scale,input_dtype", [(True, torch.bfloat16), (True, E4), (False, torch.bfloat16)])
@pytest.mark.parametrize("is_inv_attn_heads", [True, False])
@pytest.mark.parametrize("fused_add_shape", [None, (5, 4, 4, 6), (5, 1, 1, 6)])
def test_softmax_fp8(oracle, dev, is_scale, input_dtype, is_inv_attn_heads, fused_add_shape):
    """test_hpu_fp8_ops_any_mode.py:991-1045."""
    x = (torch.rand((5, 4, 4, 6), dtype=torch.bfloat16) * 4.0).to(input_dtype)
    s_in, s_out = (torch.tensor(0.05), torch.tensor(2.5)) if is_scale else (None, None)
    inv = torch.tensor(0.1) if is_inv_attn_heads else None
    add = torch.rand(fused_add_shape, dtype=torch.bfloat16) if (fused_add_shape and is_scale) else None
    d = lambda t: None if t is None else t.to(dev)
    got = ops.softmax_fp8(x.to(dev), -1, d(s_in), d(s_out), d(inv), d(add))
    close_enough(got, oracle.torch_softmax_fp8(x, -1, s_in, s_out, inv, add))


@pytest.mark.parametrize("is_inv_attn_heads", ["tensor", "scalar", None])
@pytest.mark.parametrize("input_dtype", [torch.bfloat16, E4])
def test_softmax_fp8_scalar(oracle, dev, is_inv_attn_heads, input_dtype):
    """test_hpu_fp8_ops_any_mode.py:1051-1081; the scalar overloads give the tensor overload's bits."""
    x = (torch.rand((5, 4, 4, 6), dtype=torch.bfloat16) * 4.0).to(input_dtype)
    inv = {"tensor": torch.tensor(0.1, device=dev), "scalar": 0.1, None: None}[is_inv_attn_heads]
    got = ops.softmax_fp8(x.to(dev), -1, 0.05, 2.5, inv)
    close_enough(got, oracle.torch_softmax_fp8(x, -1, 0.05, 2.5, 0.1 if is_inv_attn_heads else None))
    same = ops.softmax_fp8(x.to(dev), -1, torch.tensor(0.05, device=dev), torch.tensor(2.5, device=dev),
                           None if inv is None else torch.tensor(0.1, device=dev))
    assert torch.equal(got.view(torch.uint8), same.view(torch.uint8))


@pytest.mark.parametrize("shape", [
    (5, 4, 16, 64),       # one wave per row, one vector per lane
    (3, 2, 7, 1000),      # two vectors per lane, ragged
    (2, 9, 2048),         # four
    (3, 5, 4096),         # eight
    (2, 3, 8192),         # four waves per row
    (5, 16384),           # four waves, eight vectors
    (3, 20000),           # longer than a workgroup holds: three passes
    (4, 7, 100),          # not a multiple of 8: three passes
    (1, 8),
])
@pytest.mark.parametrize("input_dtype,scaled", [(torch.bfloat16, True), (E4, True), (torch.bfloat16, False)])
def test_softmax_fp8_every_kernel(oracle, dev, shape, input_dtype, scaled):
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(shape, generator=g) * 3).bfloat16().to(input_dtype)
    s_in, s_out = (0.5, 200.0) if scaled else (None, None)
    add = None
    if scaled and len(shape) >= 3:
        add_shape = (shape[0],) + (1,) * (len(shape) - 2) + (shape[-1],)
        add = torch.randn(add_shape, generator=g).bfloat16()
    if scaled:
        got = ops.softmax_fp8(x.to(dev), -1, s_in, s_out, 0.7, None if add is None else add.to(dev))
        want = oracle.torch_softmax_fp8(x, -1, s_in, s_out, 0.7, add)
    else:
        got = ops.softmax_fp8(x.to(dev), -1)
        want = oracle.torch_softmax_fp8(x, -1)
    close_enough(got, want)


def test_softmax_fp8_other_dim_and_errors(oracle, dev):
    x = torch.randn(6, 40, 9).bfloat16()
    close_enough(ops.softmax_fp8(x.to(dev), 1), oracle.torch_softmax_fp8(x, 1))
    close_enough(ops.softmax_fp8(x.to(dev), 0, 1.0, 100.0, None), oracle.torch_softmax_fp8(x, 0, 1.0, 100.0))
    xd = x.to(dev)
    s = torch.tensor(1.0, device=dev)
    with pytest.raises(RuntimeError, match="must be of torch.bfloat16 or torch.float8_e4m3fn"):
        ops.softmax_fp8(xd.float(), -1)
    with pytest.raises(RuntimeError, match="Output and input scales must be both given or None"):
        ops.softmax_fp8(xd, -1, s, None)
    with pytest.raises(RuntimeError, match="then input scale must be given"):
        ops.softmax_fp8(xd.to(E4), -1)
    with pytest.raises(RuntimeError, match="FusedAdd available only for Float8 output"):
        ops.softmax_fp8(xd, -1, None, None, None, xd)
    with pytest.raises(RuntimeError, match="same rank"):
        ops.softmax_fp8(xd, -1, s, s, None, xd[0])
    with pytest.raises(RuntimeError, match="same first and last dim"):
        ops.softmax_fp8(xd, -1, s, s, None, xd[:3])
    with pytest.raises(RuntimeError, match="should be equal to 1 or the same"):
        ops.softmax_fp8(xd, -1, s, s, None, xd[:, :20])
    with pytest.raises(RuntimeError, match="must be of dtype: Float"):
        ops.softmax_fp8(xd, -1, s.bfloat16(), s)
    meta = torch.empty(2, 3, 8, dtype=torch.bfloat16, device="meta")
    assert ops.softmax_fp8(meta, -1).dtype == torch.bfloat16 and ops.softmax_fp8(meta, -1, 1.0, 1.0, None).dtype == E4


def test_reductions_c_abi(oracle, pkg, dev):
    lib = pkg.capi()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x = torch.randint(-8, 9, (3, 1 << 20)).float().to(E4)
    xd = x.to(dev)
    ws_bytes = lib.mi355q_sum_fp8_workspace_bytes(3, 1 << 20, 1)
    assert ws_bytes > 0 and lib.mi355q_sum_fp8_workspace_bytes(4096, 64, 1) == 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    out = torch.empty(3, device=dev)
    assert lib.mi355q_sum_fp8(xd.data_ptr(), pkg.E4M3FN, 3, 1 << 20, 1, out.data_ptr(), pkg.F32, ws.data_ptr(), ws_bytes, st) == 0
    assert torch.equal(out.cpu(), x.float().sum(1))
    # a split launch without its workspace is refused
    assert lib.mi355q_sum_fp8(xd.data_ptr(), pkg.E4M3FN, 3, 1 << 20, 1, out.data_ptr(), pkg.F32, None, 0, st) != 0
    r = torch.randn(12, 256).bfloat16()
    y = torch.empty(12, 256, dtype=E4, device=dev)
    assert lib.mi355q_softmax_fp8(r.to(dev).data_ptr(), pkg.BF16, 12, 256, None, 0.5, None, 100.0, None, 1.0, None, 0, None, None,
                                  y.data_ptr(), pkg.E4M3FN, st) == 0
    close_enough(y, oracle.torch_softmax_fp8(r, -1, 0.5, 100.0))
    assert lib.mi355q_softmax_fp8(r.to(dev).data_ptr(), pkg.F32, 12, 256, None, 0.5, None, 100.0, None, 1.0, None, 0, None, None,
                                  y.data_ptr(), pkg.E4M3FN, st) != 0
