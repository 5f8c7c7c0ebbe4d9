"""Shared comparison helpers for the parity tests."""
import torch

E4 = torch.float8_e4m3fn
E5 = torch.float8_e5m2
FP8_DTYPES = [E5, E4]


def fp8_nan_mask(codes, dtype):
    """Which uint8 codes are NaN in the given fp8 format."""
    c = codes.to(torch.int32) & 0x7F
    if dtype == E4:
        return c == 0x7F
    return c > 0x7C


def assert_fp8_equal(a, b, dtype, what=""):
    """Bit equality of fp8 tensors; every NaN encoding counts as the same NaN.

    A NaN has no value to be exact about: e4m3fn has two encodings (sign), e5m2
    six.  The hardware conversion emits one canonical NaN, the oracle keeps the
    sign; both are NaN and compare equal here.
    """
    a = a.detach().cpu().contiguous().view(torch.uint8)
    b = b.detach().cpu().contiguous().view(torch.uint8)
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    na, nb = fp8_nan_mask(a, dtype), fp8_nan_mask(b, dtype)
    assert torch.equal(na, nb), f"{what}: NaN positions differ"
    ok = (a == b) | na
    if not bool(ok.all()):
        idx = (~ok).nonzero()[:5].tolist()
        raise AssertionError(f"{what}: {int((~ok).sum())} of {a.numel()} codes differ, first at {idx}: "
                             f"{[hex(int(a[tuple(i)])) for i in idx]} vs {[hex(int(b[tuple(i)])) for i in idx]}")


def assert_bits_equal(a, b, what=""):
    """Bit equality of bf16 / fp32 tensors; NaNs compare equal to NaNs."""
    a = a.detach().cpu().contiguous()
    b = b.detach().cpu().contiguous()
    assert a.dtype == b.dtype and a.shape == b.shape, f"{what}: {a.dtype}{tuple(a.shape)} vs {b.dtype}{tuple(b.shape)}"
    it = torch.int16 if a.dtype == torch.bfloat16 else torch.int32
    na, nb = torch.isnan(a), torch.isnan(b)
    assert torch.equal(na, nb), f"{what}: NaN positions differ"
    ok = (a.view(it) == b.view(it)) | na
    if not bool(ok.all()):
        idx = (~ok).nonzero()[:5].tolist()
        raise AssertionError(f"{what}: {int((~ok).sum())} of {a.numel()} values differ, first at {idx}: "
                             f"{[float(a[tuple(i)]) for i in idx]} vs {[float(b[tuple(i)]) for i in idx]}")


def gemm_errors(out, ref):
    """(max|out-ref| / max|ref|, allclose(atol=1e-3*max|ref|, rtol=1e-2))."""
    out = out.detach().cpu().float()
    ref = ref.detach().cpu().float()
    scale = ref.abs().max().clamp_min(1e-30)
    rel = ((out - ref).abs().max() / scale).item()
    ok = torch.allclose(out, ref, atol=1e-3 * scale.item(), rtol=1e-2)
    return rel, ok


def c1_input(rows=4096, cols=4096, seed=0xC001A1):
    """bf16 N(0,1)*3 with 0.1 % of the values set to +-1e4 (seeded)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) * 3
    n = x.numel()
    k = -(-n // 1000)
    pos = torch.randperm(n, generator=g)[:k]
    sign = torch.randint(0, 2, (k,), generator=g).float() * 2 - 1
    x.view(-1)[pos] = sign * 1e4
    return x.bfloat16()
