"""ctypes front-end of the C oracle plus a pure-PyTorch twin.

TEST INFRASTRUCTURE ONLY: used by tests/, by __graft_entry__.smoke() as the
checker, and by bench.py to time the CPU baseline.  Never imported by the
product package.

Two independent statements of the same semantics live here:
  * ``c_*``     call oracle/mi355q_oracle.c (bit-level C, scalar loops);
  * ``torch_*`` are the "PyTorch CPU float8 emulation" formulas: what the
    reference's tests compute on the CPU to judge the device
    (tests/pytest_working/any_mode/test_hpu_fp8_ops_any_mode.py:85-87,
    any_mode/test_hpu_cast.py:35-55, any_mode/test_hpu_convert_from_int4.py:
    104-131,224-247).  They run multi-threaded and serve as the CPU baseline.
The tests check the two against each other and against the reference's
known answers.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmi355q_oracle.so")

F32, BF16, E4M3FN, E5M2 = 0, 1, 2, 3
SCALE_NONE, SCALE_HOST, SCALE_DEV, SCALE_MID, SCALE_FULL = 0, 1, 2, 3, 4

_DT = {torch.float32: F32, torch.bfloat16: BF16,
       torch.float8_e4m3fn: E4M3FN, torch.float8_e5m2: E5M2}
FP8_MAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}
ROW_SCALE_CAP = 3.3895313892515355e38   # 0x7f7f0000, the largest finite bf16


def build(force=False):
    """Compile the C oracle with gcc (seconds)."""
    src = os.path.join(_HERE, "mi355q_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libmi355q_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        L.ora_f32_to_e4m3fn.argtypes = [c.c_float]
        L.ora_f32_to_e4m3fn.restype = c.c_uint8
        L.ora_f32_to_e5m2.argtypes = [c.c_float]
        L.ora_f32_to_e5m2.restype = c.c_uint8
        L.ora_f32_to_bf16.argtypes = [c.c_float]
        L.ora_f32_to_bf16.restype = c.c_uint16
        L.ora_e4m3fn_to_f32.argtypes = [c.c_uint8]
        L.ora_e4m3fn_to_f32.restype = c.c_float
        L.ora_e5m2_to_f32.argtypes = [c.c_uint8]
        L.ora_e5m2_to_f32.restype = c.c_float
        L.ora_cast_to_fp8.argtypes = [c.c_void_p, c.c_int, c.c_void_p, c.c_int, c.c_void_p,
                                      c.c_float, c.c_int, c.c_int64, c.c_int64, c.c_int64,
                                      c.c_void_p]
        L.ora_cast_to_fp8.restype = None
        L.ora_amax.argtypes = [c.c_void_p, c.c_int, c.c_int64, c.c_int64, c.c_void_p]
        L.ora_amax.restype = None
        L.ora_cast_from_fp8.argtypes = [c.c_void_p, c.c_int, c.c_void_p, c.c_int, c.c_void_p,
                                        c.c_float, c.c_int, c.c_int64, c.c_int64, c.c_int64]
        L.ora_cast_from_fp8.restype = None
        L.ora_dequant_4bit.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_int,
                                       c.c_int, c.c_int64, c.c_int64, c.c_int64, c.c_void_p]
        L.ora_dequant_4bit.restype = None
        L.ora_fp8_gemm.argtypes = [c.c_void_p, c.c_int, c.c_int64, c.c_int64,
                                   c.c_void_p, c.c_int, c.c_int64, c.c_int64,
                                   c.c_int64, c.c_int64, c.c_int64,
                                   c.c_void_p, c.c_float, c.c_int,
                                   c.c_void_p, c.c_float, c.c_int,
                                   c.c_void_p, c.c_int, c.c_void_p, c.c_int, c.c_void_p]
        L.ora_fp8_gemm.restype = None
        _lib = L
    return _lib


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _scale_args(x_shape, scale, scale_shape):
    """Classify a scale the way the C ABI does.

    Returns (tensor_or_None, host_value, mode, mid, inner).  ``scale`` may be
    None, a python float, a list of floats or a tensor; ``scale_shape`` is the
    optional broadcast shape (hpu_ops/backend/fp8_ops.cpp:29-100).
    """
    if scale is None:
        return None, 1.0, SCALE_NONE, 1, 1
    if isinstance(scale, (int, float)):
        return None, float(scale), SCALE_HOST, 1, 1
    if isinstance(scale, (list, tuple)):
        scale = torch.tensor(scale, dtype=torch.float64).to(torch.float32)
    scale = scale.detach().to("cpu", torch.float32).contiguous()
    if scale.numel() == 1:
        return scale.reshape(1), 0.0, SCALE_DEV, 1, 1
    shape = list(scale_shape) if scale_shape is not None else list(scale.shape)
    n = 1
    for d in shape:
        n *= d
    if n != scale.numel():
        raise ValueError(
            f"Number of scale elements ({scale.numel()}) is not equal to number of "
            f"scale_shape elements ({n}).")
    full = scale.reshape(shape).expand(x_shape).contiguous().reshape(-1)
    return full, 0.0, SCALE_FULL, 1, 1


# ---------------------------------------------------------------- C oracle

def c_cast_to_fp8(x, scale, out_dtype, is_amax=False, scale_shape=None):
    """(fp8 tensor, amax) as hpu::cast_to_fp8_v2 defines them (RNE)."""
    x = x.detach().cpu().contiguous()
    st, host, mode, mid, inner = _scale_args(x.shape, scale, scale_shape)
    y = torch.empty(x.shape, dtype=torch.uint8)
    amax = torch.zeros((), dtype=torch.float32)
    lib().ora_cast_to_fp8(_ptr(x), _DT[x.dtype], _ptr(y), _DT[out_dtype], _ptr(st), host, mode,
                          x.numel(), mid, inner, _ptr(amax) if is_amax else None)
    return y.view(out_dtype), (amax if is_amax else torch.empty(0, dtype=torch.float32))


def c_amax(x, rowwise=False):
    x = x.detach().cpu().contiguous()
    rows = x.shape[0] if rowwise else 1
    cols = x.numel() // max(rows, 1)
    out = torch.zeros(rows, dtype=torch.float32)
    lib().ora_amax(_ptr(x), _DT[x.dtype], rows, cols, _ptr(out))
    return out if rowwise else out.reshape(())


def c_cast_from_fp8(x8, scale, out_dtype, scale_shape=None):
    x8 = x8.detach().cpu().contiguous()
    st, host, mode, mid, inner = _scale_args(x8.shape, scale, scale_shape)
    y = torch.empty(x8.shape, dtype=out_dtype)
    lib().ora_cast_from_fp8(_ptr(x8), _DT[x8.dtype], _ptr(y), _DT[out_dtype], _ptr(st), host,
                            mode, x8.numel(), mid, inner)
    return y


def c_dequant_4bit(packed, scale, zero_point, out_dtype, signed):
    """hpu::convert_from_int4 / convert_from_uint4 on CPU tensors."""
    packed = packed.detach().cpu().contiguous()
    pcols = packed.shape[-1]
    rows = packed.numel() // max(pcols, 1)
    scale = scale.detach().cpu().to(out_dtype).contiguous()
    srows = scale.numel() // (pcols * 8)
    group = rows // srows
    zp_kind = 0
    zp = None
    if zero_point is not None:
        zero_point = zero_point.detach().cpu().contiguous()
        if zero_point.dtype == torch.int32:
            zp_kind, zp = 2, zero_point
        else:
            zp_kind, zp = 1, zero_point.to(out_dtype).contiguous()
    out = torch.empty(list(packed.shape[:-1]) + [pcols * 8], dtype=out_dtype)
    lib().ora_dequant_4bit(_ptr(packed), _ptr(scale), _ptr(zp), zp_kind, int(signed),
                           _DT[out_dtype], rows, pcols, group, _ptr(out))
    return out


def _gemm_scale(s, M, N, shape=None):
    if s is None:
        return None, 1.0, 0
    if isinstance(s, (int, float)):
        return None, float(s), 1
    if isinstance(s, (list, tuple)):
        s = torch.tensor(s, dtype=torch.float64).to(torch.float32)
    s = s.detach().cpu().to(torch.float32).contiguous()
    if s.numel() == 1:
        return s.reshape(1), 0.0, 2
    shp = list(shape) if shape is not None else list(s.shape)
    while len(shp) > 2 and shp[0] == 1:
        shp = shp[1:]
    if len(shp) == 1:
        shp = [1] + shp
    if shp == [M, 1]:
        return s.reshape(-1), 0.0, 3
    if shp == [1, N]:
        return s.reshape(-1), 0.0, 4
    raise ValueError(f"unsupported gemm scale shape {shp} for output [{M},{N}]")


def c_fp8_gemm(A, trans_A, B, trans_B, out_dtype, A_scale_inv=None, B_scale_inv=None,
               bias=None, D=None, B_scale_shape=None):
    """One 2-D fp8 GEMM through the C oracle (small sizes only: scalar loops)."""
    A = A.detach().cpu()
    B = B.detach().cpu()
    a = A.t() if trans_A else A
    b = B.t() if trans_B else B
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    sa, sah, sam = _gemm_scale(A_scale_inv, M, N)
    sb, sbh, sbm = _gemm_scale(B_scale_inv, M, N, B_scale_shape)
    bias_mode = 0
    if bias is not None:
        bias = bias.detach().cpu().to(out_dtype).contiguous()
        bias_mode = 1 if bias.numel() == N and bias.dim() <= 1 or list(bias.shape) == [1, N] else 2
        if bias_mode == 2:
            bias = bias.expand(M, N).contiguous()
    if D is not None:
        D = D.detach().cpu().to(out_dtype).expand(M, N).contiguous()
    C = torch.empty(M, N, dtype=out_dtype)
    lib().ora_fp8_gemm(_ptr(a), _DT[A.dtype], a.stride(0), a.stride(1),
                       _ptr(b), _DT[B.dtype], b.stride(0), b.stride(1), M, N, K,
                       _ptr(sa), sah, sam, _ptr(sb), sbh, sbm,
                       _ptr(bias), bias_mode, _ptr(D), _DT[out_dtype], _ptr(C))
    return C


# ------------------------------------------------------------ PyTorch twin

def _as_tensor_scale(scale, scale_shape):
    if scale is None:
        return None
    if isinstance(scale, (int, float)):
        return torch.tensor(float(scale), dtype=torch.float32)
    if isinstance(scale, (list, tuple)):
        scale = torch.tensor(scale, dtype=torch.float64).to(torch.float32)
    scale = scale.detach().cpu().to(torch.float32)
    if scale_shape is not None and scale.numel() > 1:
        scale = scale.reshape(list(scale_shape))
    return scale


def torch_cast_to_fp8(x, scale, out_dtype, is_amax=False, scale_shape=None):
    """(x * scale.to(x.dtype)) clamped to the finite fp8 range, PyTorch CPU RNE cast."""
    x = x.detach().cpu()
    s = _as_tensor_scale(scale, scale_shape)
    p = x if s is None else x * s.to(x.dtype)
    mx = FP8_MAX[out_dtype]
    y = p.clamp(-mx, mx).to(out_dtype)
    amax = x.abs().max().float() if is_amax else torch.empty(0, dtype=torch.float32)
    return y, amax


def torch_cast_from_fp8(x8, scale, out_dtype, scale_shape=None):
    s = _as_tensor_scale(scale, scale_shape)
    v = x8.detach().cpu().to(out_dtype)
    return v if s is None else v * s.to(out_dtype)


def torch_unpack_nibbles(packed, signed):
    """int32 [..., P] -> int32 [..., 8P]; element 8p+i sits in bits [4i, 4i+4)."""
    shifts = torch.arange(0, 32, 4, dtype=torch.int32)
    q = (packed.detach().cpu().unsqueeze(-1) >> shifts) & 0xF
    if signed:
        q = torch.where(q > 7, q - 16, q)
    return q.reshape(*packed.shape[:-1], packed.shape[-1] * 8)


def torch_dequant_4bit(packed, scale, zero_point, out_dtype, signed):
    q = torch_unpack_nibbles(packed, signed)
    scale = scale.detach().cpu().to(out_dtype)
    cols = q.shape[-1]
    rows = q.numel() // cols
    srows = scale.numel() // cols
    group = rows // srows
    q2 = q.reshape(srows, group, cols)
    s2 = scale.reshape(srows, 1, cols)
    if zero_point is None:
        d = q2.to(out_dtype)
    elif zero_point.dtype == torch.int32:
        z = torch_unpack_nibbles(zero_point, signed).reshape(srows, 1, cols)
        d = (q2 - z).to(out_dtype)
    else:
        d = q2.to(out_dtype) - zero_point.detach().cpu().to(out_dtype).reshape(srows, 1, cols)
    return (d * s2).reshape(q.shape)


def torch_fp8_gemm(A, trans_A, B, trans_B, out_dtype, A_scale_inv=None, B_scale_inv=None,
                   bias=None, D=None, B_scale_shape=None):
    """fp32-accumulated GEMM of the dequantised operands, torch.matmul batching."""
    a = A.detach().cpu().float()
    b = B.detach().cpu().float()
    if trans_A and a.dim() > 1:
        a = a.transpose(-2, -1)
    if trans_B and b.dim() > 1:
        b = b.transpose(-2, -1)
    v = torch.matmul(a, b)
    sa = _as_tensor_scale(A_scale_inv, None)
    sb = _as_tensor_scale(B_scale_inv, B_scale_shape)
    if sa is not None:
        v = v * sa
    if sb is not None:
        v = v * sb
    if bias is not None:
        v = v + bias.detach().cpu().float()
    if D is not None:
        v = v + D.detach().cpu().float()
    return v.to(out_dtype)


def torch_w4a8_gemm(A8, packed, scale, zero_point, signed, out_dtype, A_scale_inv=None, bias=None):
    """mi355q::w4a8_gemm: fp8 activations [M, K] times 4-bit weights packed as convert_from_int4 /
    convert_from_uint4 take them (int32 [K, N / 8], nibble i of word p is column 8 p + i, test_hpu_convert_
    from_int4.py:41-71; group-wise scales [K / g, N] and packed zero-points [K / g, N / 8], :224-247, 434-470):
        C = out_dtype( (A8 @ W) * A_scale_inv + bias ),   W[k, n] = (q[k, n] - z[k / g, n]) * s[k / g, n].
    The reference has no fused op; this is hpu::convert_from_[u]int4 (int4_ops.cpp:40-56) followed by the GEMM
    of fp8_ops.cpp:403-496, with W kept exact: (q - z) is an integer of at most 5 bits and s has at most 24, so
    the product is exact in fp32 (in float64 here, rounded once), where the unfused route would round W to bf16.
    Accumulation in float64, so the result does not depend on the order of the sums."""
    q = torch_unpack_nibbles(packed, signed).to(torch.float64)
    K, N = q.shape
    s = scale.detach().cpu().to(torch.float64)
    groups = s.shape[0]
    g = K // groups
    if zero_point is not None:
        q = q - torch_unpack_nibbles(zero_point, signed).to(torch.float64).repeat_interleave(g, dim=0)
    w = q * s.repeat_interleave(g, dim=0)
    v = A8.detach().cpu().to(torch.float64) @ w
    if A_scale_inv is not None:
        v = v * _as_tensor_scale(A_scale_inv, None).to(torch.float64)
    if bias is not None:
        v = v + bias.detach().cpu().to(torch.float64)
    return v.to(torch.float32).to(out_dtype)


def torch_w4a16_gemm(A, packed, scale, zero_point, signed, out_dtype, bias=None):
    """mi355q::w4a16_gemm: bf16 activations [M, K] times the same 4-bit weights,
        C = out_dtype( A @ W + bias ),   W[k, n] = (q[k, n] - z[k / g, n]) * s[k / g, n],
    i.e. hpu::convert_from_[u]int4 (int4_ops.cpp:40-56; layout of test_hpu_convert_from_int4.py:398-476) followed by
    the matmul a bf16 model runs on its output, with W kept exact and the sums in float64 (the unfused route rounds W
    to bf16 first)."""
    assert A.dtype == torch.bfloat16
    return torch_w4a8_gemm(A, packed, scale, zero_point, signed, out_dtype, None, bias)


def split_rows_fp8x2(x):
    """mi355q_split_rows_fp8x2: rows of a bf16 matrix as two e4m3fn planes and 1 / s per row, with
    x s = hi + lo / 16: s is the largest power of two with max |x| s <= 448 (1 for a row of zeros),
    hi = e4m3fn(x s) rounded to nearest even, lo = e4m3fn((x s - hi) 16).  Returns (hi, lo, scale_inv)."""
    x = x.detach().cpu()
    assert x.dtype == torch.bfloat16 and x.dim() == 2
    xf = x.float()
    amax = xf.abs().amax(dim=1, keepdim=True)
    m, ea = torch.frexp(amax)                      # amax = m 2^ea, 0.5 <= m < 1
    e = torch.where(m * 2 <= 1.75, 8, 7) - (ea - 1)
    e = torch.where(amax > 0, e, torch.zeros_like(e)).clamp(-126, 126)
    s = torch.exp2(e.float())
    p = xf * s
    hi = p.clamp(-448, 448).to(torch.float8_e4m3fn)
    lo = ((p - hi.float()) * 16).clamp(-448, 448).to(torch.float8_e4m3fn)
    return hi, lo, torch.exp2(-e.float()).reshape(-1)


def c_silu_mul_bf16(gate, up):
    """bf16(bf16(silu(gate)) * up) with the oracle's spelled-out exp (ora_silu_mul_bf16)."""
    g = gate.detach().cpu().contiguous()
    u = up.detach().cpu().contiguous()
    assert g.dtype == torch.bfloat16 and u.dtype == torch.bfloat16 and g.shape == u.shape
    h = torch.empty_like(g)
    L = lib()
    L.ora_silu_mul_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    L.ora_silu_mul_bf16.restype = None
    L.ora_silu_mul_bf16(_ptr(g), _ptr(u), _ptr(h), g.numel())
    return h


def quantize_rows(x, out_dtype):
    """Dynamic per-row quantisation as mi355q::quantize_rows states it: (x8, 1 / scale) with
    scale = fp8_max / rowwise amax (fp32 division) and cast_to_fp8_v2's rounding."""
    x = x.detach().cpu()
    x2 = x.reshape(-1, x.shape[-1])
    amax = x2.abs().amax(dim=-1, keepdim=True).float()
    # tensor / tensor is an IEEE division; torch evaluates scalar / tensor as scalar * (1 / tensor)
    scale = torch.full_like(amax, FP8_MAX[out_dtype]) / amax
    # capped at the largest finite bf16 value: a row of zeros (amax 0, quotient inf) would otherwise turn
    # into NaN codes through 0 * inf; a NaN amax stays NaN (the comparison is false)
    scale = torch.where(scale > ROW_SCALE_CAP, torch.full_like(scale, ROW_SCALE_CAP), scale)
    y, _ = c_cast_to_fp8(x2, scale.reshape(-1), out_dtype, scale_shape=[x2.shape[0], 1])
    return y.reshape(x.shape), (torch.ones_like(scale) / scale).reshape(x.shape[:-1] + (1,))


def torch_scaled_mm(mat1, mat2, scale_a, scale_b, bias=None, scale_result=None, out_dtype=None):
    """aten::_scaled_mm as the reference's test states it (any_mode/test_hpu_scaled_mm.py:177):
    (mat1 @ mat2) * scale_a * scale_b * scale_result + bias, accumulated and scaled in fp32,
    one rounding to out_dtype (default: mat1's dtype, scaled_mm_gen.cpp:72-75); an fp8
    out_dtype saturates."""
    v = torch.matmul(mat1.detach().cpu().float(), mat2.detach().cpu().float())
    sa = scale_a.detach().cpu().float()
    if scale_result is not None:
        sa = sa * scale_result.detach().cpu().float().reshape(())
    v = v * sa * scale_b.detach().cpu().float()
    if bias is not None:
        v = v + bias.detach().cpu().float()
    out_dtype = out_dtype or mat1.dtype
    if out_dtype in FP8_MAX:
        mx = FP8_MAX[out_dtype]
        return v.clamp(-mx, mx).to(out_dtype)
    return v.to(out_dtype)


def torch_sum_fp8(x, dim=None, keepdim=False, out_dtype=None):
    """hpu::sum_fp8 as the reference's test states it (any_mode/test_hpu_sum_fp8.py:36-47): torch.sum of
    the fp8 values; here accumulated in float64, so that the result is the exactly rounded sum whatever
    the order (for inputs whose fp32 partial sums are all exact, as the test's are, any fp32 order gives
    the same).  An fp8 out_dtype (the default, the input's) is the saturating round-to-nearest cast of
    the sum: the reference compares that case with its own device result only -- parity unpinned."""
    out_dtype = out_dtype or x.dtype
    dims = list(range(x.dim())) if dim is None or (isinstance(dim, (list, tuple)) and len(dim) == 0) else dim
    v = torch.sum(x.detach().cpu().to(torch.float64), dims, keepdim) if x.dim() else x.detach().cpu().to(torch.float64)
    v = v.to(torch.float32)
    if out_dtype in FP8_MAX:
        mx = FP8_MAX[out_dtype]
        return v.clamp(-mx, mx).to(out_dtype)
    return v.to(out_dtype)


def torch_softmax_fp8(x, dim=-1, input_scale=None, output_scale=None, inv_attn_heads=None, fused_add=None):
    """hpu::softmax_fp8 (hpu_ops/backend/softmax_fp8_gen.cpp:73-158; semantics from
    any_mode/test_hpu_fp8_ops_any_mode.py:1030-1045): softmax((x * inv_attn_heads) * input_scale + fused_add),
    rounded to bf16; with scales the bf16 value times output_scale, cast to e4m3fn (saturating).  fp32
    arithmetic up to the rounding to bf16 (the test rounds every step to bf16 and allows rtol 0.1251,
    one e4m3 step; the device's internal precision is not stated) -- parity pinned to that tolerance only."""
    v = x.detach().cpu().float()
    if inv_attn_heads is not None:
        v = v * float(inv_attn_heads)
    if input_scale is not None:
        v = v * torch.tensor(float(input_scale), dtype=torch.float32)
        if fused_add is not None:
            v = v + fused_add.detach().cpu().float()
    p = torch.softmax(v, dim).to(torch.bfloat16)
    if input_scale is None:
        return p
    q = p.float() * torch.tensor(float(output_scale), dtype=torch.float32)
    return q.clamp(-448.0, 448.0).to(torch.float8_e4m3fn)


def pack_nibbles(q):
    """int tensor [..., 8P] with values in -8..15 -> packed int32 [..., P]."""
    q = q.detach().cpu().to(torch.int64) & 0xF
    q = q.reshape(*q.shape[:-1], q.shape[-1] // 8, 8)
    shifts = torch.arange(0, 32, 4, dtype=torch.int64)
    w = (q << shifts).sum(-1)
    w = torch.where(w >= 2 ** 31, w - 2 ** 32, w)
    return w.to(torch.int32)


def _sdpa_scale(s, default):
    if s is None:
        return default
    if isinstance(s, torch.Tensor):
        if s.numel() == 0:
            return default
        return float(s.detach().cpu().float().reshape(-1)[0])
    return float(s) if float(s) != 0.0 else default


def key_window(valid_seq_len, seq_padding_type, S, batch_rank):
    """bool [B, 1, ..., 1, S] (batch_rank + 2 dimensions): the keys entry b of the outermost batch dimension may
    attend to, valid_seq_len[b] of them, the last ones for left padding and the first ones for right padding."""
    n = torch.as_tensor(valid_seq_len).detach().cpu().to(torch.int64).reshape(-1, 1).clamp(0, S)
    j = torch.arange(S).reshape(1, S)
    pad = seq_padding_type.lower()
    assert pad in ("left", "right")
    w = (j >= S - n) if pad == "left" else (j < n)
    if batch_rank == 0:
        return w.reshape(1, S)
    return w.reshape(w.shape[0], *([1] * batch_rank), S)


def torch_fp8_sdpa_unfused(q, k, v, attn_mask=None, scale=None, is_causal=False, d_scale_q=None, d_scale_k=None, d_scale_v=None,
                           q_scale_s=None, q_scale_o=None, d_scale_s=None, valid_seq_len=None, seq_padding_type="left"):
    """hpu::fp8_sdpa_fwd without dropout, fp8 q / k / v: the forward that keeps the probability matrix
    (Fp8SDPAFwd::AddNode, hpu_ops/backend/sdpa_gen.cpp:340-437; outputs :103-150).  The kernel behind the
    reference's node is closed; this restates the op as the three steps its outputs imply, each step one of
    the family's own ops: scores = bf16((q d_scale_q)(k d_scale_k)^T) (fp8_gemm_v2, fp32 accumulation),
    P = fp8(bf16(softmax(scores scale + mask)) q_scale_s) (softmax_fp8), out = bf16((P d_scale_s)(v d_scale_v))
    (fp8_gemm_v2), or fp8(out q_scale_o).  Masked scores take the most negative finite bf16-representable value
    -3e38 instead of -inf, so a row with every key masked attends to all keys evenly.  Returns (out, P, amax_s),
    amax_s the largest bf16 probability."""
    f8 = q.dtype
    dq, dk, dv = _sdpa_scale(d_scale_q, 1.0), _sdpa_scale(d_scale_k, 1.0), _sdpa_scale(d_scale_v, 1.0)
    qs = _sdpa_scale(q_scale_s, 1.0)
    ds = _sdpa_scale(d_scale_s, float(torch.tensor(qs, dtype=torch.float32).reciprocal()))
    qo = _sdpa_scale(q_scale_o, None)
    L, S = q.shape[-2], k.shape[-2]
    if scale is None:
        scale = 1.0 / (q.shape[-1] ** 0.5)
    f32 = lambda x: torch.tensor(float(x), dtype=torch.float32)
    sc = (torch.matmul(q.detach().cpu().float(), k.detach().cpu().float().transpose(-2, -1)) * f32(dq) * f32(dk)).to(torch.bfloat16)
    x = sc.float() * f32(scale)
    masked = torch.tensor(-3.0e38).to(torch.bfloat16).float()
    if attn_mask is not None:
        m_ = attn_mask.detach().cpu()
        x = x + (torch.where(m_, 0.0, masked) if m_.dtype == torch.bool else m_.to(torch.bfloat16).float().clamp_min(masked))
    else:
        keep = None
        if is_causal:
            keep = torch.ones(L, S, dtype=torch.bool).tril(0)
        if valid_seq_len is not None:
            w = key_window(valid_seq_len, seq_padding_type, S, sc.dim() - 2)
            keep = w if keep is None else keep & w
        if keep is not None:
            x = x + torch.where(keep, 0.0, masked)
    pb = torch.softmax(x, -1).to(torch.bfloat16)
    amax_s = pb.float().max() if pb.numel() else torch.tensor(0.0)
    mx8 = FP8_MAX[f8]
    P = (pb.float() * f32(qs)).clamp(-mx8, mx8).to(f8)
    out = (torch.matmul(P.float(), v.detach().cpu().float()) * f32(ds) * f32(dv))
    if qo is not None:
        res = (out.to(torch.bfloat16).float() * f32(qo)).clamp(-mx8, mx8).to(f8)
    else:
        res = out.to(torch.bfloat16)
    return res, P, amax_s


def torch_fp8_sdpa(q, k, v, attn_mask=None, scale=None, is_causal=False, d_scale_q=None, d_scale_k=None,
                   d_scale_v=None, q_scale_s=None, q_scale_o=None, d_scale_s=None, block=64, quantize_p=True,
                   key_streams=None, valid_seq_len=None, seq_padding_type="left"):
    """hpu::fp8_sdpa_recomp_fwd in inference (requires_backward False, dropout 0), fp8 q/k/v.

    The arithmetic of that op lives in a closed device-kernel library (GUID "sdpa_recomp_fwd",
    hpu_ops/backend/sdpa_gen.cpp:806-1000 only wires tensors, flags and output types), so this is a
    restatement of the published algorithm it names -- attention with an online ("recompute") softmax,
    FlashAttention-2 forward -- with the fp8 scales placed where the op's argument names put them
    (python_packages/habana_frameworks/torch/hpex/kernels/Fp8FusedSDPA.py:92-160) and checked the way
    the reference's test checks the device (tests/pytest_working/any_mode/FusedSDPA/test_hpu_sdpa_fp8.py:
    292-320 vanilla attention, :1046-1052 tolerances):

        S   = (q * d_scale_q) (k * d_scale_k)^T * scale  [+ float mask | -inf where a bool mask is False
                                                           | -inf above the diagonal, row i sees j <= i]
        per block of `block` key columns, with m the running row maximum:
        p   = exp(S - m)                      in [0, 1]
        P8  = fp8(p * q_scale_s)              the format of v; saturating round-to-nearest-even
        l   = l * exp(m_old - m) + sum(p),    O = O * exp(m_old - m) + P8 v
        out = O * d_scale_s * d_scale_v / l   d_scale_s defaults to 1 / q_scale_s
        out -> bf16, or fp8(out * q_scale_o) when q_scale_o is given.

    float64 throughout except the stated roundings.  block=None takes the whole row at once (m is the
    final row maximum); quantize_p=False leaves p unrounded.  Rows with every key masked by -inf give 0.
    key_streams=(splits, blocks_per_split, waves): the keys are walked as the few-queries kernel walks
    them -- `splits` ranges of `blocks_per_split` blocks, inside a range `waves` streams that take every
    waves-th block, each stream with its own running maximum (which is what p is rounded against), the
    streams' (m, l, O) merged exactly at the end.  Without rounding the result does not depend on it.
    valid_seq_len (one integer per entry of the outermost batch dimension; flags VALID_SEQ_LEN_PRESENT,
    SEQ_PADDING_LEFT / RIGHT, sdpa_gen.cpp:849-851; the wrapper allows it only with is_causal and no mask,
    Fp8FusedSDPA.py:123-126): entry b attends to its last valid_seq_len[b] keys when the padding is on the
    left and to its first when it is on the right, on top of the triangular mask.  (Nothing in the
    reference's tree runs the op with it; this is the reading of the argument names and of the wrapper's
    contract, pinned in tests/test_oracle_sdpa.py as plain attention on the valid slice.)
    Returns (out, amax_s, amax_o): amax_s = max softmax probability = max_i 1 / l_i, amax_o = max |out|
    before q_scale_o.  Batch dimensions broadcast as torch.matmul's do."""
    f8 = v.dtype
    mx8 = FP8_MAX[f8]
    dq, dk, dv = _sdpa_scale(d_scale_q, 1.0), _sdpa_scale(d_scale_k, 1.0), _sdpa_scale(d_scale_v, 1.0)
    qs = _sdpa_scale(q_scale_s, 1.0)
    ds = _sdpa_scale(d_scale_s, 1.0 / qs)
    qo = _sdpa_scale(q_scale_o, None)
    Q = q.detach().cpu().double() * dq
    K = k.detach().cpu().double() * dk
    V = v.detach().cpu().double()
    L, S = Q.shape[-2], K.shape[-2]
    if scale is None:
        scale = 1.0 / (Q.shape[-1] ** 0.5)
    s = torch.matmul(Q, K.transpose(-2, -1)) * float(scale)
    if attn_mask is not None:
        m_ = attn_mask.detach().cpu()
        if m_.dtype == torch.bool:
            s = s.masked_fill(~m_, float("-inf"))
        else:
            s = s + m_.double()
    if is_causal:
        keep = torch.ones(L, S, dtype=torch.bool).tril(0)
        s = s.masked_fill(~keep, float("-inf"))
    bshape = torch.broadcast_shapes(s.shape[:-2], V.shape[:-2])
    s = s.expand(*bshape, L, S)
    if valid_seq_len is not None:
        s = s.masked_fill(~key_window(valid_seq_len, seq_padding_type, S, len(bshape)), float("-inf"))
    V = V.expand(*bshape, S, V.shape[-1])
    step = S if block is None else block

    def walk(starts):
        m = torch.full((*bshape, L, 1), float("-inf"), dtype=torch.float64)
        l = torch.zeros((*bshape, L, 1), dtype=torch.float64)
        O = torch.zeros((*bshape, L, V.shape[-1]), dtype=torch.float64)
        for j0 in starts:
            sb = s[..., j0:j0 + step]
            m_new = torch.maximum(m, sb.max(dim=-1, keepdim=True).values)
            m_use = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)
            alpha = torch.exp(m - m_use)
            p = torch.exp(sb - m_use)
            if quantize_p:
                p8 = (p * qs).float().clamp(-mx8, mx8).to(f8).double()
            else:
                p8 = p * qs
            l = l * alpha + p.sum(dim=-1, keepdim=True)
            O = O * alpha + torch.matmul(p8, V[..., j0:j0 + step, :])
            m = m_new
        return m, l, O

    if key_streams is None:
        m, l, O = walk(range(0, S, step))
    else:
        splits, per_split, waves = key_streams
        nblk = -(-S // step)
        parts = []
        for sp in range(splits):
            b0, b1 = sp * per_split, min((sp + 1) * per_split, nblk)
            for w in range(waves):
                parts.append(walk([b * step for b in range(b0 + w, b1, waves)]))
        m = torch.stack([p_[0] for p_ in parts]).max(dim=0).values
        m_use = torch.where(torch.isinf(m), torch.zeros_like(m), m)
        l = sum(p_[1] * torch.exp(p_[0] - m_use) for p_ in parts)
        O = sum(p_[2] * torch.exp(p_[0] - m_use) for p_ in parts)
    live = l > 0
    out = torch.where(live, O * (ds * dv) / torch.where(live, l, torch.ones_like(l)), torch.zeros_like(O))
    out32 = out.float()
    amax_s = (1.0 / l[live]).max().float() if live.any() else torch.tensor(0.0)
    amax_o = out32.abs().max()
    if qo is not None:
        res = (out32 * torch.tensor(qo, dtype=torch.float32)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    else:
        res = out32.to(torch.bfloat16)
    return res, amax_s, amax_o
