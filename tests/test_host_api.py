"""Host layer without a GPU: the C-ABI library loads and exports what
include/mi355q.h declares, the hpu:: schemas are the reference's, and shapes,
dtypes and error strings follow the reference (exercised on meta tensors)."""
import os
import re

import pytest
import torch

from helpers import E4, E5

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# habana_eager/eager_custom_op_register.cpp:2146-2171
REFERENCE_SCHEMAS = {
    ("cast_from_fp8", ""): "hpu::cast_from_fp8(Tensor input, Tensor? scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor",
    ("cast_from_fp8", "scalar"): "hpu::cast_from_fp8.scalar(Tensor input, float scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor",
    ("cast_from_fp8", "scalar_list"): "hpu::cast_from_fp8.scalar_list(Tensor input, float[] scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor",
    ("cast_to_fp8_v2", ""): "hpu::cast_to_fp8_v2(Tensor input, Tensor? scale=None, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)",
    ("cast_to_fp8_v2", "scalar"): "hpu::cast_to_fp8_v2.scalar(Tensor input, float scale, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)",
    ("cast_to_fp8_v2", "scalar_list"): "hpu::cast_to_fp8_v2.scalar_list(Tensor input, float[] scale, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)",
    # the deprecated out-variants, eager_custom_op_register.cpp:2152, 2165
    ("cast_to_fp8", ""): "hpu::cast_to_fp8(Tensor input, Tensor? scale, bool stochastic_rounding, Tensor(a!) out, Tensor(b!) amax) -> (Tensor(a!), Tensor(b!))",
    ("fp8_gemm", ""): "hpu::fp8_gemm(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor D, ScalarType out_dtype, Tensor? A_scale_inv, Tensor? B_scale_inv, Tensor? bias, bool accumulate, Tensor(a!) out) -> Tensor(a!)",
    # scripts/hpu_op.yaml:7365-7366
    ("cast_to_fp8_hybrid", ""): "hpu::cast_to_fp8_hybrid(Tensor input, Tensor? scale_152=None, Tensor? scale_143=None, bool stochastic_rounding=False, bool is_amax=False) -> (Tensor, Tensor, Tensor)",
    # scripts/hpu_op.yaml:7399-7418, 7448-7453
    ("softmax_fp8", ""): "hpu::softmax_fp8(Tensor input, int dim, Tensor? input_scale=None, Tensor? output_scale=None, Tensor? inv_attn_heads=None, Tensor? fused_add=None) -> Tensor",
    ("softmax_fp8", "Scalar_scales"): "hpu::softmax_fp8.Scalar_scales(Tensor input, int dim, float input_scale, float output_scale, Tensor? inv_attn_heads=None, Tensor? fused_add=None) -> Tensor",
    ("softmax_fp8", "Scalar"): "hpu::softmax_fp8.Scalar(Tensor input, int dim, float input_scale, float output_scale, float inv_attn_heads, Tensor? fused_add=None) -> Tensor",
    ("sum_fp8", ""): "hpu::sum_fp8(Tensor self, int[1]? dim=None, bool keepdim=False, ScalarType? out_dtype=None) -> Tensor",
    ("convert_from_int4", ""): "hpu::convert_from_int4(Tensor input, Tensor scale, Tensor? zero_point, ScalarType out_dtype) -> Tensor",
    ("convert_from_uint4", ""): "hpu::convert_from_uint4(Tensor input, Tensor scale, Tensor? zero_point, ScalarType out_dtype) -> Tensor",
    ("fp8_gemm_v2", ""): "hpu::fp8_gemm_v2(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, Tensor? A_scale_inv=None, Tensor? B_scale_inv=None, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None) -> Tensor",
    ("fp8_gemm_v2", "scalar"): "hpu::fp8_gemm_v2.scalar(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, float A_scale_inv, float B_scale_inv, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None) -> Tensor",
    ("fp8_gemm_v2", "scalar_list"): "hpu::fp8_gemm_v2.scalar_list(Tensor input, float[] A_scale_inv, float[] B_scale_inv)".replace(
        "Tensor input, float[] A_scale_inv, float[] B_scale_inv",
        "Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, float[] A_scale_inv, float[] B_scale_inv, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None") + " -> Tensor",
}


def meta(shape, dtype):
    return torch.empty(shape, device="meta", dtype=dtype)


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "mi355q.h")).read()
    declared = set(re.findall(r"^(?:int|size_t|const char\*)\s+(mi355q_[a-z0-9_]+)\s*\(", header, flags=re.M))
    assert declared == set(pkg.EXPORTED_SYMBOLS)
    lib = pkg.capi()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.mi355q_abi_version() == 7
    assert lib.mi355q_status_string(0) == b"ok"
    assert b"invalid" in lib.mi355q_status_string(1)


def test_no_compute_entry_point_accepts_bad_enums(pkg):
    """Argument validation happens before any launch, so it runs without a GPU."""
    lib = pkg.capi()
    assert lib.mi355q_cast_to_fp8(None, 0, None, 7, None, 1.0, 0, 1, 1, 1, None, None) == 1
    assert lib.mi355q_cast_to_fp8(None, 0, None, pkg.E4M3FN, None, 1.0, pkg.SCALE_DEV, 1, 1, 1, None, None) == 1
    assert lib.mi355q_cast_from_fp8(None, pkg.E4M3FN, None, pkg.E5M2, None, 1.0, 0, 1, 1, 1, None) == 1
    assert lib.mi355q_dequant_4bit(None, None, None, 0, 0, pkg.BF16, 4, 4, 0, None, None) == 1
    assert lib.mi355q_fp8_gemm(None, 0, 0, 0, None, 2, 0, 0, None, 1, 0, 1, 1, 1, None, 1.0, 0, None, 1.0, 0,
                               None, 0, 0, None, 0, 1, 0, 0, 0, 0, 0, None) == 1
    # empty problems succeed without touching the device
    assert lib.mi355q_cast_from_fp8(None, pkg.E4M3FN, None, pkg.BF16, None, 1.0, 0, 0, 1, 1, None) == 0
    assert lib.mi355q_fp8_gemm(None, 2, 0, 0, None, 2, 0, 0, None, 1, 0, 0, 16, 16, None, 1.0, 0, None, 1.0, 0,
                               None, 0, 0, None, 0, 1, 0, 0, 0, 0, 0, None) == 0


def test_variant_names(pkg):
    lib = pkg.capi()
    assert b"256x256" in lib.mi355q_fp8_gemm_variant(0, 4096, 0, 14336, 8192, 14336, 4096)
    assert lib.mi355q_fp8_gemm_variant(0, 24, 0, 36, 12, 36, 24) == b"simple"
    # where m or n is the contiguous dimension only the pitch has to be a multiple of 16
    assert b"simple" not in lib.mi355q_fp8_gemm_variant(0, 1024, 0, 1008, 515, 1001, 1024)
    assert b"simple" not in lib.mi355q_fp8_gemm_variant(1, 528, 0, 1008, 515, 1001, 1030)   # K contiguous in neither operand
    assert lib.mi355q_fp8_gemm_variant(0, 1040, 0, 1008, 515, 1001, 1030) == b"simple"       # K contiguous and ragged


@pytest.mark.parametrize("key", sorted(REFERENCE_SCHEMAS))
def test_schemas_are_the_references(pkg, key):
    name, overload = key
    packet = getattr(torch.ops.hpu, name)
    op = getattr(packet, overload or "default")
    assert str(op._schema) == REFERENCE_SCHEMAS[key]


def test_no_cpu_implementation(pkg):
    with pytest.raises((RuntimeError, NotImplementedError), match="CPU"):
        torch.ops.hpu.cast_to_fp8_v2(torch.zeros(4), None, False, False, E4)
    with pytest.raises((RuntimeError, NotImplementedError), match="CPU"):
        torch.ops.hpu.convert_from_int4(torch.zeros(4, dtype=torch.int32), torch.ones(32), None, torch.bfloat16)


@pytest.mark.parametrize("is_amax", [True, False])
@pytest.mark.parametrize("dtype", [E4, E5])
def test_cast_to_fp8_v2_meta(pkg, is_amax, dtype):
    """dynamo/_custom_op_meta_registrations.py:56-76 and fp8_ops.cpp:170-178."""
    x = meta((16, 24, 8), torch.bfloat16)
    for scale in (None, meta((), torch.float32), 1.3, [1.0] * 8):
        args = [x, scale, False, is_amax, dtype] + ([[1, 8]] if isinstance(scale, list) else [])
        out, amax = torch.ops.hpu.cast_to_fp8_v2(*args)
        assert out.shape == x.shape and out.dtype == dtype
        assert amax.dtype == torch.float32
        assert tuple(amax.shape) == (() if is_amax else (0,))


def test_cast_to_fp8_v2_errors(pkg):
    """Strings of fp8_ops.cpp:46-52,203-215 (test_hpu_fp8_ops_any_mode.py:179-202)."""
    for src in (E4, E5):
        for dst in (E4, E5):
            x = meta((16, 24, 8), src)
            with pytest.raises(RuntimeError, match="CastToFp8V2 must have no amax for float8."):
                torch.ops.hpu.cast_to_fp8_v2(x, None, False, True, dst)
            if src != dst:
                msg = ("CastToFp8V2 input and output must have the same dtype for float8, but are "
                       f"{str(src).replace('torch.f', 'F')} and {str(dst).replace('torch.f', 'F')}")
                with pytest.raises(RuntimeError, match=re.escape(msg)):
                    torch.ops.hpu.cast_to_fp8_v2(x, 1.0, False, False, dst)
            else:
                out, _ = torch.ops.hpu.cast_to_fp8_v2(x, None, False, False, dst)
                assert out.dtype == dst
    with pytest.raises(RuntimeError, match=re.escape(
            "CastToFp8V2 input dtype must be one of [float, bfloat16, float8_e5m2, float8_e4m3fn].")):
        torch.ops.hpu.cast_to_fp8_v2(meta((4,), torch.float16), None, False, False, E4)
    with pytest.raises(RuntimeError, match=re.escape(
            "Number of scale elements (8) is not equal to number of scale_shape elements (24).")):
        torch.ops.hpu.cast_to_fp8_v2(meta((16, 24, 8), torch.bfloat16), meta((8,), torch.float32), False, False, E4, [24, 1])
    with pytest.raises(RuntimeError, match="dtype must be given"):
        torch.ops.hpu.cast_to_fp8_v2(meta((4,), torch.float32))
    # stochastic rounding changes values, not shapes (GetCastParams, fp8_ops.cpp:105-119)
    y, a = torch.ops.hpu.cast_to_fp8_v2(meta((4,), torch.float32), None, True, False, E4)
    assert y.shape == (4,) and y.dtype == E4 and a.shape == (0,)
    with pytest.raises(RuntimeError, match="stochastic rounding needs a float or bfloat16 input"):
        torch.ops.hpu.cast_to_fp8_v2(meta((4,), E4), None, True, False, E4)


def test_cast_from_fp8_meta_and_errors(pkg):
    x = meta((8, 16), E4)
    for dt in (torch.float32, torch.bfloat16):
        for scale in (None, meta((1,), torch.float32)):
            out = torch.ops.hpu.cast_from_fp8(x, scale, dt)
            assert out.shape == x.shape and out.dtype == dt
        assert torch.ops.hpu.cast_from_fp8(x, 0.5, dt).dtype == dt
        assert torch.ops.hpu.cast_from_fp8(x, [0.5] * 16, dt, [1, 16]).dtype == dt
    with pytest.raises(RuntimeError, match="CastFromFp8 output dtype must be equal to float or bfloat16."):
        torch.ops.hpu.cast_from_fp8(x, None, torch.float16)
    with pytest.raises(RuntimeError, match="Number of scale elements"):
        torch.ops.hpu.cast_from_fp8(x, [0.5] * 16, torch.float32, [1, 8])


GEMM_SHAPES = [
    ((24, 12), (24, 36), True, False),
    ((2, 1, 4, 2), (1, 3, 4, 8), True, False),
    ((2, 1, 4, 2), (4, 8), True, False),
    ((4, 2), (3, 4, 8), True, False),
    ((10,), (10,), False, False),
    ((2, 10), (10,), False, False),
    ((10,), (10, 2), False, False),
    ((4, 8, 16), (16,), False, False),
    ((8,), (2, 4, 8, 16), False, False),
    ((5, 7, 3), (5, 3, 9), False, False),
    ((5, 7, 3), (5, 9, 3), False, True),
]


@pytest.mark.parametrize("sa, sb, ta, tb", GEMM_SHAPES)
def test_fp8_gemm_v2_shape_rule_is_torch_matmul(pkg, sa, sb, ta, tb):
    """batched_matmul_output_shape.cpp:33-85; tests :504-514,534-596."""
    A, B = meta(sa, E4), meta(sb, E4)
    a = torch.empty(sa).transpose(-2, -1) if ta else torch.empty(sa)
    b = torch.empty(sb).transpose(-2, -1) if tb else torch.empty(sb)
    expect = torch.matmul(a, b).shape
    for dt in (torch.bfloat16, torch.float32):
        out = torch.ops.hpu.fp8_gemm_v2(A, ta, B, tb, None, dt)
        assert out.shape == expect and out.dtype == dt
    assert torch.ops.hpu.fp8_gemm_v2(A, ta, B, tb, None, torch.bfloat16, 1.0, 2.0).shape == expect
    assert torch.ops.hpu.fp8_gemm_v2(A, ta, B, tb, None, torch.bfloat16, [1.0], [2.0]).shape == expect


def test_fp8_gemm_v2_errors(pkg):
    A, B = meta((12, 24), E4), meta((25, 36), E4)
    with pytest.raises(RuntimeError, match=re.escape(
            "Common dimension sizes of matmul inputs should be the same. Got 24 and 25")):
        torch.ops.hpu.fp8_gemm_v2(A, False, B, False, None, torch.bfloat16)
    with pytest.raises(RuntimeError, match=re.escape(
            "Batch dimension 0 of matmul inputs should be the same or at least one of them should be equal to 1. Got 2 and 3")):
        torch.ops.hpu.fp8_gemm_v2(meta((2, 4, 8), E4), False, meta((3, 8, 4), E4), False, None, torch.bfloat16)
    B = meta((24, 36), E4)
    with pytest.raises(RuntimeError, match=re.escape(
            "Accumulation tensor must be provided at index 4 for Fp8GemmV2, when accumulate is true")):
        torch.ops.hpu.fp8_gemm_v2(A, False, B, False, None, torch.bfloat16, None, None, None, True)
    with pytest.raises(RuntimeError, match="Number of scale elements"):
        torch.ops.hpu.fp8_gemm_v2(A, False, B, False, None, torch.bfloat16, [1.0], [1.0] * 36, None, False, [1, 12])
    with pytest.raises(RuntimeError, match="output dtype"):
        torch.ops.hpu.fp8_gemm_v2(A, False, B, False, None, torch.float16)
    with pytest.raises(RuntimeError, match="operands must be float8"):
        torch.ops.hpu.fp8_gemm_v2(meta((12, 24), torch.bfloat16), False, B, False, None, torch.bfloat16)


@pytest.mark.parametrize("variant", ["int4", "uint4"])
def test_convert_from_int4_meta(pkg, variant):
    """int4_ops.cpp:22-30: last dim times 8, dtype = out_dtype."""
    fn = getattr(torch.ops.hpu, "convert_from_" + variant)
    for shape in ((10,), (4, 6, 4), (64, 8)):
        real = list(shape)
        real[-1] *= 8
        for dt in (torch.float32, torch.bfloat16):
            out = fn(meta(shape, torch.int32), meta(real, dt), None, dt)
            assert list(out.shape) == real and out.dtype == dt
    with pytest.raises(RuntimeError, match="must be int32"):
        fn(meta((4, 4), torch.int64), meta((4, 32), torch.float32), None, torch.float32)
    with pytest.raises(RuntimeError, match="output dtype must be float or bfloat16"):
        fn(meta((4, 4), torch.int32), meta((4, 32), torch.float32), None, E4)


def test_ops_trace_under_fake_tensors(pkg):
    """The Meta kernels are what lets torch.compile / export trace the ops."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(32, 64, dtype=torch.bfloat16, device="cuda")
        w = torch.empty(64, 48, dtype=E4, device="cuda")
        x8, amax = torch.ops.hpu.cast_to_fp8_v2(x, None, False, True, E4)
        y = torch.ops.hpu.fp8_gemm_v2(x8, False, w, False, None, torch.bfloat16, 0.5, 0.25)
        assert x8.dtype == E4 and amax.shape == () and y.shape == (32, 48) and y.device.type == "cuda"


def test_quantize_rows_meta(pkg):
    """mi355q::quantize_rows: fp8 tensor shaped like the input, fp32 inverse scales [..., 1]."""
    y, s = torch.ops.mi355q.quantize_rows(meta((3, 16, 64), torch.bfloat16), E4)
    assert y.shape == (3, 16, 64) and y.dtype == E4
    assert s.shape == (3, 16, 1) and s.dtype == torch.float32
    with pytest.raises(RuntimeError, match="float or bfloat16"):
        torch.ops.mi355q.quantize_rows(meta((4, 8), torch.float16), E4)
    with pytest.raises(RuntimeError, match="float8"):
        torch.ops.mi355q.quantize_rows(meta((4, 8), torch.float32), torch.bfloat16)
    lib = pkg.capi()
    assert lib.mi355q_quantize_rows(None, pkg.BF16, 4, 8, None, pkg.E4M3FN, 448.0, None, None, None) == 1
    assert lib.mi355q_quantize_rows(None, pkg.BF16, 0, 8, None, pkg.E4M3FN, 448.0, None, None, None) == 0


@pytest.mark.parametrize("is_amax", [True, False])
def test_cast_to_fp8_hybrid_meta(pkg, is_amax):
    """CastToFp8HybridMeta, hpu_ops/backend/cast_to_fp8_hybrid_gen.cpp:39-61."""
    y5, y4, amax = torch.ops.hpu.cast_to_fp8_hybrid(meta((16, 24, 8), torch.bfloat16), None, meta((), torch.float32), True, is_amax)
    assert y5.shape == (16, 24, 8) and y5.dtype == E5 and y4.shape == (16, 24, 8) and y4.dtype == E4
    assert amax.dtype == torch.float32 and amax.shape == (() if is_amax else (0,))
    with pytest.raises(RuntimeError, match="CastToFp8Hybrid input must be of float or bfloat16 dtype."):
        torch.ops.hpu.cast_to_fp8_hybrid(meta((4,), torch.float16))


def test_scaled_mm_meta_shapes_and_errors(pkg):
    """mi355q::scaled_mm carries aten::_scaled_mm's signature, the reference's checks
    (scaled_mm_gen.cpp:78-107) and its default out_dtype (:72-75)."""
    import re
    schema = str(torch.ops.mi355q.scaled_mm.default._schema)
    aten = str(torch.ops.aten._scaled_mm.default._schema)
    assert re.sub(r"^mi355q::scaled_mm", "", schema) == re.sub(r"^aten::_scaled_mm", "", aten)
    a = torch.empty(12, 16, dtype=torch.float8_e5m2, device="meta")
    b = torch.empty(16, 24, dtype=torch.float8_e4m3fn, device="meta")
    s = torch.empty((), device="meta")
    out = torch.ops.mi355q.scaled_mm(a, b, s, s)
    assert out.shape == (12, 24) and out.dtype == torch.float8_e5m2
    assert torch.ops.mi355q.scaled_mm(a, b, s, s, None, None, torch.bfloat16).dtype == torch.bfloat16
    with pytest.raises(RuntimeError, match="mat2 must be a matrix"):
        torch.ops.mi355q.scaled_mm(a, b[0], s, s)
    with pytest.raises(RuntimeError, match=r"mat1 and mat2 shapes cannot be multiplied \(12x16 and 24x16\)"):
        torch.ops.mi355q.scaled_mm(a, b.t(), s, s)
    with pytest.raises(RuntimeError, match="Expected mat2 to be Float8_e5m2 or Float8_e4m3fn matrix got"):
        torch.ops.mi355q.scaled_mm(a, b.to(torch.bfloat16), s, s)
    with pytest.raises(RuntimeError, match="scale_a must hold one value or have shape"):
        torch.ops.mi355q.scaled_mm(a, b, torch.empty(3, device="meta"), s)


def test_sum_fp8_meta_and_errors(pkg):
    """SumFp8Meta, hpu_ops/backend/fp8_ops_gen.cpp:20-33: reduction shape, out_dtype or the input's."""
    x = meta((10, 20, 30), E4)
    for dim, keep, shape in ((None, False, ()), ([0], False, (20, 30)), ([1], True, (10, 1, 30)), ([0, 2], False, (20,)),
                             ([-1], False, (10, 20)), ([0, 1, 2], True, (1, 1, 1))):
        out = torch.ops.hpu.sum_fp8(x, dim, keep, None)
        assert tuple(out.shape) == shape and out.dtype == E4
        assert torch.ops.hpu.sum_fp8(x, dim, keep, torch.float).dtype == torch.float
        assert tuple(out.shape) == tuple(torch.sum(torch.empty(10, 20, 30, device="meta"), dim if dim is not None else [0, 1, 2], keep).shape)
    with pytest.raises(RuntimeError, match="sum_fp8 input must be float8"):
        torch.ops.hpu.sum_fp8(meta((4,), torch.bfloat16))
    with pytest.raises(RuntimeError, match="out_dtype"):
        torch.ops.hpu.sum_fp8(x, None, False, torch.int32)
    with pytest.raises(RuntimeError, match="appears multiple times"):
        torch.ops.hpu.sum_fp8(x, [1, -2])
    with pytest.raises((RuntimeError, IndexError), match="[Dd]imension out of range"):
        torch.ops.hpu.sum_fp8(x, [3])


def test_softmax_fp8_meta_and_errors(pkg):
    """SoftmaxFp8Meta and the checks of SoftmaxFp8::AddNode, hpu_ops/backend/softmax_fp8_gen.cpp:65-119."""
    x = meta((5, 4, 4, 6), torch.bfloat16)
    s = meta((), torch.float32)
    f = torch.ops.hpu.softmax_fp8
    assert f(x, -1).dtype == torch.bfloat16 and tuple(f(x, -1).shape) == (5, 4, 4, 6)
    assert f(x, -1, s, s).dtype == E4 and f(x, -1, 0.05, 2.5).dtype == E4 and f(x, -1, 0.05, 2.5, 0.1).dtype == E4
    assert f(x.to(E4), 3, s, s, s, meta((5, 1, 1, 6), torch.bfloat16)).dtype == E4
    for args, msg in (((x.float(), -1), "must be of torch.bfloat16 or torch.float8_e4m3fn"),
                      ((x.to(E5), -1, s, s), "must be of torch.bfloat16 or torch.float8_e4m3fn"),
                      ((x, -1, s, None), "Output and input scales must be both given or None"),
                      ((x, -1, None, s), "Output and input scales must be both given or None"),
                      ((x.to(E4), -1), "then input scale must be given"),
                      ((x, -1, None, None, None, x), "FusedAdd available only for Float8 output"),
                      ((x, -1, s, s, None, meta((5, 4, 6), torch.bfloat16)), "same rank"),
                      ((x, -1, s, s, None, meta((4, 4, 4, 6), torch.bfloat16)), "same first and last dim"),
                      ((x, -1, s, s, None, meta((5, 4, 4, 8), torch.bfloat16)), "same first and last dim"),
                      ((x, -1, s, s, None, meta((5, 2, 4, 6), torch.bfloat16)), "should be equal to 1 or the same"),
                      ((x, -1, s, s, None, meta((5, 1, 1, 6), torch.float32)), "must be of dtype: BFloat16"),
                      ((x, -1, meta((), torch.bfloat16), s), "must be of dtype: Float"),
                      ((x, 4), "[Dd]imension out of range")):
        with pytest.raises((RuntimeError, IndexError), match=msg):
            f(*args)


# ------------------------------------------------------------------ the attention ops' boundary

# habana_eager/eager_custom_op_register.cpp:2274, 2278, 2284-2296
SDPA_SCHEMAS = {
    ("fp8_sdpa_fwd", ""): "hpu::fp8_sdpa_fwd(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor)",
    ("fp8_sdpa_fwd_non_dropout", ""): "hpu::fp8_sdpa_fwd_non_dropout(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor)",
    ("fp8_sdpa_recomp_fwd", ""): "hpu::fp8_sdpa_recomp_fwd(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)",
    ("fp8_sdpa_recomp_fwd_non_dropout", ""): "hpu::fp8_sdpa_recomp_fwd_non_dropout(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)",
    ("fp8_sdpa_recomp_fwd", "scalar"): "hpu::fp8_sdpa_recomp_fwd.scalar(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, float d_scale_q, float d_scale_k, float d_scale_v, float q_scale_s, float q_scale_o, float d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)",
    ("fp8_sdpa_recomp_fwd_non_dropout", "scalar"): "hpu::fp8_sdpa_recomp_fwd_non_dropout.scalar(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, float d_scale_q, float d_scale_k, float d_scale_v, float q_scale_s, float q_scale_o, float d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)",
}


@pytest.mark.parametrize("key", sorted(SDPA_SCHEMAS))
def test_attention_schemas_are_the_references(pkg, key):
    name, overload = key
    op = getattr(torch.ops.hpu, name)
    got = str(getattr(op, overload or "default")._schema)
    assert got == SDPA_SCHEMAS[key]


@pytest.mark.parametrize("qdt,fast,qo,expect", [
    # out, m, linv dtypes of the recompute forward (sdpa_gen.cpp:917-947, eager_custom_op_register.cpp:1795-1808)
    (E4, False, False, (torch.bfloat16, torch.bfloat16, torch.bfloat16)),
    (E4, False, True, (E4, torch.bfloat16, torch.bfloat16)),
    (torch.bfloat16, False, False, (torch.bfloat16, torch.bfloat16, torch.float32)),
    (torch.bfloat16, True, False, (torch.bfloat16, torch.bfloat16, torch.bfloat16)),
    (torch.float32, True, False, (torch.float32, torch.float32, torch.float32)),
    # e5m2 q: treated like e4m3fn here (the reference would give an e5m2 output and Float linv; stated as a deviation)
    (E5, False, False, (torch.bfloat16, torch.bfloat16, torch.bfloat16)),
])
def test_fp8_sdpa_recomp_fwd_meta_dtypes(pkg, qdt, fast, qo, expect):
    q, k, v = meta((2, 4, 33, 64), qdt), meta((2, 4, 50, 64), qdt), meta((2, 4, 50, 48), qdt)
    outs = torch.ops.hpu.fp8_sdpa_recomp_fwd.scalar(q, k, v, None, 0.0, 0.125, True, False, "fast" if fast else "None",
                                                    1.0, 1.0, 1.0, 128.0, 16.0 if qo else 0.0, 0.0, True, True, None, "left")
    out, m, linv, seed, amax_s, amax_o = outs
    assert tuple(out.shape) == (2, 4, 33, 48)
    assert (out.dtype, m.dtype, linv.dtype) == expect
    assert seed.dtype == torch.int32 and amax_s.dtype == torch.float32 and amax_o.dtype == torch.float32
    assert all(tuple(t.shape) == (1,) for t in (m, linv, seed, amax_s, amax_o))


def test_fp8_sdpa_fwd_meta(pkg):
    """out, P [batch..., L, S] in q's dtype, the one-element Char dropout mask, Float amax_s
    (SDPAFwdOutputShapeCommon, sdpa_gen.cpp:103-150; types :412-436)."""
    q, k, v = meta((2, 2, 2, 33, 64), E4), meta((2, 2, 1, 50, 64), E4), meta((2, 2, 1, 50, 48), E4)
    sc = meta((1,), torch.float32)
    out, P, dm, amax_s = torch.ops.hpu.fp8_sdpa_fwd(q, k, v, None, 0.0, 0.125, True, "None", None, None, None, sc, None, None, False, None, "left")
    assert tuple(out.shape) == (2, 2, 2, 33, 48) and out.dtype == torch.bfloat16
    assert tuple(P.shape) == (2, 2, 2, 33, 50) and P.dtype == E4
    assert tuple(dm.shape) == (1,) and dm.dtype == torch.int8 and tuple(amax_s.shape) == (1,) and amax_s.dtype == torch.float32
    out = torch.ops.hpu.fp8_sdpa_fwd_non_dropout(q, k, v, None, 0.0, 0.125, True, "None", None, None, None, sc, sc, None, False, None, "left")[0]
    assert out.dtype == E4
    with pytest.raises(RuntimeError, match="valid_seq_len is supported only"):
        torch.ops.hpu.fp8_sdpa_fwd(q, k, v, None, 0.0, 0.125, False, "None", None, None, None, None, None, None, False,
                                   meta((2,), torch.int32), "left")
    with pytest.raises(RuntimeError, match="dropout is not implemented"):
        torch.ops.hpu.fp8_sdpa_fwd(q, k, v, None, 0.5, 0.125, True, "None", None, None, None, None, None, None, False, None, "left")


def test_w4a8_gemm_rejects_a_zero_point_or_bias_on_another_device(pkg):
    """Every pointer the kernel dereferences is checked against A's device before anything is launched (a host
    pointer read on the GPU is a memory fault); exercised on meta tensors, where nothing can be launched."""
    A, packed, scale = meta((16, 256), E4), meta((256, 32), torch.int32), meta((2, 256), torch.bfloat16)
    out = torch.ops.mi355q.w4a8_gemm(A, packed, scale, meta((2, 32), torch.int32), False, torch.bfloat16, None, meta((256,), torch.bfloat16))
    assert tuple(out.shape) == (16, 256)
    with pytest.raises(RuntimeError, match="zero_point must be on the same device as A"):
        torch.ops.mi355q.w4a8_gemm(A, packed, scale, torch.zeros(2, 32, dtype=torch.int32), False, torch.bfloat16, None, None)
    with pytest.raises(RuntimeError, match="bias must be on the same device as A"):
        torch.ops.mi355q.w4a8_gemm(A, packed, scale, None, False, torch.bfloat16, None, torch.zeros(256, dtype=torch.bfloat16))
