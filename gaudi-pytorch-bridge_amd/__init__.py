"""MI355X-native fp8 / int4 quantized-inference ops behind ``torch.ops.hpu``.

Importing this package loads two in-tree shared libraries:

  libmi355q.so     hand-written gfx950 HIP kernels behind a C ABI
                   (include/mi355q.h)
  mi355q_torch.so  the TORCH_LIBRARY(hpu) host layer; after the import
                   ``torch.ops.hpu.cast_to_fp8_v2``, ``cast_from_fp8``,
                   ``fp8_gemm_v2``, ``convert_from_int4`` and
                   ``convert_from_uint4`` exist with the reference's schemas
                   (habana_eager/eager_custom_op_register.cpp:2146-2171).

The directory name holds a hyphen, so the package is loaded by path under the
module name ``gaudi_pytorch_bridge_amd`` (see ``__graft_entry__.load_package``).
There is no CPU implementation and no fallback: if a library is missing the
import raises, and the ops only accept tensors on the GPU (or meta tensors for
tracing).
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_KERNELS = os.path.join(_HERE, "libmi355q.so")
LIB_TORCH = os.path.join(_HERE, "mi355q_torch.so")

_capi = None


def _load():
    global _capi
    if _capi is not None:
        return _capi
    for p in (LIB_KERNELS, LIB_TORCH):
        if not os.path.exists(p):
            raise ImportError(
                f"{p} is missing: build it with `python {os.path.join(_HERE, 'build.py')}` "
                "(there is no fallback implementation)")
    # torch is imported first so that the HIP runtime PyTorch ships is the one
    # both libraries bind to.
    _capi = ctypes.CDLL(LIB_KERNELS, mode=ctypes.RTLD_GLOBAL)
    torch.ops.load_library(LIB_TORCH)
    return _capi


def capi():
    """ctypes handle of libmi355q.so with argument types declared."""
    L = _load()
    if getattr(L, "_typed", False):
        return L
    c = ctypes
    i64, vp, f32, i32 = c.c_int64, c.c_void_p, c.c_float, c.c_int
    L.mi355q_abi_version.restype = i32
    L.mi355q_status_string.argtypes = [i32]
    L.mi355q_status_string.restype = c.c_char_p
    L.mi355q_amax.argtypes = [vp, i32, i64, vp, vp]
    L.mi355q_rowwise_amax.argtypes = [vp, i32, i64, i64, vp, vp]
    L.mi355q_quantize_rows.argtypes = [vp, i32, i64, i64, vp, i32, f32, vp, vp, vp]
    L.mi355q_silu_mul_quantize_rows.argtypes = [vp, i64, vp, i64, i64, i64, vp, i32, f32, vp, vp, vp, vp]
    L.mi355q_cast_to_fp8.argtypes = [vp, i32, vp, i32, vp, f32, i32, i64, i64, i64, vp, vp]
    L.mi355q_cast_to_fp8_sr.argtypes = [vp, i32, vp, i32, vp, f32, i32, i64, i64, i64, vp, c.c_uint64, c.c_uint64, i32, vp]
    L.mi355q_cast_to_fp8_hybrid.argtypes = [vp, i32, i64, vp, vp, vp, vp, i32, c.c_uint64, c.c_uint64, vp, vp]
    L.mi355q_cast_from_fp8.argtypes = [vp, i32, vp, i32, vp, f32, i32, i64, i64, i64, vp]
    L.mi355q_dequant_4bit.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, i64, vp, vp]
    L.mi355q_fp8_gemm.argtypes = [vp, i32, i32, i64, vp, i32, i32, i64, vp, i32, i64,
                                  i64, i64, i64, vp, f32, i32, vp, f32, i32,
                                  vp, i32, i64, vp, i64, i64, i64, i64, i64, i64, i64, vp]
    L.mi355q_w4a8_gemm.argtypes = [vp, i32, i64, vp, i64, vp, i32, vp, i32, i64, vp, i32, i64, i64, i64, i64,
                                   vp, f32, i32, vp, vp, c.c_size_t, vp]
    L.mi355q_w4a16_gemm.argtypes = [vp, i32, i64, vp, i64, vp, i32, vp, i32, i64, vp, i32, i64, i64, i64, i64, vp, vp, c.c_size_t, i32, vp]
    L.mi355q_w4a16_gemm_workspace_bytes.argtypes = [i64, i64, i64, i64, i32]
    L.mi355q_w4a16_gemm_workspace_bytes.restype = c.c_size_t
    L.mi355q_split_rows_fp8x2.argtypes = [vp, i32, i64, i64, i64, vp, vp, i64, vp, vp]
    L.mi355q_w4a8_gemm_workspace_bytes.argtypes = [i64, i64, i64, i64, i32]
    L.mi355q_w4a8_gemm_workspace_bytes.restype = c.c_size_t
    L.mi355q_fp8_gemm_variant.argtypes = [i32, i64, i32, i64, i64, i64, i64]
    L.mi355q_sum_fp8_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355q_sum_fp8_workspace_bytes.restype = c.c_size_t
    L.mi355q_sum_fp8.argtypes = [vp, i32, i64, i64, i64, vp, i32, vp, c.c_size_t, vp]
    L.mi355q_sum_fp8_static.argtypes = [vp, i32, i64, i64, i64, vp, i32, vp]
    L.mi355q_softmax_fp8.argtypes = [vp, i32, i64, i64, vp, f32, vp, f32, vp, f32, vp, i32, vp, vp, vp, i32, vp]
    L.mi355q_fp8_sdpa_fwd.argtypes = [vp, vp, vp, i32, vp, i32, vp, i32, vp, f32, i32, vp, vp, vp, vp, vp, c.c_size_t, vp]
    L.mi355q_fp8_sdpa_workspace_bytes.argtypes = [vp]
    L.mi355q_fp8_sdpa_workspace_bytes.restype = c.c_size_t
    L.mi355q_fp8_sdpa_key_splits.argtypes = [vp, vp]
    L.mi355q_fp8_sdpa_key_splits.restype = i32
    L.mi355q_fp8_gemm_variant.restype = c.c_char_p
    for name in ("mi355q_amax", "mi355q_rowwise_amax", "mi355q_quantize_rows", "mi355q_silu_mul_quantize_rows", "mi355q_cast_to_fp8", "mi355q_cast_to_fp8_sr", "mi355q_cast_to_fp8_hybrid", "mi355q_cast_from_fp8",
                 "mi355q_dequant_4bit", "mi355q_fp8_gemm", "mi355q_w4a8_gemm", "mi355q_w4a16_gemm", "mi355q_split_rows_fp8x2", "mi355q_sum_fp8", "mi355q_sum_fp8_static", "mi355q_softmax_fp8", "mi355q_fp8_sdpa_fwd"):
        getattr(L, name).restype = i32
    L._typed = True
    return L


def probes():
    """ctypes handle of libmi355q_probe.so: measurement kernels for ``bench.py --only ceilings``
    (csrc/bench/probe_kernels.hip); not part of the product ABI, loaded on request only."""
    path = os.path.join(_HERE, "libmi355q_probe.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python {os.path.join(_HERE, 'build.py')}`")
    c = ctypes
    i64, vp, i32 = c.c_int64, c.c_void_p, c.c_int
    P = c.CDLL(path)
    P.mi355q_probe_mfma.argtypes = [i32, i32, i32, vp, vp]
    P.mi355q_probe_read.argtypes = [vp, i64, i32, vp, vp]
    P.mi355q_probe_coexec.argtypes = [i32, i32, i32, i32, i32, vp, vp]
    P.mi355q_probe_strip_read.argtypes = [vp, i64, i64, i32, i32, i32, vp, vp]
    P.mi355q_probe_amax_ticket.argtypes = [vp, i64, vp, vp]
    P.mi355q_probe_sum_columns_ticket.argtypes = [vp, i64, i64, vp, vp]
    for name in ("mi355q_probe_mfma", "mi355q_probe_read", "mi355q_probe_strip_read", "mi355q_probe_coexec", "mi355q_probe_amax_ticket",
                 "mi355q_probe_sum_columns_ticket"):
        getattr(P, name).restype = i32
    return P


# enums of include/mi355q.h
F32, BF16, E4M3FN, E5M2 = 0, 1, 2, 3
SCALE_NONE, SCALE_HOST, SCALE_DEV, SCALE_MID, SCALE_FULL = 0, 1, 2, 3, 4
GS_NONE, GS_HOST, GS_DEV, GS_PER_ROW, GS_PER_COL = 0, 1, 2, 3, 4
BIAS_NONE, BIAS_ROW_VECTOR, BIAS_FULL = 0, 1, 2
ZP_NONE, ZP_FLOAT, ZP_PACKED = 0, 1, 2
SDPA_MASK_NONE, SDPA_MASK_BOOL, SDPA_MASK_BF16, SDPA_MASK_F32 = 0, 1, 2, 3

EXPORTED_SYMBOLS = (
    "mi355q_abi_version", "mi355q_status_string", "mi355q_amax", "mi355q_rowwise_amax",
    "mi355q_quantize_rows", "mi355q_silu_mul_quantize_rows", "mi355q_cast_to_fp8", "mi355q_cast_to_fp8_sr", "mi355q_cast_to_fp8_hybrid", "mi355q_cast_from_fp8", "mi355q_dequant_4bit", "mi355q_fp8_gemm",
    "mi355q_w4a8_gemm", "mi355q_w4a8_gemm_workspace_bytes", "mi355q_w4a16_gemm", "mi355q_w4a16_gemm_workspace_bytes", "mi355q_split_rows_fp8x2", "mi355q_fp8_gemm_variant", "mi355q_sum_fp8_workspace_bytes", "mi355q_sum_fp8", "mi355q_sum_fp8_static", "mi355q_softmax_fp8", "mi355q_fp8_sdpa_fwd", "mi355q_fp8_sdpa_workspace_bytes", "mi355q_fp8_sdpa_key_splits",
)

_load()

hpu = torch.ops.hpu

_aten_override = None


def use_for_aten_scaled_mm(enable=True):
    """Route ``torch._scaled_mm`` on HIP tensors to this package's fp8 GEMM (``mi355q::scaled_mm``).

    The reference serves ``aten::_scaled_mm`` with the same node as ``hpu::fp8_gemm_v2``
    (hpu_ops/backend/scaled_mm_gen.cpp:66-141).  On PyTorch-ROCm the operator already has a
    kernel (the vendor library), so the replacement is opt-in and reversible:
    ``use_for_aten_scaled_mm(False)`` restores what was registered before.
    """
    global _aten_override
    if not enable:
        if _aten_override is not None:
            _aten_override._destroy()
            _aten_override = None
        return
    if _aten_override is not None:
        return
    import warnings
    lib = torch.library.Library("aten", "IMPL")
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")  # "Overriding a previously registered kernel": intended
        lib.impl("_scaled_mm", torch.ops.mi355q.scaled_mm.default, "CUDA")
    _aten_override = lib
