"""PT2E quantizer and observers that put a model's linear / matmul operands into fp8.

The caller side of the fp8 ops: `prepare_pt2e(model, Fp8Quantizer().set_global(cfg))`,
calibration, `convert_pt2e`, then `fx_passes.lower_to_fp8_ops` turns the
quantize / dequantize pairs into `hpu::cast_to_fp8_v2` and `hpu::fp8_gemm_v2`.

Mirrors the reference's interface for this flow:
python_packages/habana_frameworks/torch/core/quantizer.py:100-123 (`habana_quantizer`:
`set_global`, `annotate`), :173-236 (linear and matmul annotation), :292-339
(`habana_quant_config_symmetric`) and core/observer.py:36-255 (`AbsMaxObserver`),
:258-452 (`SimpleAbsMaxObserver`).  Only the operators that end in the fp8 GEMM are
annotated; the reference's conv2d and max-pool annotations have no fp8 kernel behind
them here and are left out.

Everything in this file is host-side graph and statistics code; the device work is in
the ops the lowered graph calls.
"""
import math

import torch
from torch.ao.quantization.observer import PlaceholderObserver, UniformQuantizationObserverBase
from torch.ao.quantization.quantizer import QuantizationAnnotation, QuantizationSpec, Quantizer
from torch.ao.quantization.quantizer.utils import _annotate_input_qspec_map, _annotate_output_qspec
from torch.ao.quantization.quantizer.xnnpack_quantizer_utils import QuantizationConfig

FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)

# quantizer.py:56: the quantised range the reference's configuration states for both
# fp8 formats (Gaudi2's e4m3 maximum); the scale is derived from it.
QUANTIZER_MIN_MAX = {torch.float8_e4m3fn: (-240, 240), torch.float8_e5m2: (-240, 240)}
# quantizer.py:57-58
OBSERVER_ARGS_ACT = {"eps": 2 ** -12, "backoff_margin": 2}
OBSERVER_ARGS_WEIGHT = {"eps": 2 ** -12, "backoff_margin": 1}

# observer.py:159-201 builds, for the device it always picks (Gaudi2), the scales its
# matrix engine applies for free: 2^(7 - b) for the exponent biases b in {3, 7, 11, 15}
# of e4m3fn, i.e. 16, 1, 1/16, 1/256, and the single bias 15 (scale 1) of e5m2.  A scale
# is rounded up to a power of two whose exponent is a multiple of 4 and clamped to that
# set's range.  MI355X has no exponent bias to set; the rule is kept so that a model
# calibrated here carries the scales the reference would give it.
_HW_SCALE_RANGE = {torch.float8_e4m3fn: (2.0 ** -8, 2.0 ** 4), torch.float8_e5m2: (1.0, 1.0)}
_HW_SCALE_EXPONENT_STEP = 4


def scale_to_pow2_hw(scale: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """observer.py:203-217: 2^ceil(log2 s), exponent rounded up to a multiple of 4, clamped."""
    lo, hi = _HW_SCALE_RANGE[dtype]
    pow2 = 2 ** torch.ceil(torch.log2(scale))
    stepped = 2 ** (torch.ceil(torch.log2(pow2) / _HW_SCALE_EXPONENT_STEP) * _HW_SCALE_EXPONENT_STEP)
    return torch.clamp(stepped, min=lo, max=hi)


def _check_observer_args(name, dtype, qscheme, reduce_range, is_dynamic):
    # observer.py:105-112, same messages
    if dtype not in FP8_DTYPES:
        raise NotImplementedError(f"{name}: dtype only supports torch.float8_e5m2 and torch.float8_e4m3fn.")
    if qscheme != torch.per_tensor_symmetric:
        raise NotImplementedError(f"{name}: qscheme only supports torch.per_tensor_symmetric.")
    if reduce_range:
        raise NotImplementedError(f"{name}: reduce_range is not supported.")
    if is_dynamic:
        raise NotImplementedError(f"{name}: is_dynamic is not supported.")


class AbsMaxObserver(UniformQuantizationObserverBase):
    """Running minimum and maximum; scale = hw(max(absmax * 2^margin / half_range, eps)), zero point 0.

    absmax = max(-min(x_min, 0), max(x_max, 0)); half_range = (quant_max - quant_min) / 2
    (observer.py:219-229).
    """

    def __init__(self, dtype=torch.float8_e4m3fn, qscheme=torch.per_tensor_symmetric, reduce_range=False,
                 quant_min=torch.finfo(torch.float8_e4m3fn).min, quant_max=torch.finfo(torch.float8_e4m3fn).max,
                 factory_kwargs=None, eps=torch.finfo(torch.float32).eps, backoff_margin=0, is_dynamic=False,
                 **kwargs):
        _check_observer_args("AbsMaxObserver", dtype, qscheme, reduce_range, is_dynamic)
        assert quant_min == -quant_max
        super().__init__(dtype=dtype, qscheme=qscheme, reduce_range=reduce_range, quant_min=quant_min,
                         quant_max=quant_max, factory_kwargs=factory_kwargs, eps=eps, is_dynamic=is_dynamic, **kwargs)
        fk = torch.nn.factory_kwargs(factory_kwargs)
        self.register_buffer("min_val", torch.tensor(float("inf"), **fk))
        self.register_buffer("max_val", torch.tensor(float("-inf"), **fk))
        self.backoff_margin = backoff_margin

    def forward(self, x_orig):
        if x_orig.numel() == 0:
            return x_orig
        lo, hi = torch.aminmax(x_orig.detach().to(self.min_val.dtype))
        self.min_val.copy_(torch.min(lo, self.min_val))
        self.max_val.copy_(torch.max(hi, self.max_val))
        return x_orig

    def _absmax(self):
        neg = torch.min(self.min_val, torch.zeros_like(self.min_val))
        pos = torch.max(self.max_val, torch.zeros_like(self.max_val))
        return torch.max(-neg, pos)

    @torch.jit.export
    def calculate_qparams(self):
        half_range = float(self.quant_max - self.quant_min) / 2
        scale = torch.max(self._absmax() / half_range * (2 ** self.backoff_margin), self.eps)
        scale = scale_to_pow2_hw(scale, self.dtype)
        return scale, torch.zeros(scale.size(), dtype=torch.int64, device=scale.device)

    @torch.jit.export
    def extra_repr(self):
        return f"min_val={self.min_val}, max_val={self.max_val}"

    @torch.jit.export
    def reset_observer_state(self):
        self.min_val.copy_(torch.tensor(float("inf")))
        self.max_val.copy_(torch.tensor(float("-inf")))


class SimpleAbsMaxObserver(UniformQuantizationObserverBase):
    """Running maximum of |x|; scale = hw(max(absmax * 2^margin / quant_max, eps)) (observer.py:420-437)."""

    def __init__(self, dtype=torch.float8_e4m3fn, qscheme=torch.per_tensor_symmetric, reduce_range=False,
                 quant_min=torch.finfo(torch.float8_e4m3fn).min, quant_max=torch.finfo(torch.float8_e4m3fn).max,
                 factory_kwargs=None, eps=torch.finfo(torch.float32).eps, backoff_margin=0, is_dynamic=False,
                 **kwargs):
        _check_observer_args("SimpleAbsMaxObserver", dtype, qscheme, reduce_range, is_dynamic)
        assert quant_min == -quant_max
        super().__init__(dtype=dtype, qscheme=qscheme, reduce_range=reduce_range, quant_min=quant_min,
                         quant_max=quant_max, factory_kwargs=factory_kwargs, eps=eps, is_dynamic=is_dynamic, **kwargs)
        fk = torch.nn.factory_kwargs(factory_kwargs)
        self.register_buffer("abs_max_val", torch.tensor(0.0, **fk))
        self.backoff_margin = backoff_margin

    def forward(self, x_orig):
        if x_orig.numel() == 0:
            return x_orig
        cur = x_orig.detach().to(self.abs_max_val.dtype).abs().max()
        self.abs_max_val.copy_(torch.max(cur, self.abs_max_val))
        return x_orig

    @torch.jit.export
    def calculate_qparams(self):
        scale = torch.max(self.abs_max_val / float(self.quant_max) * (2 ** self.backoff_margin), self.eps)
        scale = scale_to_pow2_hw(scale, self.dtype)
        return scale, torch.zeros(scale.size(), dtype=torch.int64, device=scale.device)

    @torch.jit.export
    def extra_repr(self):
        return f"abs_max_val={self.abs_max_val}"

    @torch.jit.export
    def reset_observer_state(self):
        self.abs_max_val.copy_(torch.tensor(0.0))


def fp8_quant_config_symmetric(quant_dtype, observer=AbsMaxObserver) -> QuantizationConfig:
    """Per-tensor symmetric fp8 for activations and weights, bias left in floating point
    (quantizer.py:292-339)."""
    if quant_dtype not in FP8_DTYPES:
        raise NotImplementedError(f"fp8_quant_config_symmetric: {quant_dtype} is not an fp8 dtype")
    qmin, qmax = QUANTIZER_MIN_MAX[quant_dtype]

    def spec(args, **extra):
        return QuantizationSpec(dtype=quant_dtype, quant_min=qmin, quant_max=qmax, qscheme=torch.per_tensor_symmetric,
                                is_dynamic=False, observer_or_fake_quant_ctr=observer.with_args(**args), **extra)

    bias = QuantizationSpec(dtype=torch.float, observer_or_fake_quant_ctr=PlaceholderObserver)
    return QuantizationConfig(spec(OBSERVER_ARGS_ACT), None, spec(OBSERVER_ARGS_WEIGHT, ch_axis=0), bias)


_aten = torch.ops.aten
# operand positions: (activation inputs, weight input or None, bias input or None)
_GEMM_LIKE = {
    _aten.linear.default: ((0,), 1, 2),
    _aten.addmm.default: ((1,), 2, 0),
    _aten.mm.default: ((0, 1), None, None),
    _aten.bmm.default: ((0, 1), None, None),
    _aten.matmul.default: ((0, 1), None, None),
}


def _annotated(node):
    a = node.meta.get("quantization_annotation")
    return a is not None and a._annotated


class Fp8Quantizer(Quantizer):
    """Annotates linear, matmul, mm, bmm and addmm nodes: inputs quantised, output left alone.

    The reference finds these through source partitions of `torch.nn.Linear` and
    `torch.matmul` (quantizer.py:173-236); graphs exported by current PyTorch carry
    `aten.linear.default` / `aten.matmul.default` nodes themselves, so the nodes are
    matched by target.  A linear's weight and bias are the parameters it reads.
    """

    def __init__(self):
        super().__init__()
        self.global_config = None

    def set_global(self, quantization_config: QuantizationConfig):
        self.global_config = quantization_config
        return self

    def annotate(self, model: torch.fx.GraphModule) -> torch.fx.GraphModule:
        cfg = self.global_config
        if cfg is None:
            raise RuntimeError("Fp8Quantizer: call set_global(config) first")
        for node in model.graph.nodes:
            if node.op != "call_function" or node.target not in _GEMM_LIKE or _annotated(node):
                continue
            acts, weight, bias = _GEMM_LIKE[node.target]
            operands = [(i, cfg.input_activation) for i in acts]
            if weight is not None:
                operands.append((weight, cfg.weight))
            if bias is not None and len(node.args) > bias and isinstance(node.args[bias], torch.fx.Node):
                operands.append((bias, cfg.bias))
            if any(not isinstance(node.args[i], torch.fx.Node) for i, _ in operands):
                continue
            for i, qspec in operands:
                _annotate_input_qspec_map(node, node.args[i], qspec)
            if cfg.output_activation is not None:
                _annotate_output_qspec(node, cfg.output_activation)
            node.meta["quantization_annotation"]._annotated = True
        return model

    def validate(self, model: torch.fx.GraphModule) -> None:
        pass

    @classmethod
    def get_supported_operators(cls):
        return []


# the names the reference exports
habana_quantizer = Fp8Quantizer
habana_quant_config_symmetric = fp8_quant_config_symmetric
