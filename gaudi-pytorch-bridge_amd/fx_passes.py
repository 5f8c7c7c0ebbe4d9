"""FX graph rewrites that land a PT2E-quantised model on the fp8 ops.

A model quantised with torch.ao's PT2E flow carries
`quantized_decomposed.quantize_per_tensor` / `dequantize_per_tensor` nodes
around its matmuls.  The two passes here turn them into `hpu::cast_to_fp8_v2`
and `hpu::fp8_gemm_v2`, the rewrites the reference applies in
python_packages/habana_frameworks/torch/core/pattern_matcher.py:100-138
(quantize -> cast with the inverted scale) and :182-300 (bmm of two
dequantised operands -> fp8 GEMM with the two scales as *_scale_inv).  Written
against the FX node API only; no graph is executed here.
"""
import operator

import torch

_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)
def _is(node, name):
    return (isinstance(node, torch.fx.Node) and node.op == "call_function"
            and getattr(node.target, "__name__", None) == name)


def _arg(node, index, name, default=None):
    if len(node.args) > index:
        return node.args[index]
    return node.kwargs.get(name, default)


def replace_quantize_with_cast(gm: torch.fx.GraphModule) -> int:
    """quantize_per_tensor(x, s, 0, qmin, qmax, fp8) -> cast_to_fp8_v2(x, 1 / s, False, False, fp8)[0].

    Only fp8 targets with a zero zero-point are rewritten (the cast saturates at
    the format's maximum, which is what qmin / qmax say for fp8).  Returns the
    number of nodes replaced.
    """
    graph = gm.graph
    count = 0
    for node in list(graph.nodes):
        if not _is(node, "quantize_per_tensor.default"):
            continue
        x, scale = node.args[0], node.args[1]
        zero_point, dtype = _arg(node, 2, "zero_point", 0), _arg(node, 5, "dtype")
        if dtype not in _FP8 or zero_point != 0 or isinstance(scale, torch.fx.Node):
            continue
        with graph.inserting_before(node):
            cast = graph.call_function(torch.ops.hpu.cast_to_fp8_v2.scalar, args=(x, 1.0 / float(scale), False, False, dtype))
            out = graph.call_function(operator.getitem, args=(cast, 0))
        node.replace_all_uses_with(out)
        graph.erase_node(node)
        count += 1
    if count:
        graph.lint()
        gm.recompile()
    return count


def _dequant_behind(node):
    """(dequantize node, operand is transposed in its last two dims, nodes in between) or None.

    Between the dequantize and the product only clones and transposes of the
    last two dimensions of a 3-D tensor are looked through.
    """
    chain, transposed = [], False
    while isinstance(node, torch.fx.Node) and node.op == "call_function":
        if _is(node, "dequantize_per_tensor.default"):
            return node, transposed, chain
        if _is(node, "transpose.int"):
            if {d % 3 for d in node.args[1:3]} != {1, 2}:
                return None
            transposed = not transposed
        elif not _is(node, "clone.default"):
            return None
        chain.append(node)
        node = node.args[0]
    return None


def replace_dequant_bmm_with_fp8_gemm(gm: torch.fx.GraphModule, out_dtype=torch.bfloat16, device=None) -> int:
    """bmm(dequantize(a8, sa), [transpose] dequantize(b8, sb)) -> fp8_gemm_v2(a8, False, b8, trans_B, None, out_dtype, sa, sb).

    The dequantise scales become the GEMM's A_scale_inv / B_scale_inv, as 0-dim
    fp32 buffers of the module on `device` (default: the current GPU if there
    is one).  Operands that reach the bmm through anything but a transpose of
    their last two dimensions (or a clone) are left alone.  Returns the number
    of bmm nodes replaced.
    """
    graph = gm.graph
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    count = 0
    for node in list(graph.nodes):
        if not _is(node, "bmm.default"):
            continue
        a, b = _dequant_behind(node.args[0]), _dequant_behind(node.args[1])
        if a is None or b is None or a[1]:
            continue
        (dq_a, _, chain_a), (dq_b, trans_b, chain_b) = a, b
        scales = []
        for dq in (dq_a, dq_b):
            s, zp, dt = dq.args[1], _arg(dq, 2, "zero_point", 0), _arg(dq, 5, "dtype")
            if isinstance(s, torch.fx.Node) or zp != 0 or dt not in _FP8:
                scales = None
                break
            scales.append(float(s))
        if scales is None:
            continue
        names = []
        for s in scales:
            name = f"_fp8_scale_inv_{sum(1 for _ in gm.buffers())}"
            gm.register_buffer(name, torch.tensor(s, dtype=torch.float32, device=device))
            names.append(name)
        with graph.inserting_before(node):
            sa, sb = graph.get_attr(names[0]), graph.get_attr(names[1])
            gemm = graph.call_function(torch.ops.hpu.fp8_gemm_v2.default,
                                       args=(dq_a.args[0], False, dq_b.args[0], trans_b, None, out_dtype, sa, sb, None, False))
        node.replace_all_uses_with(gemm)
        graph.erase_node(node)
        for n in chain_a + [dq_a] + chain_b + [dq_b]:
            if not n.users:
                graph.erase_node(n)
        count += 1
    if count:
        graph.lint()
        gm.recompile()
    return count


def lower_to_fp8_ops(gm: torch.fx.GraphModule, out_dtype=torch.bfloat16, device=None):
    """Both rewrites; returns (quantize nodes replaced, bmm nodes replaced)."""
    return replace_quantize_with_cast(gm), replace_dequant_bmm_with_fp8_gemm(gm, out_dtype, device)
