"""FX graph rewrites that land a PT2E-quantised model on the fp8 ops.

A model quantised with torch.ao's PT2E flow carries
`quantized_decomposed.quantize_per_tensor` / `dequantize_per_tensor` nodes
around its matmuls.  The two passes here turn them into `hpu::cast_to_fp8_v2`
and `hpu::fp8_gemm_v2`, the rewrites the reference applies in
python_packages/habana_frameworks/torch/core/pattern_matcher.py:100-138
(quantize -> cast with the inverted scale), :182-300 (bmm of two dequantised
operands -> fp8 GEMM with the two scales as *_scale_inv) and :305-404 (the same
for the mm / addmm a linear layer becomes; graphs exported by current PyTorch
keep `aten.linear` / `aten.matmul` nodes, which are matched as well).  Written
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


_FP8_MAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


def replace_quantize_with_cast(gm: torch.fx.GraphModule) -> int:
    """quantize_per_tensor(x, s, 0, qmin, qmax, fp8) -> cast_to_fp8_v2(x, 1 / s, False, False, fp8)[0].

    Only fp8 targets with a zero zero-point are rewritten.  The cast saturates at the format's
    maximum (448 for e4m3fn, 57344 for e5m2).  A node whose [qmin, qmax] is narrower than that --
    the reference's quantizer asks for +-240, the e4m3 range of the device it was written for
    (core/quantizer.py:100-123) -- gets a clamp of x to [qmin * s, qmax * s] in front of the cast,
    so that values beyond the node's range saturate where the node says and not at the format's
    maximum.  Returns the number of nodes replaced.
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
        qmin, qmax = _arg(node, 3, "quant_min"), _arg(node, 4, "quant_max")
        fmax = _FP8_MAX[dtype]
        with graph.inserting_before(node):
            src = x
            lo = None if qmin is None or float(qmin) <= -fmax else float(qmin) * float(scale)
            hi = None if qmax is None or float(qmax) >= fmax else float(qmax) * float(scale)
            if lo is not None or hi is not None:
                src = graph.call_function(torch.ops.aten.clamp.default, args=(x, lo, hi))
            cast = graph.call_function(torch.ops.hpu.cast_to_fp8_v2.scalar, args=(src, 1.0 / float(scale), False, False, dtype))
            out = graph.call_function(operator.getitem, args=(cast, 0))
        node.replace_all_uses_with(out)
        graph.erase_node(node)
        count += 1
    if count:
        graph.lint()
        gm.recompile()
    return count


def _rank(node):
    val = node.meta.get("val", node.meta.get("tensor_meta")) if isinstance(node, torch.fx.Node) else None
    shape = getattr(val, "shape", None)
    return None if shape is None else len(shape)


def _dequant_behind(node):
    """(dequantize node, operand is transposed in its last two dims, nodes in between) or None.

    Between the dequantize and the product only clones and transposes of the
    last two dimensions are looked through (`t`, or `transpose.int` whose two
    dimensions are the last two: given as -1 / -2, or judged by the operand's
    rank where the graph records it, else assumed 3-D as in a bmm).
    """
    chain, transposed = [], False
    while isinstance(node, torch.fx.Node) and node.op == "call_function":
        if _is(node, "dequantize_per_tensor.default"):
            return node, transposed, chain
        if _is(node, "transpose.int"):
            rank = _rank(node.args[0]) or 3
            if rank < 2 or {d % rank for d in node.args[1:3]} != {rank - 1, rank - 2}:
                return None
            transposed = not transposed
        elif _is(node, "t.default"):
            transposed = not transposed
        elif not _is(node, "clone.default"):
            return None
        chain.append(node)
        node = node.args[0]
    return None


# product node -> (index of A, index of B, B is stored transposed ([N, K]), index of a bias or None)
_PRODUCTS = {
    "bmm.default": (0, 1, False, None),
    "mm.default": (0, 1, False, None),
    "matmul.default": (0, 1, False, None),
    "linear.default": (0, 1, True, 2),
    "addmm.default": (1, 2, False, 0),
}


def replace_dequant_gemm_with_fp8_gemm(gm: torch.fx.GraphModule, out_dtype=None, device=None) -> int:
    """A product of two dequantised fp8 operands -> fp8_gemm_v2 on the fp8 operands.

    bmm / mm / matmul(dq(a8, sa), [transpose] dq(b8, sb))
        -> fp8_gemm_v2(a8, False, b8, trans_B, None, out_dtype, sa, sb, None, False)
    linear(dq(a8, sa), dq(w8, sw), bias) and addmm(bias, dq(a8, sa), transpose(dq(w8, sw)))
        -> fp8_gemm_v2(a8, False, w8, True, None, out_dtype, sa, sw, bias, False)
    (the reference's pattern_matcher.py:182-300 for bmm and :305-404 for mm / addmm).

    The dequantise scales become the GEMM's A_scale_inv / B_scale_inv, as 0-dim
    fp32 buffers of the module on `device` (default: the current GPU if there
    is one).  `out_dtype` defaults to the dtype the dequantise nodes produce
    (their `out_dtype` keyword), bfloat16 if they name none.  Operands that
    reach the product through anything but a transpose of their last two
    dimensions (or a clone) are left alone, and so is a transposed A.  Returns
    the number of product nodes replaced.
    """
    graph = gm.graph
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    count = 0
    for node in list(graph.nodes):
        name = getattr(node.target, "__name__", None) if node.op == "call_function" else None
        if name not in _PRODUCTS:
            continue
        ia, ib, b_stored_transposed, ibias = _PRODUCTS[name]
        if name == "addmm.default" and (node.kwargs.get("alpha", 1) != 1 or node.kwargs.get("beta", 1) != 1):
            continue
        a, b = _dequant_behind(node.args[ia]), _dequant_behind(node.args[ib])
        if a is None or b is None or a[1]:
            continue
        (dq_a, _, chain_a), (dq_b, trans_b, chain_b) = a, b
        trans_b = trans_b != b_stored_transposed
        scales = []
        for dq in (dq_a, dq_b):
            s, zp, dt = dq.args[1], _arg(dq, 2, "zero_point", 0), _arg(dq, 5, "dtype")
            if isinstance(s, torch.fx.Node) or zp != 0 or dt not in _FP8:
                scales = None
                break
            scales.append(float(s))
        if scales is None:
            continue
        dtype = out_dtype or dq_a.kwargs.get("out_dtype") or torch.bfloat16
        if dtype not in (torch.bfloat16, torch.float32):
            continue
        bias = node.args[ibias] if ibias is not None and len(node.args) > ibias else None
        names = []
        for s in scales:
            buf = f"_fp8_scale_inv_{sum(1 for _ in gm.buffers())}"
            gm.register_buffer(buf, torch.tensor(s, dtype=torch.float32, device=device))
            names.append(buf)
        with graph.inserting_before(node):
            sa, sb = graph.get_attr(names[0]), graph.get_attr(names[1])
            gemm = graph.call_function(torch.ops.hpu.fp8_gemm_v2.default,
                                       args=(dq_a.args[0], False, dq_b.args[0], trans_b, None, dtype, sa, sb, bias, False))
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


def replace_dequant_bmm_with_fp8_gemm(gm: torch.fx.GraphModule, out_dtype=torch.bfloat16, device=None) -> int:
    """The same rewrite under its first name (it began with bmm alone)."""
    return replace_dequant_gemm_with_fp8_gemm(gm, out_dtype, device)


def lower_to_fp8_ops(gm: torch.fx.GraphModule, out_dtype=None, device=None):
    """Both rewrites, products first (they read the dequantise nodes' scales); returns
    (quantize nodes replaced, product nodes replaced)."""
    products = replace_dequant_gemm_with_fp8_gemm(gm, out_dtype, device)
    return replace_quantize_with_cast(gm), products


def fold_constant_casts(gm: torch.fx.GraphModule) -> int:
    """Evaluates cast_to_fp8_v2 of a parameter or buffer once and keeps the fp8 result as a buffer.

    After `lower_to_fp8_ops` a linear layer's weight is cast to fp8 on every call.  For inference the
    weight is a constant, so the cast is run here, by the same op, and the graph reads the stored fp8
    tensor instead (the reference leaves this to its graph compiler).  Only tensors that live on a
    GPU are folded: the op has no CPU implementation.  Returns the number of casts folded.
    """
    graph = gm.graph
    count = 0
    for node in list(graph.nodes):
        if not (_is(node, "cast_to_fp8_v2.scalar") or _is(node, "cast_to_fp8_v2.default")):
            continue
        src = node.args[0]
        # the clamp that replace_quantize_with_cast puts in front of a cast with a narrow range
        clamp = src if _is(src, "clamp.default") and len(src.users) == 1 else None
        if clamp is not None:
            src = clamp.args[0]
        if not (isinstance(src, torch.fx.Node) and src.op == "get_attr"):
            continue
        if any(isinstance(a, torch.fx.Node) for a in node.args[1:]) or any(isinstance(v, torch.fx.Node) for v in node.kwargs.values()):
            continue
        if any(not (u.op == "call_function" and u.target is operator.getitem and u.args[1] == 0) for u in node.users):
            continue
        obj = gm
        for part in src.target.split("."):
            obj = getattr(obj, part)
        if not isinstance(obj, torch.Tensor) or not obj.is_cuda:
            continue
        with torch.no_grad():
            const_in = obj.detach()
            if clamp is not None:
                const_in = clamp.target(const_in, *clamp.args[1:])
            value = node.target(const_in, *node.args[1:], **node.kwargs)[0]
        name = f"_fp8_const_{sum(1 for _ in gm.buffers())}"
        gm.register_buffer(name, value)
        with graph.inserting_before(node):
            const = graph.get_attr(name)
        for user in list(node.users):
            user.replace_all_uses_with(const)
            graph.erase_node(user)
        graph.erase_node(node)
        if clamp is not None:
            graph.erase_node(clamp)
        if not src.users:
            graph.erase_node(src)
        count += 1
    if count:
        graph.lint()
        gm.recompile()
    return count
