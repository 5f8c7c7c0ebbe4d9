"""The FX rewrites that land a PT2E-quantised graph on the fp8 ops (node counts on CPU as in the
reference's compile/test_pt2e_quant_flow.py:213-232; numerics on the GPU)."""
import importlib

import pytest
import torch
import torch.ao.quantization.fx._decomposed  # noqa: F401  registers quantized_decomposed

from helpers import E4, E5, gemm_errors

q = torch.ops.quantized_decomposed
SA, SB = 0.05, 0.02


def passes(pkg):
    return importlib.import_module(pkg.__name__ + ".fx_passes")


def attention_like(a, b):
    """bmm of two quantise -> dequantise pairs, the second operand transposed (q @ k^T)."""
    a8 = q.quantize_per_tensor.default(a, SA, 0, -448, 448, E4)
    b8 = q.quantize_per_tensor.default(b, SB, 0, -448, 448, E4)
    ad = q.dequantize_per_tensor.default(a8, SA, 0, -448, 448, E4)
    bd = q.dequantize_per_tensor.default(b8, SB, 0, -448, 448, E4)
    return torch.ops.aten.bmm.default(ad, torch.ops.aten.transpose.int(bd, 1, 2))


def count(gm, name):
    return sum(1 for n in gm.graph.nodes if n.op == "call_function" and getattr(n.target, "__name__", "") == name)


def test_rewrites_node_counts(pkg):
    gm = torch.fx.symbolic_trace(attention_like)
    assert passes(pkg).lower_to_fp8_ops(gm, device="cpu") == (2, 1)
    # test_pt2e_quant_flow.py:226-227: two cast_to_fp8_v2.scalar, one fp8_gemm_v2.default, nothing left over
    assert count(gm, "cast_to_fp8_v2.scalar") == 2 and count(gm, "fp8_gemm_v2.default") == 1
    for gone in ("quantize_per_tensor.default", "dequantize_per_tensor.default", "bmm.default", "transpose.int"):
        assert count(gm, gone) == 0, gone
    gemm = next(n for n in gm.graph.nodes if getattr(n.target, "__name__", "") == "fp8_gemm_v2.default")
    assert gemm.args[1] is False and gemm.args[3] is True and gemm.args[5] == torch.bfloat16
    assert gm.get_buffer(gemm.args[6].target).item() == pytest.approx(SA) and gm.get_buffer(gemm.args[7].target).item() == pytest.approx(SB)
    cast = next(n for n in gm.graph.nodes if getattr(n.target, "__name__", "") == "cast_to_fp8_v2.scalar")
    assert cast.args[1] == pytest.approx(1.0 / SA) and cast.args[4] == E4


def test_a_narrower_quant_range_becomes_a_clamp(pkg):
    """The reference's quantizer asks for qmin / qmax = -+240 (core/quantizer.py:100-123) where e4m3fn holds
    448: the rewrite keeps the node's range with a clamp of the input to [qmin * s, qmax * s]."""
    def narrow(a):
        return q.quantize_per_tensor.default(a, SA, 0, -240, 240, E4)

    def full(a):
        return q.quantize_per_tensor.default(a, SA, 0, -448, 448, E4)

    gm = torch.fx.symbolic_trace(narrow)
    assert passes(pkg).replace_quantize_with_cast(gm) == 1
    assert count(gm, "clamp.default") == 1 and count(gm, "cast_to_fp8_v2.scalar") == 1
    clamp = next(n for n in gm.graph.nodes if getattr(n.target, "__name__", "") == "clamp.default")
    assert clamp.args[1] == pytest.approx(-240 * SA) and clamp.args[2] == pytest.approx(240 * SA)
    gm = torch.fx.symbolic_trace(full)
    assert passes(pkg).replace_quantize_with_cast(gm) == 1 and count(gm, "clamp.default") == 0


@pytest.mark.gpu
def test_values_beyond_a_narrow_range_saturate_at_it(pkg, dev):
    def narrow(a):
        return q.quantize_per_tensor.default(a, SA, 0, -240, 240, E4)

    x = torch.tensor([[0.5, 13.0, 100.0, -100.0, 11.9, -12.1]], device=dev).bfloat16()     # 240 * SA = 12
    ref = narrow(x)
    gm = torch.fx.symbolic_trace(narrow)
    passes(pkg).replace_quantize_with_cast(gm)
    out = gm(x)
    assert out.dtype == E4 and torch.equal(out.float(), ref.float())
    assert out.float().abs().max().item() == 240.0


def test_rewrites_leave_other_graphs_alone(pkg):
    def int8_quant(a):
        return q.quantize_per_tensor.default(a, 0.1, 3, -128, 127, torch.int8)

    def reshaped(a, b):
        ad = q.dequantize_per_tensor.default(a, SA, 0, -448, 448, E4)
        bd = q.dequantize_per_tensor.default(b, SB, 0, -57344, 57344, E5)
        return torch.ops.aten.bmm.default(ad, torch.ops.aten.view.default(bd, [2, 8, 4]))

    for fn in (int8_quant, reshaped):
        gm = torch.fx.symbolic_trace(fn)
        before = str(gm.graph)
        assert passes(pkg).lower_to_fp8_ops(gm, device="cpu") == (0, 0)
        assert str(gm.graph) == before


@pytest.mark.gpu
def test_rewritten_graph_runs_on_the_gpu(pkg, dev):
    gm = torch.fx.symbolic_trace(attention_like)
    assert passes(pkg).lower_to_fp8_ops(gm, device=dev) == (2, 1)
    g = torch.Generator().manual_seed(6)
    a = torch.randn(3, 64, 128, generator=g).bfloat16()
    b = torch.randn(3, 96, 128, generator=g).bfloat16()
    out = gm(a.to(dev), b.to(dev))
    assert out.shape == (3, 64, 96) and out.dtype == torch.bfloat16
    # what the quantised graph means: operands rounded to e4m3 at their scales, exact product, one rounding
    # (the cast multiplies by the bf16-rounded inverse scale in bf16 for a bf16 input)
    a8 = (a * torch.tensor(1.0 / SA).bfloat16()).clamp(-448, 448).to(E4).float() * SA
    b8 = (b * torch.tensor(1.0 / SB).bfloat16()).clamp(-448, 448).to(E4).float() * SB
    ref = torch.bmm(a8, b8.transpose(1, 2))
    rel, ok = gemm_errors(out, ref)
    assert rel <= 1e-2 and ok, rel
