"""Randomly drawn shapes, layouts, formats and epilogue forms of fp8_gemm_v2 against an exact CPU
reference: operands are small integers and scales multiples of 1/4, so every fp32 partial sum and
product is exact and the only rounding is the final one to the output dtype -- whatever the kernel,
tile edge, K tail, batch stride or epilogue a draw lands on, the result must match bit for bit."""
import random

import pytest
import torch

from helpers import E4, E5

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


def draw(rnd, case):
    def dim(big):
        if big:
            return rnd.choice([rnd.randrange(129, 700), rnd.randrange(700, 4200)]) // 16 * 16 + rnd.choice([0, 0, 16, 8, 4])
        return rnd.choice([rnd.randrange(1, 129), rnd.randrange(16, 129) // 16 * 16])

    M, N = dim(rnd.random() < 0.7), dim(rnd.random() < 0.7)
    K = rnd.choice([rnd.randrange(16, 600), rnd.randrange(16, 40) * 16, 1024, 144])
    if rnd.random() < 0.8:  # mostly shapes the tiled kernels take (multiples of 16), sometimes the any-shape kernel
        M, N, K = (M + 15) // 16 * 16, (N + 15) // 16 * 16, (K + 15) // 16 * 16
    c = {"M": M, "N": N, "K": K, "ta": rnd.random() < 0.4, "tb": rnd.random() < 0.5,
         "fa": rnd.choice([E4, E5]), "fb": rnd.choice([E4, E5]),
         "batch": rnd.choice([None, None, None, 2, 3]) if M * N < 600 * 600 else None,
         "out": rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32]),
         "sa": rnd.choice(["none", "scalar", "tensor1", "row"]), "sb": rnd.choice(["none", "scalar", "tensor1", "col", "row"]),
         "bias": rnd.choice(["none", "none", "vec", "full"]), "d": rnd.random() < 0.25, "seed": case * 7919 + 13,
         "scalar_values": (rnd.choice([0.5, 0.25, 2.0]), rnd.choice([0.5, 0.25, 2.0])), "tensor1_values": (rnd.choice([0.5, 4.0]), rnd.choice([0.5, 4.0]))}
    if (c["sa"] == "scalar") != (c["sb"] == "scalar"):  # the .scalar overload takes two floats
        c["sa"] = c["sb"] = "scalar"
    return c


def run_case(c, dev):
    M, N, K, out_dtype = c["M"], c["N"], c["K"], c["out"]
    g = torch.Generator().manual_seed(c["seed"])
    bs = (c["batch"],) if c["batch"] else ()
    A = torch.randint(-4, 5, bs + ((K, M) if c["ta"] else (M, K)), generator=g).float().to(c["fa"])
    B = torch.randint(-4, 5, (N, K) if c["tb"] else (K, N), generator=g).float().to(c["fb"])  # shared across the batch
    a = A.float().transpose(-2, -1) if c["ta"] else A.float()
    b = B.float().t() if c["tb"] else B.float()
    ref = a @ b

    def scale(kind, which, n, shape):
        if kind == "none":
            return None, 1.0, None
        if kind == "scalar":
            return c["scalar_values"][which], c["scalar_values"][which], None
        if kind == "tensor1":
            v = c["tensor1_values"][which]
            return torch.tensor([v]).to(dev), v, None
        t = torch.randint(1, 5, (n,), generator=g).float() * 0.25
        return t.to(dev), t.reshape(shape), shape

    sa, sa_ref, _ = scale(c["sa"], 0, M, [M, 1])
    if c["sa"] == "row":
        sa = sa.reshape(M, 1)
    sb, sb_ref, sb_shape = scale(c["sb"], 1, M if c["sb"] == "row" else N, [M, 1] if c["sb"] == "row" else [1, N])
    bias, bias_ref = None, 0.0
    if c["bias"] == "vec":
        bias = torch.randint(-8, 9, (N,), generator=g).float().to(out_dtype)
    if c["bias"] == "full":
        bias = torch.randint(-8, 9, (M, N), generator=g).float().to(out_dtype)
    if bias is not None:
        bias_ref = bias.float()
    D = torch.randint(-8, 9, bs + (M, N), generator=g).float().to(out_dtype) if c["d"] else None
    ref = (ref * sa_ref * sb_ref + bias_ref + (D.float() if c["d"] else 0.0)).to(out_dtype)
    dv = lambda t: None if t is None else t.to(dev)
    if c["sa"] == "scalar":
        out = ops.fp8_gemm_v2(A.to(dev), c["ta"], B.to(dev), c["tb"], dv(D), out_dtype, float(sa), float(sb), dv(bias), c["d"])
    else:
        out = ops.fp8_gemm_v2(A.to(dev), c["ta"], B.to(dev), c["tb"], dv(D), out_dtype, sa, sb, dv(bias), c["d"], sb_shape)
    return out.cpu().float(), ref.float()


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_gemm_cases_are_exact(dev, seed):
    rnd = random.Random(seed)
    for case in range(60):
        c = draw(rnd, seed * 1000 + case)
        out, ref = run_case(c, dev)
        if not torch.equal(out, ref):
            d = (out - ref).abs()
            i = d.argmax().item()
            shown = {k: v for k, v in c.items() if k not in ("scalar_values", "tensor1_values")}
            pytest.fail(f"{shown}: {int((d > 0).sum())} elements differ, worst at flat index {i}: "
                        f"{out.flatten()[i].item()} against {ref.flatten()[i].item()}")
