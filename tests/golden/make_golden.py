"""Writes the small committed fixtures under tests/golden/ from the C oracle.

Run from the repo root: ``python tests/golden/make_golden.py``.  The fixtures
hold inputs and expected outputs only; the reference's tests store no vectors
(their known answers are inline literals, restated in the tests), so these
pin the oracle against accidental change and travel to the GPU box.
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as o  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    o.build()
    L = o.lib()
    out = {}
    # 256-entry decode tables as fp32 bit patterns
    out["decode_e4m3fn_bits"] = [int(torch.tensor(L.ora_e4m3fn_to_f32(i)).view(torch.int32)) & 0xFFFFFFFF
                                 for i in range(256)]
    out["decode_e5m2_bits"] = [int(torch.tensor(L.ora_e5m2_to_f32(i)).view(torch.int32)) & 0xFFFFFFFF
                               for i in range(256)]
    # encode: every bf16 pattern with exponent in a band around the fp8 ranges would be
    # 64 KiB per format; store a CRC-like digest plus 512 sampled points instead
    g = torch.Generator().manual_seed(0xC001A1)
    bits = torch.randint(0, 65536, (512,), generator=g).to(torch.int32)
    xs = (bits << 16).view(torch.float32)
    out["encode_sample_bf16_bits"] = bits.tolist()
    out["encode_sample_e4m3fn"] = [L.ora_f32_to_e4m3fn(float(v)) if v == v else 0x7F for v in xs.tolist()]
    out["encode_sample_e5m2"] = [L.ora_f32_to_e5m2(float(v)) if v == v else 0x7F for v in xs.tolist()]
    allb = (torch.arange(65536, dtype=torch.int32) << 16).view(torch.float32)
    finite = torch.isfinite(allb)
    for name, fn, mod in (("e4m3fn", L.ora_f32_to_e4m3fn, 2 ** 61 - 1), ("e5m2", L.ora_f32_to_e5m2, 2 ** 61 - 1)):
        acc = 0
        for i, v in enumerate(allb.tolist()):
            if finite[i]:
                acc = (acc * 257 + fn(v) + 1) % mod
        out[f"encode_all_finite_bf16_digest_{name}"] = acc
    # int4 case: 64 x 64, group 16, packed zero points
    q = torch.randint(0, 16, (64, 64), generator=g)
    z = torch.randint(0, 16, (4, 64), generator=g)
    s = (torch.rand(4, 64, generator=g) * 0.019 + 0.001).bfloat16()
    packed, zp = o.pack_nibbles(q), o.pack_nibbles(z)
    du = o.c_dequant_4bit(packed, s, zp, torch.bfloat16, False)
    di = o.c_dequant_4bit(packed, s, None, torch.bfloat16, True)
    out["int4_packed"] = packed.tolist()
    out["int4_zp_packed"] = zp.tolist()
    out["int4_scale_bf16_bits"] = (s.view(torch.int16).to(torch.int32) & 0xFFFF).tolist()
    out["int4_uint4_out_bf16_bits"] = (du.view(torch.int16).to(torch.int32) & 0xFFFF).tolist()
    out["int4_int4_out_bf16_bits"] = (di.view(torch.int16).to(torch.int32) & 0xFFFF).tolist()
    with open(os.path.join(HERE, "oracle_vectors.json"), "w") as f:
        json.dump(out, f)
    print("wrote", os.path.join(HERE, "oracle_vectors.json"))


if __name__ == "__main__":
    main()
