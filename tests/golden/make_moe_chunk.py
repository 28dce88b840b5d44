"""Writes tests/golden/moe_L3/c000.pt, c002.pt and PLAN.json: a routed-expert layer in the reference's packed-chunk
layout (htr/moe_encode.py:26-29, 216-225 of the reference: format string, L, K, experts[{e, n, packed{gate, up,
down}{qweight, scales, su, sv}, what_bf16_sha256}]), four tiny experts (F = 128, H = 256, K = 3) in two chunks of two.

The reference ships no such file and its encoder needs a calibration dump and a source checkpoint, so the payload here
is synthetic (seeded random trellis streams, as every 256K-bit string is a valid stream).  The reconstruction hashes
are over the BF16 bits of the float32 decode in the reference's order of operations (htr_amd.wire.dequant, as the
reference's encoder hashes its own float32 reconstruction); the script refuses to write unless the CPU oracle's float64
decode agrees with that decode within 1e-5 of the largest element everywhere and, rounded to BF16, bit for bit in
99 % of the elements (a float32 sum that lands on the other side of a BF16 rounding boundary is the only legitimate
difference).
Agreement with a chunk the reference itself wrote is not pinned by anything in this repository.

    python tests/golden/make_moe_chunk.py
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from htr_amd import wire          # noqa: E402
from oracle import oracle         # noqa: E402

FORMAT = "HTR-W1-P2-PACKED-1"
L, K, F, H, CHUNK = 3, 3, 128, 256, 2
OUT = os.path.join(ROOT, "tests", "golden", "moe_L3")


def checked_sha(t):
    w32 = wire.dequant(*t)
    w64 = torch.from_numpy(oracle.np_dequant_w(*(v.numpy() for v in t)))                 # float64 decode
    assert float((w32.double() - w64).abs().max()) <= 1e-5 * float(w64.abs().max()), "float32 decode is off the float64 oracle"
    got = w32.bfloat16().contiguous()
    same = (got.view(torch.int16) == w64.bfloat16().view(torch.int16)).float().mean()
    assert float(same) >= 0.99, "float32 decode and oracle disagree in more than 1 % of the BF16 elements"
    return hashlib.sha256(got.view(torch.int16).numpy().tobytes()).hexdigest()


def main():
    os.makedirs(os.path.join(OUT, f"L{L}"), exist_ok=True)
    for e0 in (0, 2):
        experts = []
        for e in range(e0, e0 + CHUNK):
            gate = wire.synth_linear(F, H, K, 7000 + 10 * e)
            up = wire.synth_linear(F, H, K, 7001 + 10 * e)
            up = (up[0], up[1], gate[2], up[3])                         # one su per input, as the group encoder draws it
            down = wire.synth_linear(H, F, K, 7002 + 10 * e)
            packed = {r: dict(zip(("qweight", "scales", "su", "sv"), t)) for r, t in (("gate", gate), ("up", up), ("down", down))}
            sha = {r: checked_sha(t) for r, t in (("gate", gate), ("up", up), ("down", down))}
            experts.append({"e": e, "n": 5 * e, "packed": packed, "what_bf16_sha256": sha})
        z = {"format": FORMAT, "L": L, "K": K, "experts": experts, "rows": [], "seconds": 0.0, "verify_seconds": 0.0,
             "decode_check": "float32 wire decode, checked against the float64 oracle", "decode_device": "cpu", "worker": "fixture"}
        torch.save(z, os.path.join(OUT, f"L{L}", f"c{e0:03d}.pt"))
    with open(os.path.join(OUT, "PLAN.json"), "w") as f:
        json.dump({"bits": K, "chunk": CHUNK, "seed": 7000, "damp": 0.01, "dump": "", "src": "", "layers": str(L), "format": FORMAT}, f)


if __name__ == "__main__":
    main()
