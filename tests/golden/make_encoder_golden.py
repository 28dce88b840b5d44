"""Writes tests/golden/viterbi.npz and tests/golden/encode_small.npz: input/output vectors of the reference's encoder
search and matrix encoder.

These two functions are the only ones whose outputs nothing else pins: the tail-biting Viterbi is a two-pass heuristic
(its result is not the global optimum, and equal costs are broken by index order), and the matrix encoder chains
torch linear algebra (Cholesky, block inverses) with that search.  So, as an exception, this script imports the
reference's Python (htr/reference.py, htr/wire.py, htr/encode.py; pure torch, CPU) from /root/reference, in the
build container only, and stores what it returns.  The fixtures are data; nothing of the reference travels.

    python tests/golden/make_encoder_golden.py
"""
import os
import sys

import numpy as np
import torch

REF = os.environ.get("HTR_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    sys.path.insert(0, REF)
    from htr import encode, reference, wire          # the reference, read-only
    torch.set_num_threads(4)
    cb = wire.codebook_f32()
    out = {}
    for K in (2, 3, 4, 5):
        g = torch.Generator().manual_seed(4100 + K)
        x = torch.randn(3, 256, generator=g)
        w = torch.rand(3, 256, generator=g) + 0.5
        w = w / w.mean(dim=1, keepdim=True)
        x[2] = 0.0                                    # equal costs everywhere: pins the index order of every argmin
        w[2] = 1.0
        st = reference.viterbi(x, w, cb, K)
        out[f"k{K}_x"] = x.numpy()
        out[f"k{K}_w"] = w.numpy()
        out[f"k{K}_states"] = st.numpy().astype(np.uint16)
    x = torch.linspace(-1, 1, 256)[None]              # the input of tests/test_release.py:14-15
    out["lin_x"] = x.numpy()
    out["lin_states"] = reference.viterbi(x, torch.ones_like(x), cb, 4).numpy().astype(np.uint16)
    np.savez_compressed(os.path.join(HERE, "viterbi.npz"), **out)

    # the matrix of tests/test_release.py:58-64 (seed 12, 128x128, H = I, K4), and one with a real Hessian and two
    # matrices sharing the input signs
    enc = {}
    g = torch.Generator().manual_seed(12)
    w0 = torch.randn(128, 128, generator=g) * 0.02
    r = encode.encode_group([{"W": w0, "H": torch.eye(128)}], 4, max_batch=8)[0]
    enc.update({"a_W": w0.numpy(), "a_qweight": r["qweight"].numpy(), "a_scales_f16bits": r["scales"].numpy().view(np.uint16),
                "a_su": r["su"].numpy(), "a_sv": r["sv"].numpy(), "a_What": r["What"].numpy()})
    g = torch.Generator().manual_seed(77)
    X = torch.randn(512, 256, generator=g) * (1.0 + torch.arange(256) / 128.0)
    H = (X.T @ X) / 512
    jobs = [{"W": torch.randn(128, 256, generator=g) * 0.03, "H": H}, {"W": torch.randn(256, 256, generator=g) * 0.05, "H": H}]
    rs = encode.encode_group(jobs, 3, seed=4321, max_batch=64)
    enc["b_H"] = H.numpy()
    for i, (jb, r) in enumerate(zip(jobs, rs)):
        enc.update({f"b{i}_W": jb["W"].numpy(), f"b{i}_qweight": r["qweight"].numpy(),
                    f"b{i}_scales_f16bits": r["scales"].numpy().view(np.uint16), f"b{i}_su": r["su"].numpy(),
                    f"b{i}_sv": r["sv"].numpy(), f"b{i}_What": r["What"].numpy()})
    np.savez_compressed(os.path.join(HERE, "encode_small.npz"), **enc)
    print("written", {k: v.shape for k, v in {**out, **enc}.items()})


if __name__ == "__main__":
    main()
