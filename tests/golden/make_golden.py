"""Writes tests/golden/w1_small.npz: small HTR-W1 known-answer vectors.

Nothing here imports the oracle, the package or the reference: expected values are computed from the text of the
reference's docs/FORMAT.md with plain Python integers and strings (the construction of the reference test-suite's
bit oracle, tests/test_release.py:28-38) and explicit numpy matrices.

    python tests/golden/make_golden.py
"""
import math
import os

import numpy as np
import torch

A, B = 0xDF6ADF, 0x34983


def v_of(s):
    x = (s * A + B) % (1 << 32)
    return sum((x >> (8 * i)) & 0xFF for i in range(4)) - 510


def states_of(words_row, k):
    bits = ''.join(format(w & 0xffffffff, '032b') for w in words_row)
    return [int(''.join(bits[(k * (t + 1) - 16 + j) % len(bits)] for j in range(16)), 2) for t in range(256)]


def sylvester(n):
    h = np.ones((1, 1))
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h / math.sqrt(n)


def main():
    rms = math.sqrt(sum(v_of(s) ** 2 for s in range(65536)) / 65536.0)
    H = sylvester(128)
    out = {"rms": np.array([rms])}
    m = n = 128
    for k in (2, 3, 4, 5):
        g = torch.Generator().manual_seed(9000 + k)
        qw = torch.randint(-(2 ** 31), 2 ** 31, (m // 16, n // 16, 8 * k), dtype=torch.int32, generator=g)
        sc = torch.exp(0.25 * torch.randn(m, generator=g)).half()
        su = torch.randint(0, 256, (n // 8,), dtype=torch.uint8, generator=g)
        sv = torch.randint(0, 256, (m // 8,), dtype=torch.uint8, generator=g)
        x = torch.randn(3, n, generator=g).bfloat16()
        tiles = qw.reshape(-1, 8 * k).tolist()
        v = np.array([[v_of(s) for s in states_of(row, k)] for row in tiles], dtype=np.int16)       # [tiles, 256]
        vm = v.reshape(m // 16, n // 16, 16, 16).transpose(0, 2, 1, 3).reshape(m, n)
        cb = (vm.astype(np.float64) / rms).astype(np.float32)
        Q = cb * sc.numpy().astype(np.float32)[:, None]                                               # one f32 multiply
        sgn = lambda u8, N: 1.0 - 2.0 * ((u8.numpy().reshape(-1, 1) >> np.arange(8)) & 1).reshape(-1)[:N]
        W = np.diag(sgn(sv, m)) @ H @ Q.astype(np.float64) @ H @ np.diag(sgn(su, n))
        y = x.float().numpy().astype(np.float64) @ W.T
        out[f"k{k}_qweight"] = qw.numpy()
        out[f"k{k}_scales_f16bits"] = sc.numpy().view(np.uint16)
        out[f"k{k}_su"] = su.numpy()
        out[f"k{k}_sv"] = sv.numpy()
        out[f"k{k}_x_bf16bits"] = x.view(torch.int16).numpy().view(np.uint16)
        out[f"k{k}_v"] = v
        out[f"k{k}_y"] = y
        if k == 4:
            out["k4_Q"] = Q
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "w1_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
