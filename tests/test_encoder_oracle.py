"""Pins of the CPU oracle's encoder search (oracle.c_viterbi; htr/reference.py:6-50 of the reference):
exhaustive search on small trellises (the mathematics), the stream invariants the reference's own test checks
(tests/test_release.py:12-19), and vectors the reference's function produced (tests/golden/viterbi.npz, written by
tests/golden/make_encoder_golden.py)."""
import itertools
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "viterbi.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


@pytest.mark.parametrize("L,K,T", [(6, 2, 5), (6, 3, 4), (8, 4, 3), (5, 1, 7)])
def test_viterbi_without_tailbiting_is_the_global_optimum(oracle, L, K, T):
    rng = np.random.default_rng(100 * L + K)
    S, nb = 1 << L, 1 << K
    cb = rng.standard_normal(S).astype(np.float32)
    x = rng.standard_normal((2, T)).astype(np.float32)
    w = (rng.random((2, T)) + 0.5).astype(np.float32)
    st = oracle.c_viterbi(x, w, K, cb=cb, L=L, tailbite=False)
    for b in range(2):
        best, arg = None, None
        for s0 in range(S):
            for bits in itertools.product(range(nb), repeat=T - 1):
                s, path = s0, [s0]
                for q in bits:
                    s = ((s << K) & (S - 1)) | q
                    path.append(s)
                c = float(np.sum(w[b].astype(np.float64) * (x[b].astype(np.float64) - cb[path].astype(np.float64)) ** 2))
                if best is None or c < best:
                    best, arg = c, path
        got = st[b].tolist()
        assert all(((got[t - 1] << K) & (S - 1)) == (got[t] & ~(nb - 1)) for t in range(1, T))      # a trellis path
        cg = float(np.sum(w[b].astype(np.float64) * (x[b].astype(np.float64) - cb[got].astype(np.float64)) ** 2))
        assert cg <= best * (1 + 1e-5) + 1e-9, (cg, best)
        assert got == arg or abs(cg - best) <= 1e-6 * max(1.0, best)


@pytest.mark.parametrize("K", [2, 3, 4, 5])
def test_viterbi_tailbiting_invariants(oracle, K):
    rng = np.random.default_rng(K)
    x = rng.standard_normal((2, 256)).astype(np.float32)
    w = np.ones((2, 256), dtype=np.float32)
    s = oracle.c_viterbi(x, w, K).astype(np.int64)
    mask = (1 << (16 - K)) - 1
    assert np.array_equal(s[:, 1:] >> K, s[:, :-1] & mask)                  # tests/test_release.py:17
    assert np.array_equal(s[:, 0] >> K, s[:, -1] & mask)                    # :18, the stream is circular
    words = oracle.c_pack_states(s.astype(np.uint16), K)
    assert np.array_equal(oracle.c_unpack_states(words, K), s.astype(np.uint16))          # :19
    # the search is useful: far better than the best memoryless K-bit choice would be impossible, but it must beat
    # a random stream by a wide margin
    cb = oracle.c_codebook_f32()
    err = float(np.mean((x - cb[s]) ** 2))
    rnd = float(np.mean((x - cb[rng.integers(0, 65536, size=s.shape)]) ** 2))
    assert err < 0.5 * rnd and err < {2: 0.12, 3: 0.04, 4: 0.012, 5: 0.004}[K], err


@pytest.mark.parametrize("K", [2, 3, 4, 5])
def test_viterbi_matches_reference_vectors(oracle, gold, K):
    st = oracle.c_viterbi(gold[f"k{K}_x"], gold[f"k{K}_w"], K)
    assert np.array_equal(st.astype(np.uint16), gold[f"k{K}_states"])


def test_viterbi_matches_reference_on_its_own_test_input(oracle, gold):
    x = gold["lin_x"]
    st = oracle.c_viterbi(x, np.ones_like(x), 4)
    assert np.array_equal(st.astype(np.uint16), gold["lin_states"])
