"""Pins the CPU oracle (oracle/) against answers that do not come from the oracle itself.

Sources of the expected values:
* generator / codebook constants: evaluated once by hand from the closed form in the
  reference's docs/FORMAT.md:10-12 and written here as literals;
* stream layout: the string-based bit oracle that the reference's own test-suite uses
  (tests/test_release.py:28-38 of the reference), with the same seeds and generator call;
* sign byte 170 (tests/test_release.py:40-43), Hadamard orthogonality (:45-47), the trellis
  chain invariants (:17-18);
* hand-made streams whose decode is obvious (all zeros, all ones, one set bit).
"""
import math

import numpy as np
import pytest
import torch


# ------------------------------------------------------------------ generator (a1)
V_KAT = {0: -303, 1: -6, 2: -219, 3: -177, 4: 120, 5: -93, 6: -51, 7: -264,
         255: 207, 256: -6, 4095: 314, 65535: -16}


def _bytesum_py(s):
    x = (s * 0xDF6ADF + 0x34983) % (1 << 32)
    return sum((x >> (8 * i)) & 0xFF for i in range(4)) - 510


def test_generator_known_answers(oracle):
    for s, v in V_KAT.items():
        assert oracle.c_gen_value(s) == v
        assert int(oracle.np_gen_values(np.array([s]))[0]) == v
        assert _bytesum_py(s) == v          # the literals themselves follow the closed form


def test_generator_population_statistics(oracle):
    v_np = oracle.np_gen_values(np.arange(65536))
    v_c = np.array([oracle.c_gen_value(s) for s in range(65536)])
    v_py = np.array([_bytesum_py(s) for s in range(65536)])
    assert np.array_equal(v_np, v_py) and np.array_equal(v_c, v_py)
    assert v_py.min() == -486 and v_py.max() == 472
    assert int(v_py.sum()) == -5849
    assert len(np.unique(v_py)) == 887
    assert int((v_py.astype(np.int64) ** 2).sum()) == 1433042863
    # the mod 2^32 wrap is exercised by almost every state
    assert sum(1 for s in range(65536) if s * 0xDF6ADF + 0x34983 >= (1 << 32)) == 65242


# ------------------------------------------------------------------ codebook (a2)
def test_codebook_constants(oracle):
    rms = 147.87325236173743
    assert oracle.c_rms() == rms and oracle.np_rms() == rms
    assert oracle.c_cbscale() == 0.006762548223080488 == oracle.np_cbscale()
    assert np.float32(oracle.c_cbscale()) == np.float32(0.006762548349797726)
    want = np.array([-2.0490520000457764, -0.040575288236141205, -1.4809980392456055,
                     -1.19697105884552, 0.8115057945251465], dtype=np.float32)
    for cb in (oracle.c_codebook_f32(), oracle.np_codebook_f32()):
        assert cb.dtype == np.float32 and cb.shape == (65536,)
        assert np.array_equal(cb[:5], want)
    assert np.array_equal(oracle.c_codebook_f32(), oracle.np_codebook_f32())
    # unit gain: rms of the codebook over all states is 1
    cb = oracle.c_codebook_f32().astype(np.float64)
    assert abs(math.sqrt(np.mean(cb * cb)) - 1.0) < 1e-7


# ------------------------------------------------------------------ stream layout (a3-a5)
def _string_oracle(words, k):
    expected = []
    for row in words.tolist():
        bits = ''.join(format(w & 0xffffffff, '032b') for w in row)
        expected.append([int(''.join(bits[(k * (t + 1) - 16 + j) % len(bits)] for j in range(16)), 2)
                         for t in range(256)])
    return np.array(expected, dtype=np.int64)


@pytest.mark.parametrize("k", [2, 3, 4, 5, 6, 7, 8])
def test_unpack_states_matches_string_bit_oracle(oracle, k):
    g = torch.Generator().manual_seed(k)
    words = torch.randint(-(2 ** 31), 2 ** 31, (2, 8 * k), dtype=torch.int32, generator=g)
    want = _string_oracle(words, k)
    w = words.numpy()
    assert np.array_equal(oracle.np_unpack_states(w, k), want)
    assert np.array_equal(oracle.c_unpack_states(w, k, literal=True).astype(np.int64), want)
    assert np.array_equal(oracle.c_unpack_states(w, k, literal=False).astype(np.int64), want)
    # round trip (tests/test_release.py:38 of the reference)
    assert np.array_equal(oracle.np_pack_states(want, k), w)
    assert np.array_equal(oracle.c_pack_states(want, k), w)


@pytest.mark.parametrize("k", [2, 3, 4, 5])
def test_trellis_chain_invariants(oracle, k):
    rng = np.random.default_rng(100 + k)
    w = rng.integers(-2 ** 31, 2 ** 31, size=(64, 8 * k), dtype=np.int64).astype(np.int32)
    s = oracle.c_unpack_states(w, k).astype(np.int64)
    lowmask = (1 << (16 - k)) - 1
    assert np.array_equal(s[:, 1:] >> k, s[:, :-1] & lowmask)
    assert np.array_equal(s[:, 0] >> k, s[:, -1] & lowmask)        # tail-biting wrap
    assert np.array_equal(s, oracle.np_unpack_states(w, k))


@pytest.mark.parametrize("k", [2, 3, 4, 5])
def test_hand_made_streams(oracle, k):
    zeros = np.zeros((1, 8 * k), dtype=np.int32)
    ones = np.full((1, 8 * k), -1, dtype=np.int32)
    assert np.all(oracle.c_decode_raw(zeros) == -303)             # state 0
    assert np.all(oracle.c_decode_raw(ones) == -16)               # state 65535
    # one set bit at stream position p is seen by the steps whose window covers p, at a
    # position that moves up by k bits per step
    for p in (0, 5, 17, 32 * k + 3, 256 * k - 1):
        w = np.zeros((1, 8 * k), dtype=np.uint32)
        w[0, p >> 5] = np.uint32(1) << np.uint32(31 - (p & 31))
        st = oracle.c_unpack_states(w.view(np.int32), k)[0].astype(np.int64)
        for t in range(256):
            end = (t + 1) * k - 1                                 # last bit of b_t
            d = (end - p) % (256 * k)                             # distance from p up to the window end
            want = (1 << d) if d < 16 else 0
            assert st[t] == want, (k, p, t)


# ------------------------------------------------------------------ signs (a6)
def test_sign_convention(oracle):
    signs = np.array([1., -1., 1., -1., 1., -1., 1., -1.], dtype=np.float32)
    assert oracle.np_pack_signs(signs).tolist() == [170]
    assert oracle.c_pack_signs(signs).tolist() == [170]
    assert np.array_equal(oracle.np_unpack_signs(np.array([170], dtype=np.uint8), 8), signs)
    assert np.array_equal(oracle.c_unpack_signs(np.array([170], dtype=np.uint8), 8), signs)
    rng = np.random.default_rng(3)
    u = rng.integers(0, 256, size=64, dtype=np.uint8)
    assert np.array_equal(oracle.c_pack_signs(oracle.c_unpack_signs(u, 512)), u)
    assert np.array_equal(oracle.np_unpack_signs(u, 512), oracle.c_unpack_signs(u, 512))


# ------------------------------------------------------------------ H128 (a7)
def test_hadamard(oracle):
    for H in (oracle.np_hadamard(128), oracle.c_hadamard(128)):
        assert H.dtype == np.float32
        assert np.allclose(H @ H.T, np.eye(128), atol=2e-6)       # tests/test_release.py:45-47
        assert np.array_equal(H, H.T)
        assert np.all(np.abs(H) == np.float32(1.0 / math.sqrt(128.0)))
        assert np.all(H[0] > 0) and np.all(H[:, 0] > 0)
        assert H[1, 1] < 0 and H[2, 1] > 0 and H[3, 3] > 0 and H[127, 127] < 0
    assert np.array_equal(oracle.np_hadamard(128), oracle.c_hadamard(128))


# ------------------------------------------------------------------ Q placement (a8)
def _rand_layer(rng, m, n, k):
    qw = rng.integers(-2 ** 31, 2 ** 31, size=(m // 16, n // 16, 8 * k), dtype=np.int64).astype(np.int32)
    sc = np.exp(0.25 * rng.standard_normal(m)).astype(np.float16)
    su = rng.integers(0, 256, size=n // 8, dtype=np.uint8)
    sv = rng.integers(0, 256, size=m // 8, dtype=np.uint8)
    return qw, sc, su, sv


@pytest.mark.parametrize("k", [2, 3, 4, 5])
def test_dequant_q_brute_force_placement(oracle, k):
    rng = np.random.default_rng(k)
    qw, sc, _, _ = _rand_layer(rng, 128, 256, k)
    Qc = oracle.c_dequant_q(qw, sc)
    Qn = oracle.np_dequant_q(qw, sc)
    assert Qc.dtype == np.float32 and np.array_equal(Qc, Qn)
    Vc = oracle.c_decode_v_matrix(qw)
    assert np.array_equal(Vc, oracle.np_decode_v_matrix(qw))
    rms = 147.87325236173743
    # element-by-element from the format text, through the string oracle
    for ti, tj in ((0, 0), (3, 7), (7, 15)):
        st = _string_oracle(torch.from_numpy(qw[ti, tj][None]), k)[0]
        for r in (0, 5, 15):
            for c in (0, 9, 15):
                s = int(st[16 * r + c])
                v = _bytesum_py(s)
                assert Vc[16 * ti + r, 16 * tj + c] == v
                want = np.float32(np.float32(v / rms) * np.float32(sc[16 * ti + r]))
                assert Qc[16 * ti + r, 16 * tj + c] == want
    raw = oracle.c_decode_raw(qw)
    assert np.array_equal(raw.reshape(8, 16, 16, 16).transpose(0, 2, 1, 3).reshape(128, 256), Vc)


# ------------------------------------------------------------------ W and y (a9, a10)
def test_dequant_w_special_case_outer_product(oracle):
    """su = sv = +1 and Q a single non-zero entry => W = q * (row of Ho)^T (row of Hi)."""
    k = 4
    qw = np.zeros((8, 8, 32), dtype=np.int32)
    sc = np.ones(128, dtype=np.float16)
    su = np.zeros(16, dtype=np.uint8)
    sv = np.zeros(16, dtype=np.uint8)
    W = oracle.c_dequant_w(qw, sc, su, sv)
    # all states 0 => Q constant c0 => W = c0 * 128 * e0 e0^T (Hadamard of a constant vector)
    c0 = float(np.float32(-303 / 147.87325236173743))
    want = np.zeros((128, 128))
    want[0, 0] = c0 * 128.0
    assert np.allclose(W, want, atol=1e-9 * abs(c0) * 128)
    assert np.allclose(oracle.np_dequant_w(qw, sc, su, sv), want, atol=1e-9 * abs(c0) * 128)


@pytest.mark.parametrize("k", [3, 4])
def test_linear_factorised_equals_decode_then_matmul(oracle, k):
    rng = np.random.default_rng(40 + k)
    qw, sc, su, sv = _rand_layer(rng, 256, 384, k)
    x = rng.standard_normal((3, 384)).astype(np.float32)
    bias = rng.standard_normal(256)
    Wn = oracle.np_dequant_w(qw, sc, su, sv)
    Wc = oracle.c_dequant_w(qw, sc, su, sv)
    assert np.allclose(Wn, Wc, rtol=0, atol=1e-12 * np.abs(Wn).max() * 128)
    y_direct = x.astype(np.float64) @ Wn.T + bias[None]
    y_fact = oracle.c_linear(x, qw, sc, su, sv, bias)
    assert np.allclose(y_fact, y_direct, rtol=0, atol=1e-11 * np.abs(y_direct).max())
    assert np.allclose(oracle.np_linear(x, qw, sc, su, sv, bias), y_direct)
    # float32 baseline path stays within float32 rounding of the float64 one
    y32 = oracle.c_decode_then_matmul_f32(x, qw, sc, su, sv)
    assert np.abs(y32 - (y_direct - bias[None])).max() < 2e-5 * np.abs(y_direct).max()


def test_w_is_orthogonal_image_of_q(oracle):
    """Both rotations are orthogonal: ||W||_F == ||Q||_F and W W^T has the spectrum of Q Q^T."""
    rng = np.random.default_rng(9)
    qw, sc, su, sv = _rand_layer(rng, 128, 128, 4)
    Q = oracle.c_dequant_q(qw, sc).astype(np.float64)
    W = oracle.c_dequant_w(qw, sc, su, sv)
    assert abs(np.linalg.norm(W) - np.linalg.norm(Q)) < 1e-9 * np.linalg.norm(Q)
    H = np.sign(oracle.c_hadamard(128).astype(np.float64)) / math.sqrt(128)
    Su = np.diag(oracle.c_unpack_signs(su, 128).astype(np.float64))
    Sv = np.diag(oracle.c_unpack_signs(sv, 128).astype(np.float64))
    assert np.allclose(W, Sv @ H @ Q @ H @ Su, atol=1e-10 * np.abs(Q).max() * 128)


def test_half_to_float_all_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().htr_o_half_to_float(int(b)) for b in bits], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_payload_accounting():
    """docs/EVIDENCE.md:36-41 of the reference: W1 payload of a 4096x4096 matrix."""
    from htr_amd import wire
    assert [wire.payload_bytes(4096, 4096, k) for k in (2, 3, 4, 5)] == [4203520, 6300672, 8397824, 10494976]
