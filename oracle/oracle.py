"""CPU oracle for the HTR-W1 packed-linear path.  TEST INFRASTRUCTURE ONLY.

Two restatements of the reference decode live here:

* ``np_*`` functions: numpy, written from docs/FORMAT.md and htr/wire.py of the reference
  (line numbers cited per function).  Slow, literal, used on small inputs.
* ``c_*`` functions: ctypes wrappers over ``libhtr_oracle.so`` (oracle/htr_oracle.c), the
  same algorithm in C with OpenMP, used at sizes where numpy would take minutes and as the
  timed CPU baseline.

The shipped package (htr_amd/) never imports this module.  Only tests/, the smoke check in
__graft_entry__.py and the cpu_baseline leg of bench.py do, and only as the checker.

All functions are pinned by known-answer tests in tests/test_oracle_kat.py that were not
produced by this code: generator/codebook constants from the closed form, the reference
test-suite's string bit-oracle construction (tests/test_release.py:28-38 of the reference),
sign byte 170 (:40-43), Hadamard orthogonality (:45-47), hand-made streams.  The encoder search
(c_viterbi) is pinned by exhaustive search on small trellises, by the stream invariants of the reference's own
test (tests/test_release.py:12-19) and by vectors the reference's function produced (tests/golden/viterbi.npz).
No function here is "parity unpinned".
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhtr_oracle.so")

GEN_A, GEN_B = 0xDF6ADF, 0x34983
L = 16
S = 1 << L


# ----------------------------------------------------------------------------- numpy
def np_gen_values(states):
    """v(s) = bytesum((s*A + B) mod 2^32) - 510.  htr/wire.py:10-13, docs/FORMAT.md:11."""
    x = (np.asarray(states).astype(np.uint64) * np.uint64(GEN_A) + np.uint64(GEN_B)) & np.uint64(0xFFFFFFFF)
    bs = (x & np.uint64(0xFF)) + ((x >> np.uint64(8)) & np.uint64(0xFF)) + \
         ((x >> np.uint64(16)) & np.uint64(0xFF)) + ((x >> np.uint64(24)) & np.uint64(0xFF))
    return bs.astype(np.int64) - 510


def np_rms():
    """sqrt(mean v^2) over all 65536 states in float64.  htr/wire.py:23-24."""
    v = np_gen_values(np.arange(S)).astype(np.float64)
    return math.sqrt(float(np.mean(v * v)))


def np_cbscale():
    """htr/wire.py:28-30."""
    return 1.0 / np_rms()


def np_codebook_f32():
    """cb[s] = float32(v(s) / rms64).  htr/wire.py:19-25."""
    v = np_gen_values(np.arange(S)).astype(np.float64)
    return (v / np_rms()).astype(np.float32)


def np_stream_bits(words):
    """int32 [B, 8K] -> bits [B, 256K], MSB first inside each word.  htr/wire.py:46-51."""
    u = np.asarray(words).astype(np.int64) & 0xFFFFFFFF
    sh = np.arange(31, -1, -1, dtype=np.int64)
    return ((u[:, :, None] >> sh) & 1).reshape(u.shape[0], -1)


def np_unpack_states(words, K):
    """s_t = 16 stream bits ending at bit (t+1)K-1, circular.  htr/wire.py:54-63."""
    bits = np_stream_bits(words)
    NB = 256 * K
    t = np.arange(256)
    pos = ((t[:, None] + 1) * K - 16 + np.arange(16)[None, :]) % NB
    sel = bits[:, pos]
    wts = 1 << np.arange(15, -1, -1, dtype=np.int64)
    return (sel * wts).sum(-1)


def np_pack_states(states, K):
    """[B,256] states -> int32 [B, 8K] (low K bits per step, MSB first).  htr/wire.py:33-43."""
    states = np.asarray(states).astype(np.int64)
    B = states.shape[0]
    b = states & ((1 << K) - 1)
    sh = np.arange(K - 1, -1, -1, dtype=np.int64)
    bits = ((b[:, :, None] >> sh) & 1).reshape(B, 8 * K, 32)
    wsh = np.arange(31, -1, -1, dtype=np.int64)
    words = (bits << wsh).sum(-1)
    return words.astype(np.uint32).view(np.int32)


def np_pack_signs(s):
    """+-1 vector -> uint8, LSB first, bit set = -1.  htr/wire.py:66-69."""
    neg = (np.asarray(s) < 0).astype(np.uint8).reshape(-1, 8)
    return (neg << np.arange(8, dtype=np.uint8)).sum(-1).astype(np.uint8)


def np_unpack_signs(u8, N):
    """htr/wire.py:72-74."""
    bits = (np.asarray(u8, dtype=np.uint8).reshape(-1, 1).astype(np.int64) >> np.arange(8)) & 1
    return (1.0 - 2.0 * bits.reshape(-1)[:N]).astype(np.float32)


def np_hadamard(n=128):
    """Sylvester H_n / sqrt(n), float64 build, float32 result.  htr/wire.py:80-87."""
    h = np.ones((1, 1), dtype=np.float64)
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return (h / math.sqrt(n)).astype(np.float32)


def np_dequant_q(qweight, scales):
    """Q[16ti+r,16tj+c] = cb[s] * float32(scale[16ti+r]).  htr/wire.py:95-102."""
    qweight = np.asarray(qweight)
    mt, nt, W = qweight.shape
    K = W // 8
    st = np_unpack_states(qweight.reshape(-1, W), K)
    cb = np_codebook_f32()
    R = cb[st].reshape(mt, nt, 16, 16).transpose(0, 2, 1, 3).reshape(mt * 16, nt * 16)
    return R * np.asarray(scales).astype(np.float32)[:, None]


def np_decode_v_matrix(qweight):
    """integer v(s) with the placement of np_dequant_q."""
    qweight = np.asarray(qweight)
    mt, nt, W = qweight.shape
    st = np_unpack_states(qweight.reshape(-1, W), W // 8)
    return np_gen_values(st).reshape(mt, nt, 16, 16).transpose(0, 2, 1, 3).reshape(mt * 16, nt * 16).astype(np.int16)


def np_dequant_w(qweight, scales, su8, sv8, dtype=np.float64):
    """W = Sv.Ho.Q.Hi.Su.  htr/wire.py:105-113 (dense block products, in `dtype`)."""
    Q = np_dequant_q(qweight, scales).astype(dtype)
    m, n = Q.shape
    H = np_hadamard(128).astype(np.float64)
    H = (np.sign(H) / math.sqrt(128.0)).astype(dtype)
    su = np_unpack_signs(su8, n).astype(dtype)
    sv = np_unpack_signs(sv8, m).astype(dtype)
    W = (Q.T.reshape(n, m // 128, 128) @ H).reshape(n, m).T      # wire.py:111
    W = (np.ascontiguousarray(W).reshape(m, n // 128, 128) @ H).reshape(m, n)   # wire.py:112
    return W * sv[:, None] * su[None, :]


def np_linear(x, qweight, scales, su8, sv8, bias=None):
    """decode-then-matmul in float64: y = x @ W^T (+ bias).  docs/FORMAT.md:7-8."""
    W = np_dequant_w(qweight, scales, su8, sv8, np.float64)
    y = np.asarray(x, dtype=np.float64) @ W.T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y


# ----------------------------------------------------------------------------- C library
_lib = None


def build(force=False):
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "htr_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libhtr_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.htr_o_gen_value.restype = ctypes.c_int
        _lib.htr_o_gen_value.argtypes = [ctypes.c_uint32]
        for f in ("htr_o_mean_sq", "htr_o_rms", "htr_o_cbscale"):
            getattr(_lib, f).restype = ctypes.c_double
        _lib.htr_o_half_to_float.restype = ctypes.c_float
        _lib.htr_o_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.htr_o_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _words(qweight):
    a = np.ascontiguousarray(np.asarray(qweight), dtype=np.int32)
    return a


def _f16bits(scales):
    return np.ascontiguousarray(np.asarray(scales, dtype=np.float16)).view(np.uint16)


def c_gen_value(s):
    return lib().htr_o_gen_value(int(s))


def c_rms():
    return lib().htr_o_rms()


def c_cbscale():
    return lib().htr_o_cbscale()


def c_codebook_f32():
    cb = np.empty(S, dtype=np.float32)
    lib().htr_o_codebook_f32(_p(cb))
    return cb


def c_unpack_states(words, K, literal=False):
    w = _words(words).reshape(-1, 8 * K)
    out = np.empty((w.shape[0], 256), dtype=np.uint16)
    fn = lib().htr_o_unpack_states_literal if literal else lib().htr_o_unpack_states
    fn(_p(w), ctypes.c_int64(w.shape[0]), ctypes.c_int(K), _p(out))
    return out


def c_pack_states(states, K):
    st = np.ascontiguousarray(np.asarray(states), dtype=np.uint16).reshape(-1, 256)
    out = np.empty((st.shape[0], 8 * K), dtype=np.int32)
    lib().htr_o_pack_states(_p(st), ctypes.c_int64(st.shape[0]), ctypes.c_int(K), _p(out))
    return out


def c_unpack_signs(u8, N):
    u = np.ascontiguousarray(np.asarray(u8, dtype=np.uint8))
    out = np.empty(N, dtype=np.float32)
    lib().htr_o_unpack_signs(_p(u), ctypes.c_int64(N), _p(out))
    return out


def c_pack_signs(s):
    s = np.ascontiguousarray(np.asarray(s, dtype=np.float32))
    out = np.empty(s.size // 8, dtype=np.uint8)
    lib().htr_o_pack_signs(_p(s), ctypes.c_int64(s.size), _p(out))
    return out


def c_hadamard(n=128):
    H = np.empty((n, n), dtype=np.float32)
    lib().htr_o_hadamard(ctypes.c_int(n), _p(H))
    return H


def c_decode_raw(qweight):
    q = _words(qweight)
    K = q.shape[-1] // 8
    nt = q.size // (8 * K)
    out = np.empty((nt, 256), dtype=np.int16)
    lib().htr_o_decode_raw(_p(q), ctypes.c_int64(nt), ctypes.c_int(K), _p(out))
    return out


def c_decode_v_matrix(qweight):
    q = _words(qweight)
    mt, nt, W = q.shape
    out = np.empty((mt * 16, nt * 16), dtype=np.int16)
    lib().htr_o_decode_v_matrix(_p(q), ctypes.c_int(mt), ctypes.c_int(nt), ctypes.c_int(W // 8), _p(out))
    return out


def c_dequant_q(qweight, scales):
    q = _words(qweight)
    mt, nt, W = q.shape
    sc = _f16bits(scales)
    out = np.empty((mt * 16, nt * 16), dtype=np.float32)
    lib().htr_o_dequant_q(_p(q), _p(sc), ctypes.c_int(mt), ctypes.c_int(nt), ctypes.c_int(W // 8), _p(out))
    return out


def c_dequant_w(qweight, scales, su8, sv8, dtype=np.float64):
    q = _words(qweight)
    mt, nt, W = q.shape
    sc = _f16bits(scales)
    su = np.ascontiguousarray(np.asarray(su8, dtype=np.uint8))
    sv = np.ascontiguousarray(np.asarray(sv8, dtype=np.uint8))
    out = np.empty((mt * 16, nt * 16), dtype=dtype)
    fn = lib().htr_o_dequant_w_f64 if dtype == np.float64 else lib().htr_o_dequant_w_f32
    fn(_p(q), _p(sc), _p(su), _p(sv), ctypes.c_int(mt), ctypes.c_int(nt), ctypes.c_int(W // 8), _p(out))
    return out


def c_linear(x, qweight, scales, su8, sv8, bias=None):
    """float64 y[M, m] = sv . Ho(Q . Hi(su . x)) (+bias); x is any float array [M, n]."""
    q = _words(qweight)
    mt, nt, W = q.shape
    sc = _f16bits(scales)
    su = np.ascontiguousarray(np.asarray(su8, dtype=np.uint8))
    sv = np.ascontiguousarray(np.asarray(sv8, dtype=np.uint8))
    xf = np.ascontiguousarray(np.asarray(x, dtype=np.float32)).reshape(-1, nt * 16)
    M = xf.shape[0]
    y = np.empty((M, mt * 16), dtype=np.float64)
    b = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float64))
    lib().htr_o_linear_f64(_p(q), _p(sc), _p(su), _p(sv), ctypes.c_int(mt), ctypes.c_int(nt), ctypes.c_int(W // 8),
                           _p(xf), ctypes.c_int(M), None if b is None else _p(b), _p(y))
    return y


def c_decode_then_matmul_f32(x, qweight, scales, su8, sv8):
    """The timed CPU baseline: decode the whole float32 W, then x @ W^T in float32."""
    W = c_dequant_w(qweight, scales, su8, sv8, dtype=np.float32)
    xf = np.ascontiguousarray(np.asarray(x, dtype=np.float32)).reshape(-1, W.shape[1])
    y = np.empty((xf.shape[0], W.shape[0]), dtype=np.float32)
    lib().htr_o_matmul_xwT_f32(_p(xf), _p(W), ctypes.c_int(xf.shape[0]), ctypes.c_int64(W.shape[0]),
                               ctypes.c_int64(W.shape[1]), _p(y))
    return y


def c_viterbi(x, w, K, cb=None, L=16, tailbite=True):
    """Tail-biting bitshift-trellis Viterbi (htr/reference.py:6-50): x, w float32 [B, T] -> states uint32 [B, T].
    cb: [2^L] float32 state values (default: the RDNA24 codebook, L = 16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    if cb is None:
        cb = c_codebook_f32()
    cb = np.ascontiguousarray(cb, dtype=np.float32)
    assert cb.size == 1 << L and x.shape == w.shape and x.ndim == 2
    B, T = x.shape
    out = np.empty((B, T), dtype=np.uint32)
    f = lib().htr_o_viterbi
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                  ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    rc = f(_p(x), _p(w), _p(cb), L, K, T, B, 1 if tailbite else 0, _p(out))
    assert rc == 0
    return out


def c_num_threads():
    return lib().htr_o_num_threads()


def c_set_num_threads(t):
    lib().htr_o_set_num_threads(ctypes.c_int(int(t)))
