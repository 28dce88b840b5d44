"""GPU parity: the gfx950 library (through its C ABI) against the CPU oracle on identical seeded inputs.

Bars: integer decode (int16 v) and float32 Q bit-exact; float32-output linear within 1e-3 of the float64
decode-then-matmul, measured as max|y - y_ref| / max|y_ref|; bf16 output within one bf16 ulp of bf16(y_ref).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from htr_amd import _native
    _native.lib()          # must load: there is no fallback path
    return torch.device("cuda:0")


def _case(m, n, K, M, seed, dtype=torch.bfloat16):
    from htr_amd import wire
    qw, sc, su, sv = wire.synth_linear(m, n, K, seed)
    x = wire.synth_activation(M, n, seed + 7, dtype)
    return qw, sc, su, sv, x


def _ref(oracle, qw, sc, su, sv, x, bias=None):
    return oracle.c_linear(x.float().numpy(), qw.numpy(), sc.numpy(), su.numpy(), sv.numpy(),
                           None if bias is None else bias.float().numpy().astype(np.float64))


def _rel(y, ref):
    return float(np.abs(y - ref).max() / np.abs(ref).max())


@pytest.mark.parametrize("K", [2, 3, 4, 5, 6, 7, 8])
def test_decode_raw_bit_exact(dev, oracle, K):
    from htr_amd import ops, wire
    print(f"decode_raw K={K}", flush=True)
    qw = wire.synth_linear(256, 384, K, 100 + K)[0]
    got = ops.decode_raw(qw.to(dev)).cpu().numpy()
    assert np.array_equal(got, oracle.c_decode_raw(qw.numpy()))


@pytest.mark.parametrize("K", [2, 3, 4, 5])
def test_decode_raw_edge_streams(dev, oracle, K):
    from htr_amd import ops
    print(f"decode_raw edges K={K}", flush=True)
    zeros = torch.zeros(3, 5, 8 * K, dtype=torch.int32)
    ones = torch.full((3, 5, 8 * K), -1, dtype=torch.int32)
    assert torch.all(ops.decode_raw(zeros.to(dev)) == -303)
    assert torch.all(ops.decode_raw(ones.to(dev)) == -16)
    # one set bit anywhere in the stream, including the wrap region at both ends
    words = torch.zeros(256 * K, 8 * K, dtype=torch.int64)
    for p in range(256 * K):
        words[p, p >> 5] = 1 << (31 - (p & 31))
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32).reshape(256 * K, 1, 8 * K)
    got = ops.decode_raw(words.to(dev)).cpu().numpy()
    assert np.array_equal(got, oracle.c_decode_raw(words.numpy()))


@pytest.mark.parametrize("K", [2, 3, 4, 5, 8])
def test_dequant_q_bit_exact(dev, oracle, K):
    from htr_amd import ops, wire
    print(f"dequant_q K={K}", flush=True)
    qw, sc, _, _ = wire.synth_linear(256, 512, K, 200 + K)
    got = ops.dequant_q(qw.to(dev), sc.to(dev)).cpu().numpy()
    want = oracle.c_dequant_q(qw.numpy(), sc.numpy())
    assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape", [(384, 256), (128, 128), (128, 640), (768, 128)])
@pytest.mark.parametrize("K", [2, 3, 4, 5, 7])
def test_dequant_w_original_basis(dev, oracle, K, shape):
    from htr_amd import ops, wire
    m, n = shape
    print(f"dequant_w K={K} {m}x{n}", flush=True)
    qw, sc, su, sv = wire.synth_linear(m, n, K, 300 + K + m)
    got = ops.dequant_w(*[t.to(dev) for t in (qw, sc, su, sv)])
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (m, n)
    ref = torch.from_numpy(oracle.c_dequant_w(qw.numpy(), sc.numpy(), su.numpy(), sv.numpy()))      # float64
    g = got.float().cpu().double()
    # bf16 rounding (2^-9 relative) of a value computed with float32 butterflies (error ~1e-6 of the block's scale)
    assert float((g - ref).abs().max()) <= float(ref.abs().max()) * 2.0 ** -8
    err = (g - ref).abs()
    assert bool(torch.all(err <= ref.abs() * 2.0 ** -8 + float(ref.abs().max()) * 4e-6))
    # orthogonal rotations preserve the Frobenius norm of Q
    Q = torch.from_numpy(oracle.c_dequant_q(qw.numpy(), sc.numpy())).double()
    assert abs(float(g.norm() / Q.norm()) - 1.0) < 2e-3


def test_prefill_path_dequant_then_gemm(dev, oracle):
    from htr_amd import ops
    print("prefill M=160", flush=True)
    qw, sc, su, sv, x = _case(512, 384, 4, 160, 808)
    bias = torch.randn(512, generator=torch.Generator().manual_seed(2)).bfloat16()
    assert 160 > ops.fused_max_rows(512, 384)
    y = ops.linear(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)], bias.to(dev))
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (160, 512)
    ref = _ref(oracle, qw, sc, su, sv, x, bias)
    # bf16 weights and bf16 output: compare at bf16 resolution of the largest magnitudes
    assert _rel(y.float().cpu().numpy(), ref) <= 2.0 ** -6


def test_reference_env_knobs(dev, oracle, monkeypatch):
    """The reference's HTR_PREFILL = "rot" (rotated-basis GEMM, htr/ops.py:52-54, 101-104) and HTR_GEMV_MAX_M (rows per
    decode launch, htr/ops.py:48) as module settings: same results as the default paths."""
    from htr_amd import ops
    print("env knobs: prefill rot, rows per launch", flush=True)
    qw, sc, su, sv, x = _case(512, 384, 4, 160, 809)
    bias = torch.randn(512, generator=torch.Generator().manual_seed(3)).bfloat16()
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    ref = _ref(oracle, qw, sc, su, sv, x, bias)
    monkeypatch.setattr(ops, "PREFILL", "rot")
    y = ops.linear(x.to(dev), *d, bias.to(dev))
    assert y.dtype == torch.bfloat16 and _rel(y.float().cpu().numpy(), ref) <= 2.0 ** -7      # float32 inside, bf16 out
    monkeypatch.setattr(ops, "PREFILL", "nope")
    with pytest.raises(RuntimeError, match="HTR_PREFILL"):
        ops.linear(x.to(dev), *d)
    monkeypatch.setattr(ops, "PREFILL", "w")
    y_one = ops.linear_f32out(x[:24].to(dev), *d).cpu().numpy()
    monkeypatch.setattr(ops, "LAUNCH_MAX_M", 8)                   # three launches of 8 rows, as the reference would
    y_cut = ops.linear_f32out(x[:24].to(dev), *d).cpu().numpy()
    r24 = _ref(oracle, qw, sc, su, sv, x[:24])
    assert _rel(y_one, r24) <= REL_TOL and _rel(y_cut, r24) <= REL_TOL


@pytest.mark.parametrize("K", [2, 3, 4, 5])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("shape", [(256, 384), (1024, 4096), (4096, 1024)])
def test_linear_f32_out_within_tolerance(dev, oracle, K, M, shape):
    from htr_amd import ops
    m, n = shape
    print(f"linear f32 K={K} M={M} {m}x{n}", flush=True)
    qw, sc, su, sv, x = _case(m, n, K, M, 1000 * K + 10 * M + m % 7)
    y = ops.linear_f32out(x.to(dev), qw.to(dev), sc.to(dev), su.to(dev), sv.to(dev)).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert y.shape == ref.shape
    assert _rel(y, ref) <= REL_TOL, _rel(y, ref)


@pytest.mark.parametrize("K,M", [(3, 16), (4, 9), (4, 16), (4, 32), (3, 32), (5, 17), (4, 45), (4, 100), (2, 8), (8, 24), (4, 6), (4, 7), (4, 64),
                                 (3, 50), (5, 33), (6, 64), (2, 49), (7, 40), (8, 64), (4, 65), (4, 128), (3, 97), (8, 128), (5, 111)])
def test_linear_small_batch_blocks(dev, oracle, K, M, monkeypatch):
    from htr_amd import ops
    print(f"linear batch K={K} M={M}", flush=True)
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", 1 << 30)     # the fused launches at every M, also past the prefill switch
    qw, sc, su, sv, x = _case(512, 1024, K, M, 31 * K + M)
    y = ops.linear_f32out(x.to(dev), qw.to(dev), sc.to(dev), su.to(dev), sv.to(dev)).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert _rel(y, ref) <= REL_TOL, _rel(y, ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_linear_api_dtypes_bias_and_batch_dims(dev, oracle, dtype):
    from htr_amd import ops
    print(f"linear api dtype={dtype}", flush=True)
    qw, sc, su, sv, x = _case(384, 256, 4, 6, 77, dtype)
    bias = torch.randn(384, generator=torch.Generator().manual_seed(5)).to(dtype)
    x3 = x.reshape(2, 3, 256)
    y = ops.linear(x3.to(dev), qw.to(dev), sc.to(dev), su.to(dev), sv.to(dev), bias.to(dev))
    assert y.dtype == dtype and tuple(y.shape) == (2, 3, 384)
    ref = _ref(oracle, qw, sc, su, sv, x, bias)
    got = y.float().cpu().numpy().reshape(6, 384)
    if dtype == torch.float32:
        assert _rel(got, ref) <= REL_TOL
    else:
        want = torch.from_numpy(ref).to(dtype)
        # one ulp of the output type around the rounded reference, plus the fp32-path tolerance
        ulp = (torch.nextafter(want.float().abs().to(dtype), torch.tensor(float("inf"), dtype=dtype)).float()
               - want.float().abs())
        err = (torch.from_numpy(got) - want.float()).abs()
        slack = REL_TOL * float(np.abs(ref).max())
        assert bool(torch.all(err <= ulp + slack))


def test_bf16_output_within_one_ulp(dev, oracle):
    from htr_amd import ops
    print("linear bf16 ulp", flush=True)
    qw, sc, su, sv, x = _case(1024, 2048, 4, 1, 4242)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    y = ops.linear(x.to(dev), *d).float().cpu()
    y32 = ops.linear_f32out(x.to(dev), *d).cpu()
    assert torch.equal(y, y32.bfloat16().float())            # the cast is round-to-nearest-even of the f32 result
    ref = torch.from_numpy(_ref(oracle, qw, sc, su, sv, x)).float()
    want = ref.bfloat16().float()
    # the f32 result carries up to REL_TOL * max|ref| of error (measured 2e-4), so "one bf16 ulp of bf16(y_ref)" can only
    # hold where an ulp is larger than that: elements above 1/8 of the largest magnitude
    big = ref.abs() >= 0.125 * ref.abs().max()
    ulp = torch.maximum(want.abs(), ref.abs()) * 2.0 ** -7
    assert int(big.sum()) > 20
    assert bool(torch.all((y - want).abs()[big] <= ulp[big]))
    assert float((y - ref).abs().max()) <= float(ref.abs().max()) * (2.0 ** -8 + REL_TOL)


def test_large_activations_do_not_overflow(dev, oracle):
    from htr_amd import ops
    print("linear large activations", flush=True)
    qw, sc, su, sv, x = _case(256, 512, 4, 2, 99, torch.float32)
    x = x * 1e4
    x[1] *= 1e-9                                            # one huge row, one tiny row
    y = ops.linear_f32out(x.to(dev), qw.to(dev), sc.to(dev), su.to(dev), sv.to(dev)).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert np.all(np.isfinite(y))
    for r in range(2):
        assert _rel(y[r], ref[r]) <= REL_TOL


@pytest.mark.parametrize("M,chunk", [(8, 16), (5, 11), (3, 32), (8, 9), (2, 20)])
def test_workgroups_rotate_many_blocks_themselves(dev, oracle, M, chunk, monkeypatch):
    """Up to 8 rows over long chunks: more than 32 and at most 128 (row, block) pairs per workgroup are rotated inside the
    kernel in several passes, no separate rotation launch.  Rows of very different magnitude (a huge one, a tiny one, a
    zero one, one whose blocks differ by 2^30) take the per-block scales of every pass."""
    import ctypes
    from htr_amd import _native, ops
    print(f"in-kernel rotation, several passes M={M} chunk={chunk}", flush=True)
    m, n = 1024, 4096
    out = (ctypes.c_int * 6)()
    assert _native.lib().htr_linear_plan(m, n, 4, M, chunk, out) == 0
    assert out[4] == 0 and 32 < M * out[3] <= 128                       # not pre-rotated, more than one pass
    qw, sc, su, sv, x = _case(m, n, 4, M, 3100 + M, torch.bfloat16)
    x = x.float()
    x[0] *= 2.0 ** 20
    x[1] *= 2.0 ** -22
    if M > 2:
        x[2] = 0.0
    if M > 3:
        x[3, 1024:2048] *= 2.0 ** 30
    x = x.bfloat16()
    monkeypatch.setattr(ops, "NSPLIT", chunk)
    y = ops.linear_f32out(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)]).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert np.all(np.isfinite(y))
    for r in range(M):
        if r == 2:
            assert not np.any(y[r])
        else:
            assert _rel(y[r], ref[r]) <= REL_TOL, (r, _rel(y[r], ref[r]))


@pytest.mark.parametrize("M", [1, 3, 9])
def test_zero_tiny_and_non_finite_activations(dev, oracle, M):
    """All-zero rows give exactly the bias, rows of 1e-30 keep their relative accuracy, and an infinity or a NaN in a
    row stays in that row (every output of it non-finite) without touching the other rows."""
    from htr_amd import ops
    print(f"linear zero / tiny / inf rows M={M}", flush=True)
    qw, sc, su, sv, x = _case(256, 384, 4, M, 123 + M, torch.float32)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    bias = torch.randn(256, generator=torch.Generator().manual_seed(3))
    z = ops.linear_f32out(torch.zeros_like(x).to(dev), *d, bias.to(dev)).cpu()
    assert torch.equal(z, bias.expand(M, 256))
    tiny = x * 1e-30
    y = ops.linear_f32out(tiny.to(dev), *d).cpu().numpy()
    assert _rel(y, _ref(oracle, qw, sc, su, sv, tiny)) <= REL_TOL
    for bad in (float("inf"), float("nan")):
        xb = x.clone()
        xb[M - 1, 17] = bad
        yb = ops.linear_f32out(xb.to(dev), *d).cpu().numpy()
        assert not np.any(np.isfinite(yb[M - 1]))
        if M > 1:
            ref = _ref(oracle, qw, sc, su, sv, x)
            assert _rel(yb[:M - 1], ref[:M - 1]) <= REL_TOL


def test_zero_rows_and_repeatability(dev):
    from htr_amd import ops
    print("linear M=0 / repeat", flush=True)
    qw, sc, su, sv, x = _case(512, 512, 4, 4, 5)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    assert tuple(ops.linear(x[:0].to(dev), *d).shape) == (0, 512)
    xs = x.to(dev)
    a = ops.linear_f32out(xs, *d)
    for _ in range(5):                                     # counters reset themselves; result is deterministic
        assert torch.equal(a, ops.linear_f32out(xs, *d))


def test_errors(dev):
    from htr_amd import ops
    qw, sc, su, sv, x = _case(256, 256, 4, 1, 6)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    with pytest.raises(RuntimeError):
        ops.linear(x.to(dev)[:, :128].contiguous(), *d)
    with pytest.raises(RuntimeError):
        ops.linear(x.to(dev), d[0], d[1].float(), d[2], d[3])
    with pytest.raises(RuntimeError):
        ops.linear(x.to(dev), d[0][:, :, :8].contiguous(), d[1], d[2], d[3])      # K = 1


_WEIGHTS = {}


def _weights(m, n, K, seed):
    """Synthetic HTR-W1 tensors of a full-size case, generated once per (shape, K) and shared by its row counts."""
    from htr_amd import wire
    key = (m, n, K, seed)
    if key not in _WEIGHTS:
        _WEIGHTS.clear()                                   # one full-size weight at a time in host memory
        _WEIGHTS[key] = wire.synth_linear(m, n, K, seed)
    return _WEIGHTS[key]


# every cell of the bit-width sweep (K2..K5 x {4096x4096, 14336x4096} x 1, 2, 4 rows), the down projection, and the two
# fused matrices of the decoder layer as the benchmark launches them (q/k/v and gate/up concatenated along the output dim)
_FULL = [(K, m, n, M) for K in (2, 3, 4, 5) for (m, n) in ((4096, 4096), (14336, 4096)) for M in (1, 2, 4)]
_FULL += [(4, 4096, 14336, 1), (4, 6144, 4096, 1), (4, 28672, 4096, 1), (4, 1024, 4096, 1)]


@pytest.mark.parametrize("K,m,n,M", _FULL)
def test_full_size_shapes(dev, oracle, K, m, n, M):
    from htr_amd import ops, wire
    print(f"full size K={K} {m}x{n} M={M}", flush=True)
    qw, sc, su, sv = _weights(m, n, K, 20261125 + K)
    x = wire.synth_activation(M, n, 20261125 + K + 7 + M)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    y = ops.linear_f32out(x.to(dev), *d).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    for r in range(M):
        assert _rel(y[r], ref[r]) <= REL_TOL, (r, _rel(y[r], ref[r]))
    # linearity in x, a size-independent property: f(2x) == 2 f(x).  Power-of-two scaling is exact in every operation of
    # the path except where a rotated activation falls below 2^-14 and is rounded on f16's denormal grid (a block keeps
    # scale 1 while its largest rotated value lies in [2^-8, 2^15)): a handful of elements per launch, each off by at
    # most 2^-25.  The product carries the decode's offset (1534 + v) and the offset's share, 1534 * sum(x~) ~ 1e5, is
    # taken off in float32 at the end, so such a change can move that difference by one ulp of 1e5: a few 1e-4 in the
    # first output of a 128-row block, where the output rotation collects what all rows have in common.  Hence a bound
    # of 1e-5 of max|y| (a hundredth of the parity tolerance) instead of bit equality.
    y2 = ops.linear_f32out((x * 2).to(dev), *d).cpu().numpy()
    assert np.abs(y2 - 2 * y).max() <= 1e-5 * np.abs(y).max()
    # scaling by 2^20 moves every block to a scale of its own (products are then summed block by block in float32
    # instead of inside the matrix unit: another rounding order, the same values to float32 accuracy)
    y3 = ops.linear_f32out((x * float(2 ** 20)).to(dev), *d).cpu().numpy()
    assert np.abs(y3 - float(2 ** 20) * y).max() <= 1e-5 * float(2 ** 20) * np.abs(y).max()
    # the bf16 output the benchmark times is the round-to-nearest-even cast of the same float32 result
    yb = ops.linear(x.to(dev), *d)
    assert yb.dtype == torch.bfloat16
    assert torch.equal(yb.float().cpu(), torch.from_numpy(y).bfloat16().float())


# ---- the small-batch GEMM shapes (every cell of K3, K4 x 8, 16, 32 rows x gate/up and down), larger row counts, the
# 64-expert stack and the output head as parity cases
_BATCH = [(K, M, m, n) for K in (3, 4) for (m, n) in ((14336, 4096), (4096, 14336)) for M in (8, 16, 32)]
_BATCH += [(4, 64, 14336, 4096), (4, 48, 4096, 14336), (4, 6, 4096, 4096), (4, 128, 4096, 4096), (4, 100, 14336, 4096)]


@pytest.mark.parametrize("K,M,m,n", _BATCH)
def test_small_batch_gemm_shapes(dev, oracle, K, M, m, n, monkeypatch):
    from htr_amd import ops, wire
    print(f"small-batch K={K} M={M} {m}x{n}", flush=True)
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", 1 << 30)     # the fused kernel at every M
    qw, sc, su, sv = _weights(m, n, K, 4000 + 13 * K)
    x = wire.synth_activation(M, n, 4000 + 13 * K + M)
    y = ops.linear_f32out(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)]).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    for r in range(M):
        assert _rel(y[r], ref[r]) <= REL_TOL, (r, _rel(y[r], ref[r]))


# ---- more than 128 activation rows in one launch: the fused decode -> matrix-unit kernel.  Row counts on both sides of
# the tile edges, both tile heights (96 rows: nsplit bit 20, 128 rows: bit 21; neither: the planner's choice), every K,
# explicit column splits (nsplit = 2^28 + S) including the exchange between splits, and a second call on the same
# workspace (the flags must be back at zero).
_GEMM = [(4, 130, 256, 512, 0, 0), (4, 200, 256, 512, 2, 3), (4, 256, 384, 1024, 4, 3), (4, 300, 256, 512, 1, 3), (4, 257, 1024, 2048, 0, 0),
         (2, 129, 256, 384, 0, 3), (3, 192, 384, 512, 2, 3), (5, 193, 256, 512, 0, 0), (6, 150, 256, 256, 1, 3), (7, 288, 128, 384, 3, 3),
         (8, 161, 256, 512, 0, 3), (4, 1000, 256, 256, 0, 0), (4, 2048, 128, 256, 1, 3), (4, 96, 256, 512, 1, 3), (4, 40, 256, 384, 2, 3),
         (4, 200, 256, 512, 2, 4), (4, 256, 384, 1024, 4, 4), (4, 257, 256, 512, 1, 4), (2, 129, 256, 384, 0, 4), (3, 384, 384, 512, 2, 4),
         (5, 385, 256, 512, 0, 4), (6, 150, 256, 256, 1, 4), (7, 288, 128, 384, 3, 4), (8, 128, 256, 512, 2, 4), (4, 2048, 128, 256, 1, 4)]


@pytest.mark.parametrize("K,M,m,n,S,T", _GEMM)
def test_more_than_128_rows_in_one_launch(dev, oracle, K, M, m, n, S, T):
    import ctypes
    from htr_amd import _native
    print(f"gemm kernel K={K} M={M} {m}x{n} S={S} tile={T}", flush=True)
    L = _native.lib()
    nsplit = ((1 << 28) | S | {0: 0, 3: 1 << 20, 4: 1 << 21}[T]) if (S or T or M <= 128) else 0
    qw, sc, su, sv, x = _case(m, n, K, M, 9000 + 17 * K + M)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    xd = x.to(dev)
    plan = (ctypes.c_int * 6)()
    assert L.htr_linear_plan(m, n, K, M, nsplit, plan) == 0
    heights = {3: (96,), 4: (128,), 0: (96, 128)}[T]
    assert plan[2] in [-(-M // h) for h in heights] and plan[1] == plan[3] * (m // 128) * plan[2]   # row tiles; splits x row blocks x tiles
    if S:
        assert plan[3] == S
    need = L.htr_workspace_bytes(m, n, K, M, nsplit)
    assert need > 0
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    y = torch.full((M, m), float("nan"), dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream

    def call():
        _native.check(L.htr_linear(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), xd.data_ptr(), None,
                                   y.data_ptr(), m, n, K, M, _native.BF16, _native.F32, nsplit, ws.data_ptr(), ws.numel(), st))
        torch.cuda.synchronize()

    call()
    first = y.clone()
    ref = _ref(oracle, qw, sc, su, sv, x)
    got = first.cpu().numpy()
    for r in (0, 95, 96, 127, 128, M // 2, M - 1):
        if r < M:
            assert _rel(got[r], ref[r]) <= REL_TOL, (r, _rel(got[r], ref[r]))
    assert _rel(got, ref) <= REL_TOL
    y.fill_(float("nan"))
    call()
    assert torch.equal(first, y)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_more_than_128_rows_through_ops_with_bias(dev, oracle, dtype, monkeypatch):
    from htr_amd import ops
    print(f"gemm kernel through ops, {dtype}", flush=True)
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", 1 << 30)
    qw, sc, su, sv, x = _case(384, 512, 4, 210, 9100, dtype)
    bias = torch.randn(384, generator=torch.Generator().manual_seed(9)).to(dtype)
    y = ops.linear(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)], bias.to(dev))
    assert y.dtype == dtype and tuple(y.shape) == (210, 384)
    ref = _ref(oracle, qw, sc, su, sv, x, bias)
    tol = REL_TOL if dtype == torch.float32 else 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -9
    assert _rel(y.float().cpu().numpy(), ref) <= tol


def test_fused_row_limit_follows_the_shape(dev, oracle, monkeypatch):
    """ops.linear takes one launch of the fused GEMM kernel, launches of 128 rows or dequantize + GEMM depending on shape
    and row count; all three give the same product."""
    from htr_amd import ops
    big = ops.ONE_LAUNCH
    assert ops.fused_max_rows(4096, 4096) == 384 and ops.fused_max_rows(14336, 4096) == 384 and ops.fused_max_rows(1024, 4096) == 128
    assert ops.fused_max_rows(4096, 14336) == 512 and ops.fused_rows_per_launch(4096, 14336, 512) == big
    assert [ops.fused_rows_per_launch(14336, 4096, M) for M in (1, 128, 129, 384, 385)] == [128, 128, big, big, 0]
    assert [ops.fused_rows_per_launch(4096, 4096, M) for M in (129, 384, 385)] == [big, big, 0]
    assert ops.fused_rows_per_launch(2048, 2048, 129) == 0
    print("gemm kernel at the policy's shape", flush=True)
    qw, sc, su, sv, x = _case(14336, 4096, 4, 192, 9200)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    ref = _ref(oracle, qw, sc, su, sv, x)
    y = ops.linear_f32out(x.to(dev), *d).cpu().numpy()                                # one launch of the GEMM kernel
    assert _rel(y, ref) <= REL_TOL
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", 1 << 30)
    monkeypatch.setattr(ops, "LAUNCH_MAX_M", 128)
    x200 = torch.cat([x, x[:8]])
    y2 = ops.linear_f32out(x200.to(dev), *d).cpu().numpy()                            # 128 + 72 rows, batched kernel
    assert _rel(y2[:192], ref) <= REL_TOL and _rel(y2[192:], ref[:8]) <= REL_TOL
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", None)
    monkeypatch.setattr(ops, "LAUNCH_MAX_M", ops.ONE_LAUNCH)
    y3 = ops.linear(torch.cat([x, x, x[:100]]).to(dev), *d).float().cpu().numpy()     # 484 rows: dequantize + GEMM
    assert _rel(y3[:192], ref) <= 2.0 ** -6


def test_moe_expert_stack_top6_of_64(dev, oracle):
    """64 experts (gate/up 1408x2048, down 2048x1408, K4), top-6 routing of 16 tokens; each active expert is a pair of
    packed linears (the reference has no MoE kernel: docs/ADAPTERS.md:19).  Eight experts are materialised; the routing
    ids are folded onto them so that the composition, token gathering and accumulation are all exercised."""
    from htr_amd import ops, wire
    print("moe expert stack", flush=True)
    E, T, TOP, H, F = 8, 16, 6, 2048, 1408
    g = torch.Generator().manual_seed(20261125 + 5000)
    probs = torch.softmax(torch.randn(T, 64, generator=g), dim=-1)
    w, ids = torch.topk(probs, TOP, dim=-1)
    ids = ids % E
    x = torch.randn(T, H, generator=g).bfloat16()
    experts = []
    for e in range(E):
        gu = wire.synth_linear(2 * F, H, 4, 7000 + e)            # gate and up fused along the output dim (shared su)
        dn = wire.synth_linear(H, F, 4, 7100 + e)
        experts.append((gu, dn))
    y = torch.zeros(T, H, dtype=torch.float32, device=dev)
    y_ref = np.zeros((T, H))
    xd = x.to(dev)
    for e, (gu, dn) in enumerate(experts):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        wt = w[tok, slot]
        gud = [t.to(dev) for t in gu]
        dnd = [t.to(dev) for t in dn]
        h2 = ops.linear_f32out(xd[tok.to(dev)].contiguous(), *gud)
        h = (torch.nn.functional.silu(h2[:, :F]) * h2[:, F:]).bfloat16()
        out = ops.linear_f32out(h.contiguous(), *dnd)
        y.index_add_(0, tok.to(dev), out * wt.to(dev)[:, None])
        # same composition on the CPU oracle, with the same bf16 rounding of the hidden activation
        r2 = oracle.c_linear(x[tok].float().numpy(), *[t.numpy() for t in gu])
        rh = torch.from_numpy(r2).float()
        rh = (torch.nn.functional.silu(rh[:, :F]) * rh[:, F:]).bfloat16().float().numpy()
        ro = oracle.c_linear(rh, *[t.numpy() for t in dn])
        np.add.at(y_ref, tok.numpy(), ro * wt.numpy().astype(np.float64)[:, None])
    got = y.cpu().numpy()
    # two chained linears with a bf16 rounding between them: the first stage's 2e-4 error moves some hidden values by
    # one bf16 ulp, so the end-to-end bar is looser than one linear's
    assert _rel(got, y_ref) <= 4e-3, _rel(got, y_ref)


def test_grouped_launch_matches_single_launches(dev, oracle):
    """Grouped launch against per-problem launches (bit-identical partial order is not promised: compare to the oracle
    and to the single launches within tolerance), ragged row counts including 0 and more than one launch's worth."""
    from htr_amd import ops, wire
    print("grouped launch", flush=True)
    m, n, K = 384, 512, 4
    rows = [3, 0, 1, 16, 40, 7]
    ws = [wire.synth_linear(m, n, K, 900 + i) for i in range(len(rows))]
    xs = [wire.synth_activation(max(r, 1), n, 950 + i)[:r] for i, r in enumerate(rows)]
    bias = [torch.randn(m, generator=torch.Generator().manual_seed(i)).float() if i % 2 else None for i in range(len(rows))]
    # a launch with pre-rotated activations of another shape first: the scratch it leaves in the shared workspace must
    # not be mistaken for partials by the grouped launch (or by the single launches after it)
    big = _case(256, 4096, 4, 24, 123)
    ops.linear_f32out(big[4].to(dev), *[t.to(dev) for t in big[:4]])
    got = ops.linear_grouped([x.to(dev) for x in xs], [tuple(t.to(dev) for t in w) for w in ws],
                             [None if b is None else b.to(dev) for b in bias], out_dtype=torch.float32)
    for i, r in enumerate(rows):
        assert tuple(got[i].shape) == (r, m)
        if r == 0:
            continue
        ref = _ref(oracle, *ws[i], xs[i], bias[i])
        assert _rel(got[i].cpu().numpy(), ref) <= REL_TOL, (i, _rel(got[i].cpu().numpy(), ref))
        one = ops.linear_f32out(xs[i].to(dev), *[t.to(dev) for t in ws[i]], None if bias[i] is None else bias[i].to(dev))
        assert float((one - got[i]).abs().max()) <= 2e-4 * float(one.abs().max())


def test_moe_64_experts_grouped(dev, oracle):
    """The 64-expert configuration, all experts materialised: gate/up 1408x2048 (fused to 2816x2048) and down 2048x1408
    at K4, top-6 routing of 16 tokens with seeded softmax-routed ids; two grouped launches against the per-expert
    composition on the CPU oracle."""
    from htr_amd import ops, wire
    print("moe 64 experts grouped", flush=True)
    E, T, TOP, H, F = 64, 16, 6, 2048, 1408
    g = torch.Generator().manual_seed(20261125 + 5000)
    probs = torch.softmax(torch.randn(T, E, generator=g), dim=-1)
    w, ids = torch.topk(probs, TOP, dim=-1)
    x = torch.randn(T, H, generator=g).bfloat16()
    gate_up = [wire.synth_linear(2 * F, H, 4, 7000 + e) for e in range(E)]
    down = [wire.synth_linear(H, F, 4, 7100 + e) for e in range(E)]
    y = ops.moe_experts(x.to(dev), ids.to(dev), w.to(dev), [tuple(t.to(dev) for t in p) for p in gate_up],
                        [tuple(t.to(dev) for t in p) for p in down]).cpu().numpy()
    y_ref = np.zeros((T, H))
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        r2 = oracle.c_linear(x[tok].float().numpy(), *[t.numpy() for t in gate_up[e]])
        rh = torch.from_numpy(r2).float()
        rh = (torch.nn.functional.silu(rh[:, :F]) * rh[:, F:]).bfloat16().float().numpy()
        ro = oracle.c_linear(rh, *[t.numpy() for t in down[e]])
        np.add.at(y_ref, tok.numpy(), ro * w[tok, slot].numpy().astype(np.float64)[:, None])
    # two chained linears with a bf16 rounding between them (see test_moe_expert_stack_top6_of_64)
    assert _rel(y, y_ref) <= 4e-3, _rel(y, y_ref)


def test_moe_expert_shapes_grouped_per_stage(dev, oracle):
    """The grouped launch at the real expert shapes, each stage on its own at the single-linear bar: gate_up 2816x2048 and
    down 2048x1408 (K4) of three experts with ragged token counts, against the float64 oracle, 1e-3 per linear."""
    from htr_amd import ops, wire
    print("moe expert shapes, per stage", flush=True)
    H, F = 2048, 1408
    rows = [1, 6, 3]
    gate_up = [wire.synth_linear(2 * F, H, 4, 7000 + e) for e in range(3)]
    down = [wire.synth_linear(H, F, 4, 7100 + e) for e in range(3)]
    xs = [wire.synth_activation(r, H, 7200 + e) for e, r in enumerate(rows)]
    hs = [wire.synth_activation(r, F, 7300 + e) for e, r in enumerate(rows)]
    for name, ws, ins in (("gate_up", gate_up, xs), ("down", down, hs)):
        got = ops.linear_grouped([t.to(dev) for t in ins], [tuple(t.to(dev) for t in w) for w in ws], out_dtype=torch.float32)
        for e, r in enumerate(rows):
            ref = _ref(oracle, *ws[e], ins[e])
            assert tuple(got[e].shape) == ref.shape
            assert _rel(got[e].cpu().numpy(), ref) <= REL_TOL, (name, e, _rel(got[e].cpu().numpy(), ref))


def test_reference_encoded_streams_decode_on_the_gpu(dev, oracle):
    """The tensors the reference's own encoder wrote (tests/golden/encode_small.npz: qweight, scales, su, sv and its
    reconstruction What, the objects of tests/test_release.py:53-73 of the reference) through every decode entry point:
    integer decode and float32 Q bit-exact against the oracle; Q rotated back with torch's block-Hadamard products equals
    What bit for bit (as wire.dequant does on the CPU); bf16 W within bf16 rounding of What; x @ What^T within 1e-3."""
    import os
    from htr_amd import ops, wire
    print("reference-encoded streams", flush=True)
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "encode_small.npz"))
    for tag in ("a", "b0", "b1"):
        qw = torch.from_numpy(gold[f"{tag}_qweight"])
        sc = torch.from_numpy(gold[f"{tag}_scales_f16bits"].view(np.float16))
        su, sv = torch.from_numpy(gold[f"{tag}_su"]), torch.from_numpy(gold[f"{tag}_sv"])
        what = gold[f"{tag}_What"]
        m, n = what.shape
        d = [t.to(dev) for t in (qw, sc, su, sv)]
        assert np.array_equal(ops.decode_raw(d[0]).cpu().numpy(), oracle.c_decode_raw(qw.numpy())), tag
        q = ops.dequant_q(d[0], d[1])
        assert np.array_equal(q.cpu().numpy().view(np.uint32), oracle.c_dequant_q(qw.numpy(), sc.numpy()).view(np.uint32)), tag
        # the reference's own order of operations on the device's Q, on the CPU (its matmul is the fixture's)
        qc = q.cpu()
        w = wire.blk_had_cols_T(wire.blk_had_cols_T(qc.T.contiguous()).T.contiguous())
        w = (w * wire.unpack_signs(sv, m)[:, None] * wire.unpack_signs(su, n)[None, :]).contiguous()
        assert np.array_equal(w.numpy(), what), tag
        wb = ops.dequant_w(*d).float().cpu().numpy()
        assert np.all(np.abs(wb - what) <= 2.0 ** -8 * np.abs(what) + 4e-6 * np.abs(what).max()), tag
        for M in (1, 5):
            x = wire.synth_activation(M, n, 4242 + M)
            y = ops.linear_f32out(x.to(dev), *d).cpu().numpy()
            ref = x.float().numpy().astype(np.float64) @ what.astype(np.float64).T
            assert _rel(y, ref) <= REL_TOL, (tag, M, _rel(y, ref))


def test_lm_head_shape(dev, oracle):
    from htr_amd import ops
    print("lm_head 152064x4096", flush=True)
    qw, sc, su, sv, x = _case(152064, 4096, 4, 1, 20261125 + 5001)
    y = ops.linear_f32out(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)]).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert _rel(y, ref) <= REL_TOL, _rel(y, ref)


def test_seeded_sweep_of_shapes_rows_and_widths(dev, oracle, monkeypatch):
    """Forty-eight seeded combinations of output and input size (multiples of 128 up to 2048, so every chunking case
    of the planner: aligned, ragged, chunks across row blocks, a single workgroup), bit width, row count (all three
    kernels: chunked, batched, fused-launch loop), activation type and bias, each against the float64 oracle."""
    from htr_amd import ops
    monkeypatch.setattr(ops, "GEMV_LOOP_MAX", 1 << 30)     # the fused kernels at every M
    rng = np.random.default_rng(20261125)
    worst = 0.0
    for case in range(48):
        m = int(rng.integers(1, 17)) * 128
        n = int(rng.integers(1, 17)) * 128
        K = int(rng.choice([2, 3, 4, 5, 6, 7, 8]))
        M = int(rng.choice([1, 1, 1, 2, 3, 4, 5, 6, 7, 8, 9, 15, 16, 17, 31, 32, 33, 40, 48, 63, 64, 65, 96, 127, 128]))
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        with_bias = bool(rng.integers(0, 2))
        print(f"sweep case {case}: {m}x{n} K={K} M={M} {dtype} bias={with_bias}", flush=True)
        qw, sc, su, sv, x = _case(m, n, K, M, 9000 + case, dtype)
        bias = torch.randn(m, generator=torch.Generator().manual_seed(case)) if with_bias else None
        y = ops.linear_f32out(x.to(dev), qw.to(dev), sc.to(dev), su.to(dev), sv.to(dev),
                              None if bias is None else bias.to(dev)).cpu().numpy()
        ref = _ref(oracle, qw, sc, su, sv, x, bias)
        assert y.shape == ref.shape
        err = _rel(y, ref)
        worst = max(worst, err)
        assert err <= REL_TOL, (case, m, n, K, M, dtype, with_bias, err)
    print(f"sweep worst relative error {worst:.2e}", flush=True)


def test_seeded_random_cases_through_the_c_abi(dev, oracle):
    """120 seeded random problems straight through htr_linear: K 2..8, m up to 2048, n up to 3072, 1..40 rows, library
    plans and explicit chunk lengths, bf16 / f16 activations, all three output types, bias or none, a zero row, a block
    2^14 times larger than its neighbours, tiny and huge magnitudes.  Every case runs twice on one workspace, which must
    come back clean (status word and partial slots zero)."""
    import random
    from htr_amd import _native, wire
    L = _native.lib()
    rng = random.Random(20261125)
    ydts = {0: torch.bfloat16, 1: torch.float16, 2: torch.float32}
    tols = {0: 2.0 ** -8 + REL_TOL, 1: 2.0 ** -11 + REL_TOL, 2: REL_TOL}
    for it in range(120):
        K = rng.choice([2, 3, 4, 4, 4, 5, 6, 7, 8])
        m, n = 128 * rng.randint(1, 16), 128 * rng.randint(1, 24)
        M = rng.choice([1, 1, 2, 3, 4, 5, 6, 7, 8, 8, 9, 12, 16, 17, 31, 40])
        nsplit = rng.randint(1, min((m // 128) * (n // 128), 40)) if M <= 8 and rng.random() < 0.6 else 0
        dt, ydt = rng.choice([torch.bfloat16, torch.float16]), rng.choice([0, 1, 2])
        scale = rng.choice([1.0, 1e-3]) if dt == torch.float16 or ydt == 1 else rng.choice([1.0, 1.0, 3e4, 1e-6])   # inside f16's range
        print(f"random case {it}: K{K} {m}x{n} M{M} nsplit {nsplit} {dt} y{ydt} x{scale}", flush=True)
        need = L.htr_workspace_bytes(m, n, K, M, nsplit)
        if need == 0:
            continue                                                    # no plan for this explicit chunk length
        qw, sc, su, sv = wire.synth_linear(m, n, K, 1000 + it)
        x = (wire.synth_activation(M, n, 2000 + it, torch.float32) * scale).to(dt)
        if M > 2 and rng.random() < 0.5:
            x[1] = 0
        if rng.random() < 0.3 and dt == torch.bfloat16 and ydt != 1:
            x[0, :128] *= 2.0 ** 14
        d = [t.to(dev) for t in (qw, sc, su, sv)]
        xd = x.to(dev)
        y = torch.empty(M, m, dtype=ydts[ydt], device=dev)
        bias = torch.randn(m, generator=torch.Generator().manual_seed(it)).to(ydts[ydt]).to(dev) if rng.random() < 0.5 else None
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)
        for _ in range(2):
            _native.check(L.htr_linear(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), xd.data_ptr(),
                                       None if bias is None else bias.data_ptr(), y.data_ptr(), m, n, K, M,
                                       _native.BF16 if dt == torch.bfloat16 else _native.F16, ydt, nsplit, ws.data_ptr(), ws.numel(),
                                       torch.cuda.current_stream().cuda_stream))
            torch.cuda.synchronize()
        assert int(ws[:4].view(torch.int32)[0]) == 0 and not bool(ws[256:ws.numel() // 2].any()), "workspace not clean"
        ref = oracle.c_linear(x.float().numpy(), qw.numpy(), sc.numpy(), su.numpy(), sv.numpy(),
                              None if bias is None else bias.float().cpu().numpy().astype(np.float64))
        got = y.float().cpu().numpy()
        assert np.all(np.isfinite(got)), it
        for r in range(M):
            den = np.abs(ref[r]).max()
            if den == 0:
                assert not np.any(got[r]), (it, r)
            else:
                assert np.abs(got[r] - ref[r]).max() <= tols[ydt] * den, (it, r, float(np.abs(got[r] - ref[r]).max() / den))


@pytest.mark.parametrize("M,S", [(12, 1), (16, 1), (16, 2), (32, 1), (32, 4), (10, 8)])
def test_batched_kernel_with_explicit_splits(dev, oracle, M, S, monkeypatch):
    """The batched kernel with an explicit number of column splits (nsplit bit 29): one split of 32 column blocks is more
    than a workgroup rotates and keeps by itself, so those cases take the rotation launch and the staged blocks also at
    few rows; the short splits take the in-kernel rotation.  Same result either way."""
    import ctypes
    from htr_amd import _native, ops
    print(f"batched kernel, explicit splits M={M} S={S}", flush=True)
    m, n = 512, 4096
    out = (ctypes.c_int * 6)()
    assert _native.lib().htr_linear_plan(m, n, 4, M, (1 << 29) | S, out) == 0
    cb = out[0]
    assert cb == 32 // S and out[4] == (0 if (M <= 16 and cb <= 16) or cb <= 8 else 1)
    qw, sc, su, sv, x = _case(m, n, 4, M, 5200 + 10 * M + S)
    monkeypatch.setattr(ops, "NSPLIT", (1 << 29) | S)
    y = ops.linear_f32out(x.to(dev), *[t.to(dev) for t in (qw, sc, su, sv)]).cpu().numpy()
    assert _rel(y, _ref(oracle, qw, sc, su, sv, x)) <= REL_TOL


@pytest.mark.parametrize("M,S", [(12, 4), (24, 4), (32, 8), (64, 2), (100, 4), (128, 8)])
def test_batched_kernel_when_the_grid_exceeds_the_compute_units(dev, oracle, M, S, monkeypatch):
    """With a device of fewer compute units than the grid has workgroups (forced through the planner's override), the
    splits of a row block may not wait for each other: the last split finishes every row.  Same results, and with the
    override lifted the same explicit plan goes back to the splits sharing the output side."""
    import ctypes
    from htr_amd import _native, ops
    print(f"batched kernel, grid beyond the CU count M={M} S={S}", flush=True)
    L = _native.lib()
    m, n = 1024, 2048
    qw, sc, su, sv, x = _case(m, n, 4, M, 6100 + 10 * M + S)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    ref = _ref(oracle, qw, sc, su, sv, x)
    out = (ctypes.c_int * 6)()
    monkeypatch.setattr(ops, "NSPLIT", (1 << 29) | S)
    assert L.htr_plan_device_override(8, 160 * 1024) == 0
    try:
        assert L.htr_linear_plan(m, n, 4, M, (1 << 29) | S, out) == 0 and out[1] == 8 * S and out[2] == 0
        ops._NEED.clear()
        y_small = ops.linear_f32out(x.to(dev), *d).cpu().numpy()
    finally:
        assert L.htr_plan_device_override(0, 0) == 0
        ops._NEED.clear()
    assert L.htr_linear_plan(m, n, 4, M, (1 << 29) | S, out) == 0 and out[2] == 1
    y_full = ops.linear_f32out(x.to(dev), *d).cpu().numpy()
    assert _rel(y_small, ref) <= REL_TOL and _rel(y_full, ref) <= REL_TOL
    # the same products either way (the rotation may come from the launch of its own in one and from the workgroups in the other)
    assert np.abs(y_small - y_full).max() <= 2e-4 * np.abs(ref).max()
