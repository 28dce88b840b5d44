"""htr_linear_static: the entry point that uses the library's built-in workspace (no allocation, no workspace argument)
against htr_linear on a caller-owned workspace, through the C ABI: same kernels and plan, so the outputs must be
bit-identical.  Two calls in a row, the second with a smaller input, then a call after a reset."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(L, native, fn, tensors, x, y, m, n, K, M, extra):
    qw, sc, su, sv = tensors
    st = torch.cuda.current_stream().cuda_stream
    rc = fn(qw.data_ptr(), sc.data_ptr(), su.data_ptr(), sv.data_ptr(), x.data_ptr(), None, y.data_ptr(), m, n, K, M,
            native.BF16, native.F32, *extra, st)
    native.check(rc)


def test_static_workspace_entry_matches_htr_linear():
    from htr_amd import _native, wire
    L = _native.lib()
    dev = torch.device("cuda:0")
    K = 4
    for (m, n, M, seed, reset) in [(4096, 4096, 3, 11, 0), (1024, 512, 1, 12, 0), (2048, 1408, 8, 13, 1)]:
        print(f"static entry {m}x{n} M={M} reset={reset}", flush=True)
        tensors = [t.to(dev) for t in wire.synth_linear(m, n, K, 20261125 + seed)]
        x = wire.synth_activation(M, n, seed, torch.bfloat16, dev)
        need = L.htr_workspace_bytes(m, n, K, M, 0)
        assert 0 < need <= _native.STATIC_SCRATCH_BYTES
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)
        y_ref = torch.empty(M, m, dtype=torch.float32, device=dev)
        y = torch.full((M, m), float("nan"), dtype=torch.float32, device=dev)
        _call(L, _native, L.htr_linear, tensors, x, y_ref, m, n, K, M, (0, ws.data_ptr(), ws.numel()))
        _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (reset,))
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), y_ref.cpu().numpy())
    # a problem whose workspace exceeds the built-in one is refused with the workspace status, nothing is launched
    big = L.htr_workspace_bytes(14336, 4096, K, 64, 0)
    assert big > _native.STATIC_SCRATCH_BYTES
    p = ctypes.c_void_p(0x1000)
    assert L.htr_linear_static(p, p, p, p, p, None, p, 14336, 4096, K, 64, _native.BF16, _native.BF16, 0, None) == 6


def test_static_entry_in_a_graph_after_an_eager_warm_up():
    """The address look-up of the built-in workspace happens on the first (eager) call; a call recorded into a HIP
    graph afterwards neither allocates nor looks anything up.  Several replays with eager calls between them."""
    from htr_amd import _native, wire
    L = _native.lib()
    dev = torch.device("cuda:0")
    m, n, K, M = 2048, 4096, 4, 2
    tensors = [t.to(dev) for t in wire.synth_linear(m, n, K, 20261125 + 21)]
    x = wire.synth_activation(M, n, 22, torch.bfloat16, dev)
    ws = torch.zeros(L.htr_workspace_bytes(m, n, K, M, 0), dtype=torch.uint8, device=dev)
    y_ref = torch.empty(M, m, dtype=torch.float32, device=dev)
    y = torch.zeros(M, m, dtype=torch.float32, device=dev)
    _call(L, _native, L.htr_linear, tensors, x, y_ref, m, n, K, M, (0, ws.data_ptr(), ws.numel()))
    _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (0,))          # warm-up: the look-up happens here
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (0,))
    for _ in range(3):
        y.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), y_ref.cpu().numpy())
        _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (0,))      # eager work between the replays
        torch.cuda.synchronize()


def test_static_entry_recovers_with_reset_after_a_give_up():
    """A launch that gives up waiting (the bound forced down to one poll from the host; every kernel still runs to its
    end) leaves the built-in workspace marked: the next call comes out all-NaN, and a call with reset = 1 is right
    again.  Whether a given launch gives up depends on timing, so the protocol is checked whenever it happens."""
    from htr_amd import _native, wire
    L = _native.lib()
    dev = torch.device("cuda:0")
    m, n, K, M = 2048, 4096, 4, 1
    tensors = [t.to(dev) for t in wire.synth_linear(m, n, K, 20261125 + 31)]
    x = wire.synth_activation(M, n, 32, torch.bfloat16, dev)
    ws = torch.zeros(L.htr_workspace_bytes(m, n, K, M, 0), dtype=torch.uint8, device=dev)
    y_ref = torch.empty(M, m, dtype=torch.float32, device=dev)
    y = torch.empty(M, m, dtype=torch.float32, device=dev)
    _call(L, _native, L.htr_linear, tensors, x, y_ref, m, n, K, M, (0, ws.data_ptr(), ws.numel()))
    torch.cuda.synchronize()
    gave_up = 0
    try:
        L.htr_set_spin_limit(1)
        for _ in range(16):
            _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (1,))  # clean array, one poll per wait
            torch.cuda.synchronize()
            if not bool(torch.isnan(y).any()):
                assert np.array_equal(y.cpu().numpy(), y_ref.cpu().numpy())
                continue
            gave_up += 1
            L.htr_set_spin_limit(1 << 20)
            _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (0,))  # stale partials: everything NaN
            torch.cuda.synchronize()
            assert bool(torch.isnan(y).all())
            _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (1,))  # reset: right again
            torch.cuda.synchronize()
            assert np.array_equal(y.cpu().numpy(), y_ref.cpu().numpy())
            L.htr_set_spin_limit(1)
    finally:
        L.htr_set_spin_limit(1 << 20)
    _call(L, _native, L.htr_linear_static, tensors, x, y, m, n, K, M, (1,))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), y_ref.cpu().numpy())
    print(f"static entry: {gave_up} of 16 launches gave up under a one-poll bound", flush=True)
