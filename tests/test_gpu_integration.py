"""GPU tests of how callers drive the packed linear: HIP-graph capture and replay, tracing through the registered
custom op, and activation pointers that are only 2-byte aligned (which take the separate rotation launch)."""
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
    _native.lib()
    return torch.device("cuda:0")


def _case(m, n, K, M, seed, dtype=torch.bfloat16):
    from htr_amd import wire
    qw, sc, su, sv = wire.synth_linear(m, n, K, seed)
    return qw, sc, su, sv, wire.synth_activation(M, n, seed + 7, dtype)


def _ref(oracle, qw, sc, su, sv, x):
    return oracle.c_linear(x.float().numpy(), qw.numpy(), sc.numpy(), su.numpy(), sv.numpy(), None)


@pytest.mark.parametrize("M", [1, 4, 8, 40])
def test_graph_replays_match_eager(dev, M):
    """One captured call, replayed with new inputs, with eager launches of other shapes between the replays (they share
    the cached workspace): every replay must give what the eager call gives, bit for bit."""
    from htr_amd import ops, wire
    print(f"graph replay M={M}", flush=True)
    qw, sc, su, sv, x = _case(1024, 2048, 4, M, 4100 + M)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    other = [t.to(dev) for t in wire.synth_linear(2048, 1024, 3, 99)]
    x_other = wire.synth_activation(2, 1024, 5).to(dev)
    x_in = x.to(dev).clone()
    ops.linear(x_in, *d)                       # warm-up: workspace allocation happens outside the capture
    ops.linear(x_other, *other)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        y_out = ops.linear(x_in, *d)
    for i in range(4):
        xi = wire.synth_activation(M, 2048, 700 + i).to(dev)
        x_in.copy_(xi)
        ops.linear(x_other, *other)            # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = y_out.clone()
        want = ops.linear(xi, *d)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i}"


def test_custom_op_traces_and_runs(dev, oracle):
    """htr::linear inside a traced function (fake-tensor shape propagation through the registered fake), run on the GPU."""
    from htr_amd import ops
    print("custom op under torch.compile(backend=eager)", flush=True)
    qw, sc, su, sv, x = _case(512, 256, 4, 3, 4200)
    d = [t.to(dev) for t in (qw, sc, su, sv)]

    def f(a):
        return torch.ops.htr.linear(a, d[0], d[1], d[2], d[3], None).float() * 2.0

    fc = torch.compile(f, backend="eager", fullgraph=True)
    y = fc(x.to(dev))
    assert tuple(y.shape) == (3, 512)
    assert torch.equal(y, f(x.to(dev)))
    ref = 2.0 * _ref(oracle, qw, sc, su, sv, x)
    assert float(np.abs(y.cpu().numpy() - ref).max() / np.abs(ref).max()) <= 2.0 ** -7      # bf16 output


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 3, 9])
def test_two_byte_aligned_activations(dev, oracle, dtype, M):
    """x that starts one element into its allocation: only 2-byte aligned, so the in-kernel rotation (dword loads) does
    not apply and the library rotates with its own launch."""
    from htr_amd import ops
    print(f"2-byte aligned x dtype={dtype} M={M}", flush=True)
    qw, sc, su, sv, x = _case(384, 512, 4, M, 4300 + M, dtype)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    buf = torch.zeros(M * 512 + 1, dtype=dtype, device=dev)
    buf[1:].copy_(x.reshape(-1).to(dev))
    xv = buf[1:].view(M, 512)
    assert xv.data_ptr() % 4 == 2 and xv.is_contiguous()
    y = ops.linear_f32out(xv, *d).cpu().numpy()
    ref = _ref(oracle, qw, sc, su, sv, x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= REL_TOL


def test_encode_save_load_plugin_apply(dev, tmp_path):
    """The whole chain on the device: encode two projections over one input with a shared sign vector (GPU search),
    save them as a checkpoint, read it back, place the shards through the plugin's weight loaders into one fused
    module, and run the module: the result is x times the encoder's own reconstruction of the weights."""
    from htr_amd import checkpoint, encode, vllm_plugin as vp
    print("encode -> checkpoint -> plugin loaders -> apply", flush=True)

    class _Linear(vp.LinearBase):
        pass

    g = torch.Generator().manual_seed(77)
    Wg, Wu = torch.randn(256, 256, generator=g) * 0.03, torch.randn(128, 256, generator=g) * 0.03
    A = torch.randn(512, 256, generator=g)
    H = (A.T @ A / 512).to(dev)
    res = encode.encode_group([{"W": Wg.to(dev), "H": H}, {"W": Wu.to(dev), "H": H}], 4, seed=5, shared_su=True, max_batch=4096)
    path = str(tmp_path / "model.safetensors")
    checkpoint.save_linears(path, {"model.layers.0.mlp.gate_proj": tuple(res[0][k] for k in ("qweight", "scales", "su", "sv")),
                                   "model.layers.0.mlp.up_proj": tuple(res[1][k] for k in ("qweight", "scales", "su", "sv"))})
    ck = checkpoint.Checkpoint(path)
    layer = _Linear()
    meth = vp.HTRLinearMethod(4)
    meth.create_weights(layer, 256, [256, 128], 256, 384, torch.bfloat16)
    for sid, name in enumerate(("gate_proj", "up_proj")):
        qw, sc, su, sv = ck.linear(f"model.layers.0.mlp.{name}")
        layer.htr_qweight.weight_loader(layer.htr_qweight, qw, sid)
        layer.htr_scales.weight_loader(layer.htr_scales, sc, sid)
        layer.htr_su.weight_loader(layer.htr_su, su, sid)
        layer.htr_sv.weight_loader(layer.htr_sv, sv, sid)
    for nm in ("htr_qweight", "htr_scales", "htr_su", "htr_sv"):
        getattr(layer, nm).data = getattr(layer, nm).data.to(dev)
    meth.process_weights_after_loading(layer)
    x = torch.randn(5, 256, generator=g).bfloat16()
    y = meth.apply(layer, x.to(dev)).float().cpu()
    What = torch.cat([res[0]["What"], res[1]["What"]]).float().cpu()
    ref = x.float() @ What.T
    assert tuple(y.shape) == (5, 384)
    assert float((y - ref).abs().max() / ref.abs().max()) <= 2.0 ** -7          # bf16 output
    # and the encoding is a faithful one: within a few percent of the dense product
    dense = x.float() @ torch.cat([Wg, Wu]).T
    assert float((ref - dense).norm() / dense.norm()) < 0.2


@pytest.mark.parametrize("Ma,Mb", [(1, 3), (24, 40)])
def test_two_streams_with_their_own_workspaces(dev, Ma, Mb):
    """Launches of two shapes interleaved on two streams (default priority): the Python layer keeps one workspace per
    stream, so the partial slots of concurrent launches never meet; every result equals the serial one.  The second
    case runs the batched kernel on both streams, whose workgroups of one row block wait for each other."""
    from htr_amd import ops
    print(f"two streams M={Ma},{Mb}", flush=True)
    a = _case(1024, 2048, 4, Ma, 4400)
    b = _case(2048, 1024, 3, Mb, 4401)
    da, xa = [t.to(dev) for t in a[:4]], a[4].to(dev)
    db, xb = [t.to(dev) for t in b[:4]], b[4].to(dev)
    want_a, want_b = ops.linear(xa, *da), ops.linear(xb, *db)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(25):
        with torch.cuda.stream(s1):
            outs_a.append(ops.linear(xa, *da))
        with torch.cuda.stream(s2):
            outs_b.append(ops.linear(xb, *db))
    torch.cuda.synchronize()
    assert all(torch.equal(o, want_a) for o in outs_a)
    assert all(torch.equal(o, want_b) for o in outs_b)


@pytest.mark.parametrize("M", [1, 32])
def test_bounded_wait_gives_up_cleanly(dev, oracle, M):
    """The finishing workgroup's wait for the other chunks' partials is bounded (chunked kernel at 1 row; batched kernel
    at 32 rows, where the splits of a row block wait for each other).  With the bound forced down to a single
    poll from the host, a launch either comes out right or marks what it could not finish: NaN for those rows, bit 0
    of the workspace's status word and the host-side flag; every kernel still runs to its end.  The call after a
    failure clears the workspace and raises; the one after that is right again.  Nothing here touches the operator's
    workspace table by hand."""
    from htr_amd import _native, ops
    print(f"bounded wait M={M}", flush=True)
    L = _native.lib()
    qw, sc, su, sv, x = _case(2048, 4096, 4, M, 4500 + M)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    ref = _ref(oracle, qw, sc, su, sv, x)
    xd = x.to(dev)
    good = ops.linear_f32out(xd, *d).cpu().numpy()
    assert float(np.abs(good - ref).max() / np.abs(ref).max()) <= REL_TOL
    torch.cuda.synchronize()
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    gave_up = raised = 0
    pending = False                                          # the previous launch gave up and nobody has been told yet
    try:
        L.htr_set_spin_limit(1)
        for _ in range(24):
            try:
                y = ops.linear_f32out(xd, *d)
            except RuntimeError as e:
                assert pending and "gave up" in str(e)
                pending = False
                raised += 1
                ws = ops._WORKSPACES[key]
                assert int(ws.buf[:4].view(torch.int32)[0]) == 0 and int(ws.flag[0][0]) == 0
                continue
            assert not pending
            torch.cuda.synchronize()
            ws = ops._WORKSPACES[key]
            status = int(ws.buf[:4].view(torch.int32)[0])
            yn = y.cpu().numpy()
            bad = ~np.isfinite(yn)
            assert bool(bad.any()) == bool(status & 1) == bool(ws.flag[0][0])
            blocks = bad.reshape(M, -1, 128)
            assert np.all(blocks.all(axis=2) | ~blocks.any(axis=2))         # whole 128-row blocks, never single values
            ok = ~bad
            assert float(np.abs(yn[ok] - ref[ok]).max() / np.abs(ref).max()) <= REL_TOL if ok.any() else True
            pending = bool(bad.any())
            gave_up += int(pending)
        print(f"gave up {gave_up} times, raised {raised} times", flush=True)
    finally:
        L.htr_set_spin_limit(1 << 20)
    if pending:
        with pytest.raises(RuntimeError):
            ops.linear_f32out(xd, *d)
    again = ops.linear_f32out(xd, *d).cpu().numpy()
    assert np.array_equal(again, good)


def test_stale_workspace_poisons_later_launches(dev):
    """A workspace whose status word is set (an earlier launch gave up) must not be trusted: a launch on it returns NaN
    everywhere instead of summing whatever the slots hold; htr_workspace_init makes it usable again."""
    from htr_amd import _native
    print("stale workspace", flush=True)
    L = _native.lib()
    m, n, K = 1024, 2048, 4
    qw, sc, su, sv, x = _case(m, n, K, 1, 4600)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    xd = x.to(dev)
    need = L.htr_workspace_bytes(m, n, K, 1, 0)
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    y = torch.empty(1, m, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream

    def run():
        _native.check(L.htr_linear(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), xd.data_ptr(), None,
                                   y.data_ptr(), m, n, K, 1, _native.BF16, _native.F32, 0, ws.data_ptr(), ws.numel(), st))
        torch.cuda.synchronize()
        return y.clone()

    good = run()
    assert bool(torch.isfinite(good).all())
    ws[:4].view(torch.int32)[0] = 1
    assert bool(torch.isnan(run()).all())
    _native.check(L.htr_workspace_init(ws.data_ptr(), ws.numel(), None, st))
    assert torch.equal(run(), good)


def test_captures_own_their_workspaces(dev):
    """Each capture records launches against a workspace of its own; a later eager call that needs a much larger
    workspace must neither move nor free it (the graph would replay against freed memory), and two graphs do not share
    partial slots."""
    from htr_amd import ops, wire
    print("capture workspaces", flush=True)
    qw, sc, su, sv, x = _case(1024, 2048, 4, 2, 4700)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    big = [t.to(dev) for t in wire.synth_linear(14336, 4096, 4, 4701)]
    x_in = x.to(dev).clone()
    want = ops.linear(x_in, *d)
    torch.cuda.synchronize()
    g1, g2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1):
        y1 = ops.linear(x_in, *d)
    with torch.cuda.graph(g2):
        y2 = ops.linear(x_in, *d)
    caps = [w for k, w in ops._WORKSPACES.items() if len(k) == 3]
    assert len({w.buf.data_ptr() for w in caps}) >= 2
    x_big = wire.synth_activation(100, 4096, 4702).to(dev)
    ops.linear(x_big, *big)                    # needs tens of MB of workspace: far beyond what the captures hold
    filler = [torch.full((1 << 20,), 255, dtype=torch.uint8, device=dev) for _ in range(8)]    # would land in freed memory
    torch.cuda.synchronize()
    for _ in range(3):
        g1.replay()
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(y1, want) and torch.equal(y2, want)
    del filler


def test_captures_can_share_one_workspace(dev):
    """Opt-in for serving stacks that capture thousands of pieces which replay one after the other: all captures of a
    device use one workspace that exists before they start, so a capture allocates nothing and records no fill kernel.
    A capture that would need more than the shared buffer holds is refused with a clear error (inside the capture
    nothing may be allocated), and a capture's own workspace, in the default mode, is sized to the launch, not to 1 MiB."""
    from htr_amd import ops, wire
    print("shared capture workspace", flush=True)
    qw, sc, su, sv, x = _case(1024, 2048, 4, 1, 4800)
    d = [t.to(dev) for t in (qw, sc, su, sv)]
    d2 = [t.to(dev) for t in wire.synth_linear(2048, 1024, 3, 4801)]
    x1, x2 = x.to(dev).clone(), wire.synth_activation(3, 1024, 4802).to(dev)
    want1, want2 = ops.linear(x1, *d), ops.linear(x2, *d2)
    torch.cuda.synchronize()
    # default mode: one buffer per capture, as large as the launch needs
    g0 = torch.cuda.CUDAGraph()
    before = set(ops._WORKSPACES)
    with torch.cuda.graph(g0):
        y0 = ops.linear(x1, *d)
    own = [ops._WORKSPACES[k] for k in set(ops._WORKSPACES) - before]
    assert len(own) == 1 and own[0].buf.numel() < (1 << 20)
    g0.replay()
    torch.cuda.synchronize()
    assert torch.equal(y0, want1)
    ops.share_capture_workspace(True)
    try:
        ops.linear(x1, *d)
        ops.linear(x2, *d2)                      # the warm-up pass sizes the shared buffer
        torch.cuda.synchronize()
        shared = ops._WORKSPACES[(dev.index, "shared")]
        before = set(ops._WORKSPACES)
        g1, g2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
        with torch.cuda.graph(g1):
            y1 = ops.linear(x1, *d)
        with torch.cuda.graph(g2):
            y2 = ops.linear(x2, *d2)
        assert set(ops._WORKSPACES) == before and ops._WORKSPACES[(dev.index, "shared")] is shared
        for _ in range(3):
            g1.replay()
            g2.replay()
            ops.linear(x2, *d2)                  # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(y1, want1) and torch.equal(y2, want2)
        big = [t.to(dev) for t in wire.synth_linear(14336, 4096, 4, 4803)]
        xb = wire.synth_activation(100, 4096, 4804).to(dev)
        g3 = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="shared capture workspace"):
            with torch.cuda.graph(g3):
                ops.linear(xb, *big)
        torch.cuda.synchronize()
        ops.reserve_capture_workspace(dev, 64 << 20)
        g4 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g4):
            y3 = ops.linear(xb, *big)
        g4.replay()
        g1.replay()                              # the earlier graphs still replay against the buffer they recorded
        torch.cuda.synchronize()
        assert torch.equal(y1, want1)
        assert torch.equal(y3, ops.linear(xb, *big))
    finally:
        ops.share_capture_workspace(False)


def test_packed_expert_chunks_feed_the_grouped_launch(dev, oracle):
    """The committed routed-expert chunks (reference layout, htr/moe_encode.py:216-225; four experts, K3) are read with
    the weights-only loader, fused to gate_up / down lists and run through ops.moe_experts; the result is compared with
    the per-expert composition on the CPU oracle, and every decoded matrix with the oracle's float64 decode."""
    import os
    from htr_amd import checkpoint, ops
    print("packed expert chunks -> moe_experts", flush=True)
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "moe_L3")
    gate_up, down, K = checkpoint.PackedExperts(root).layer(3, device=dev)
    E, T, TOP, H, F = 4, 12, 2, 256, 128
    for e in range(E):
        for t in (gate_up[e], down[e]):
            W = ops.dequant_w(*t).float().cpu().numpy()
            W_ref = oracle.np_dequant_w(*[v.cpu().numpy() for v in t])
            assert np.abs(W - W_ref).max() <= 2.0 ** -8 * np.abs(W_ref).max()          # bf16 output
    g = torch.Generator().manual_seed(31)
    w, ids = torch.topk(torch.softmax(torch.randn(T, E, generator=g), dim=-1), TOP, dim=-1)
    x = torch.randn(T, H, generator=g).bfloat16()
    y = ops.moe_experts(x.to(dev), ids.to(dev), w.to(dev), gate_up, down).cpu().numpy()
    y_ref = np.zeros((T, H))
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        r2 = torch.from_numpy(oracle.c_linear(x[tok].float().numpy(), *[v.cpu().numpy() for v in gate_up[e]])).float()
        rh = (torch.nn.functional.silu(r2[:, :F]) * r2[:, F:]).bfloat16().float().numpy()
        ro = oracle.c_linear(rh, *[v.cpu().numpy() for v in down[e]])
        np.add.at(y_ref, tok.numpy(), ro * w[tok, slot].numpy().astype(np.float64)[:, None])
    rel = np.abs(y - y_ref).max() / np.abs(y_ref).max()
    assert rel <= 4e-3, rel          # two chained linears with a bf16 rounding between them
