"""CPU-only checks of the boundary: the C ABI library loads and exports what include/htr_gfx950.h declares, argument
validation returns the documented codes before anything touches a GPU, the launch planner is sane, and the Python
operator layer mirrors the reference's htr.ops surface (htr/ops.py:69-122 of the reference)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from htr_amd import _native, build
    if not os.path.exists(_native.LIB_PATH):
        build.build()
    return _native.lib()


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "htr_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(htr_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(L):
    from htr_amd import _native
    names = _declared_functions()
    assert {"htr_linear", "htr_decode_raw", "htr_dequant_q", "htr_workspace_bytes", "htr_linear_plan"} <= set(names)
    for n in names:
        assert hasattr(L, n), n
    assert set(_native.SIGNATURES) == set(names)          # the ctypes table binds exactly the header


def test_constants(L, oracle):
    assert L.htr_abi_version() >= 1
    assert np.float32(L.htr_cbscale()) == np.float32(oracle.c_cbscale())
    from htr_amd import wire
    assert wire.cbscale() == oracle.c_cbscale()
    assert L.htr_strerror(0) == b"ok" and b"K" in L.htr_strerror(2)
    # the batch message names the limits the header declares
    from htr_amd import _native
    msg = L.htr_strerror(4).decode()
    assert f"1..{_native.MAX_BATCH}" in msg and f"1..{_native.MAX_GROUP_ROWS}" in msg
    assert L.htr_workspace_init(None, 1 << 20, None, None) == 1          # NULL workspace: refused before any GPU call
    assert L.htr_workspace_init(256, 64, None, None) == 6                # too small


def test_validation_codes_without_gpu(L):
    from htr_amd import _native
    p = ctypes.c_void_p(0x1000)                # never dereferenced: every case below fails validation first
    ok_ws = ctypes.c_void_p(0x100000)
    call = lambda **kw: L.htr_linear(kw.get("qw", p), p, p, p, p, None, kw.get("y", p), kw.get("m", 256), kw.get("n", 256),
                                     kw.get("K", 4), kw.get("M", 1), kw.get("xd", 0), kw.get("yd", 0), kw.get("ns", 0),
                                     kw.get("ws", ok_ws), kw.get("wsb", 1 << 30), None)
    assert call(qw=None) == 1
    assert call(K=1) == 2 and call(K=9) == 2
    assert call(m=200) == 3 and call(n=0) == 3
    assert call(M=0) == 4 and call(M=_native.MAX_BATCH + 1) == 4
    assert call(M=33, ns=4) == 4               # an explicit chunked plan stops at 32 rows
    assert call(M=129, ns=(1 << 29) | 1) == 4  # an explicit batched plan at 128
    assert call(xd=3) == 5 and call(yd=-1) == 5
    assert call(ws=None) == 6 and call(wsb=16) == 6 and call(ws=ctypes.c_void_p(0x100010)) == 6
    assert call(qw=ctypes.c_void_p(0x1004)) == 7
    assert call(ns=100000) == 9
    assert L.htr_decode_raw(None, p, 8, 4, None) == 1 and L.htr_decode_raw(p, p, 8, 1, None) == 2
    assert L.htr_dequant_q(p, p, None, 8, 8, 4, None) == 1 and L.htr_dequant_q(p, p, p, 0, 8, 4, None) == 3
    assert L.htr_workspace_bytes(256, 256, 9, 1, 0) == 0


@pytest.mark.parametrize("m,n", [(128, 128), (256, 384), (4096, 4096), (1024, 4096), (6144, 4096), (14336, 4096),
                                 (28672, 4096), (4096, 14336), (152064, 4096), (1408, 2048), (2048, 1408)])
@pytest.mark.parametrize("M", [1, 2, 5, 8, 9, 16, 32, 33, 64, 65, 128])
def test_launch_plan_is_consistent(L, m, n, M):
    out = (ctypes.c_int * 6)()
    assert L.htr_linear_plan(m, n, 4, M, 0, out) == 0
    chunk, wgs, segfin, nbl, prerot, lds = list(out)
    nblk, rbs = n // 128, m // 128
    need = L.htr_workspace_bytes(m, n, 4, M, 0)
    assert need >= 256 + wgs * M * 128 * 4                                       # header + one partial slot per workgroup
    batched = M >= 9 or (M >= 6 and m // 128 >= 192)
    if not batched and M >= 7:
        # 7 and 8 rows also take the batched kernel where its splits are at most four column blocks on a full grid and
        # the workgroups rotate their own slices
        forced = (ctypes.c_int * 6)()
        assert L.htr_linear_plan(m, n, 4, M, 1 << 29, forced) == 0
        batched = forced[4] == 0 and forced[0] <= 4 and forced[1] >= 256
    if batched:
        # batched kernel: `chunk` column blocks per split, S = ceil(nblk / chunk) splits per row block, no empty split;
        # activations rotated ahead, except up to 16 rows over at most 16 column blocks per split (32 rows over 8) on a
        # grid of one workgroup per CU, where every workgroup rotates and keeps its own slice (more LDS)
        S = -(-nblk // chunk)
        in_kernel = ((M <= 16 and chunk <= 16) or (M <= 32 and chunk <= 8)) and wgs <= 256
        assert wgs == rbs * S and (S - 1) * chunk < nblk and prerot == (0 if in_kernel else 1)
        assert lds <= (112 if in_kernel else 64 if M <= 32 else 140) * 1024
        assert S <= 8 and (wgs <= 256 or S == 1)                                 # the grid fits the chip, at most 8 splits
        # an explicit split is honoured (bit 29 selects the batched kernel)
        assert L.htr_linear_plan(m, n, 4, M, (1 << 29) | 1, out) == 0 and out[0] == nblk and out[1] == rbs
        return
    assert chunk >= 1 and (wgs - 1) * chunk < rbs * nblk <= wgs * chunk          # chunks tile the step space exactly
    assert nbl == min(chunk, nblk) and lds <= 64 * 1024
    assert segfin == (chunk + nblk - 1) // nblk                                  # row blocks that can end inside one chunk
    assert prerot == (1 if M * nbl > (128 if M <= 8 else 32) else 0)                                  # a workgroup rotates at most 32 pairs itself
    # an explicit chunk length is honoured
    assert L.htr_linear_plan(m, n, 4, M, 1, out) == 0
    if out[0] == 1:
        assert out[1] == rbs * nblk


@pytest.mark.parametrize("m,n", [(128, 128), (4096, 4096), (14336, 4096), (4096, 14336), (28672, 4096)])
@pytest.mark.parametrize("M", [129, 192, 193, 384, 1000, 2048])
def test_plan_for_more_than_128_rows(L, m, n, M):
    """The fused decode -> matrix-unit kernel: tiles of 96 or 128 activation rows (the planner's choice; nsplit bits 20 / 21
    force one), up to 4 column splits by policy (8 on request) while the grid stays within the compute units, no empty
    split; the workspace holds the rotated activations and, with splits, a tile per workgroup."""
    out = (ctypes.c_int * 6)()
    nblk, rbs = n // 128, m // 128
    for tile_bit, heights in ((0, (96, 128)), (1 << 20, (96,)), (1 << 21, (128,))):
        ns = ((1 << 28) | tile_bit) if tile_bit else 0
        assert L.htr_linear_plan(m, n, 4, M, ns, out) == 0
        cb, wgs, tiles, S, prerot, lds = list(out)
        rows = [h for h in heights if tiles == -(-M // h)]
        assert rows and wgs == S * rbs * tiles and prerot == 1 and lds <= 160 * 1024
        assert 1 <= S <= 4 and S == -(-nblk // cb) and (S == 1 or wgs <= 256)
        need = L.htr_workspace_bytes(m, n, 4, M, ns)
        assert need >= 256 + M * n * 2 + (wgs * rows[0] * 128 * 4 if S > 1 else 0)
    for want in (1, 2, 8):
        ns = (1 << 28) | (1 << 20) | want
        if want > nblk or -(-nblk // -(-nblk // want)) != want:
            assert L.htr_linear_plan(m, n, 4, M, ns, out) != 0                      # such a split would leave one empty
            continue
        assert L.htr_linear_plan(m, n, 4, M, ns, out) == 0 and out[3] == want and out[1] == want * rbs * -(-M // 96)
    # bit 28 takes the kernel below its policy's row count too
    assert L.htr_linear_plan(m, n, 4, 40, (1 << 28) | 1, out) == 0 and out[2] == 1 and out[1] == rbs
    # where a third 96-row tile would start a second round of workgroups, two 128-row tiles are taken
    if (m, n, M) == (14336, 4096, 193):
        assert L.htr_linear_plan(m, n, 4, 256, 0, out) == 0 and out[2] == 2 and out[1] == 224
        assert L.htr_linear_plan(m, n, 4, 192, 0, out) == 0 and out[2] == 2 and out[5] == 101392


@pytest.mark.parametrize("cus", [32, 64, 120, 256, 304])
def test_plans_follow_the_device_compute_unit_count(L, cus):
    """The planner with another device's compute-unit count: the batched kernel's splits may only finish rows for each
    other (and so wait for each other) while the whole grid fits the chip at once; an explicit split beyond that falls
    back to the last split finishing every row.  The chunked kernel's waits only look at earlier workgroups, so any grid
    is safe there; its plan must still tile the step space."""
    out = (ctypes.c_int * 6)()
    assert L.htr_plan_device_override(cus, 160 * 1024) == 0
    try:
        for m, n in [(1024, 4096), (4096, 4096), (14336, 4096), (4096, 14336), (28672, 4096)]:
            nblk, rbs = n // 128, m // 128
            for M in (9, 16, 17, 32, 64, 128):
                assert L.htr_linear_plan(m, n, 4, M, 0, out) == 0
                cb, wgs, mutual, S, prerot, lds = list(out)
                assert wgs == rbs * S and S == -(-nblk // cb)
                assert wgs <= cus or S == 1                            # the policy never oversubscribes with splits
                assert mutual == (1 if wgs <= cus else 0)
                if prerot == 0:
                    assert wgs <= cus                                  # workgroups rotate their own slices only on a grid that fits
                for want in (2, 4, 8):
                    if L.htr_linear_plan(m, n, 4, M, (1 << 29) | want, out) != 0:
                        continue
                    assert out[3] == want and out[1] == rbs * want
                    assert out[2] == (1 if rbs * want <= cus else 0)   # mutual waits only when every workgroup is resident
                    assert L.htr_workspace_bytes(m, n, 4, M, (1 << 29) | want) >= 256 + out[1] * M * 128 * 4
            for M in (1, 4, 8):
                assert L.htr_linear_plan(m, n, 4, M, 0, out) == 0
                if M < 6 or (M < 7 and rbs < 192):
                    chunk, wgs = out[0], out[1]
                    assert (wgs - 1) * chunk < rbs * nblk <= wgs * chunk
        assert L.htr_plan_device_override(-1, 160 * 1024) == 3 and L.htr_plan_device_override(64, 1024) == 3
    finally:
        assert L.htr_plan_device_override(0, 0) == 0
    # back on the default device (none here: an unpartitioned MI355X is assumed): the decoder layer's batch-1 plans fill it
    for m, n in [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]:
        assert L.htr_linear_plan(m, n, 4, 1, 0, out) == 0 and out[1] == 256


def test_wire_helpers_match_oracle(oracle):
    from htr_amd import wire
    signs = torch.tensor([1., -1., 1., -1., 1., -1., 1., -1.])
    assert wire.pack_signs(signs).item() == 170                                  # tests/test_release.py:40-43 of the reference
    assert torch.equal(wire.unpack_signs(wire.pack_signs(signs), 8), signs)
    g = torch.Generator().manual_seed(4)
    words = torch.randint(-(2 ** 31), 2 ** 31, (5, 32), dtype=torch.int32, generator=g)
    st = torch.from_numpy(oracle.c_unpack_states(words.numpy(), 4).astype(np.int64))
    assert torch.equal(wire.pack_states(st, 4), words)
    assert torch.equal(wire.gen_values(st), torch.from_numpy(oracle.np_gen_values(st.numpy())))
    assert wire.payload_bytes(4096, 14336, 4) == 29370624 and wire.payload_bytes(152064, 4096, 4) == 311750720
    a = wire.synth_linear(256, 128, 3, 7)
    b = wire.synth_linear(256, 128, 3, 7)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert tuple(a[0].shape) == (16, 8, 24) and a[1].dtype == torch.float16 and a[2].numel() == 16 and a[3].numel() == 32
    assert wire.check_shapes(*a) == (256, 128, 3)
    with pytest.raises(RuntimeError):
        wire.check_shapes(a[0][:, :, :8].contiguous(), a[1], a[2], a[3])        # K = 1
    with pytest.raises(RuntimeError):
        wire.check_shapes(a[0][:15], a[1][:240], a[2], a[3][:30])               # m = 240, not a multiple of 128
    with pytest.raises(RuntimeError):
        wire.check_shapes(a[0], a[1].float(), a[2], a[3])


def test_operator_surface_on_cpu():
    from htr_amd import ops, wire
    qw, sc, su, sv = wire.synth_linear(256, 128, 4, 1)
    # M == 0 short-circuits before any device work (htr/ops.py:73-74 of the reference)
    y = ops.linear(torch.zeros(0, 128, dtype=torch.bfloat16), qw, sc, su, sv)
    assert tuple(y.shape) == (0, 256) and y.dtype == torch.bfloat16
    y = ops.linear(torch.zeros(2, 0, 128, dtype=torch.float16), qw, sc, su, sv)
    assert tuple(y.shape) == (2, 0, 256) and y.dtype == torch.float16
    with pytest.raises(RuntimeError):                                          # no CPU implementation, by design
        ops.linear(torch.zeros(1, 128, dtype=torch.bfloat16), qw, sc, su, sv)
    with pytest.raises(RuntimeError):
        ops.linear(torch.zeros(1, 256, dtype=torch.bfloat16), qw, sc, su, sv)  # wrong input width
    with pytest.raises(KeyError):
        ops.linear(torch.zeros(1, 128, dtype=torch.float64), qw, sc, su, sv)   # same as the reference's dtype map
    # custom op registered under the reference's name and schema, with a fake implementation
    op = torch.ops.htr.linear.default
    schema = str(op._schema)
    assert schema.startswith("htr::linear(Tensor x2, Tensor qweight, Tensor scales, Tensor su, Tensor sv, Tensor? bias) -> Tensor")
    meta = [t.to("meta") for t in (torch.zeros(3, 128, dtype=torch.bfloat16), qw, sc, su, sv)]
    out = op(*meta, None)
    assert out.device.type == "meta" and tuple(out.shape) == (3, 256) and out.dtype == torch.bfloat16


def test_missing_library_raises(monkeypatch):
    from htr_amd import _native
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", "/nonexistent/libhtr_gfx950.so")
    with pytest.raises(_native.NativeLibraryMissing):
        _native.lib()


def test_product_never_imports_the_oracle():
    bad = []
    for dirpath, _, files in os.walk(os.path.join(ROOT, "htr_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "libhtr_oracle" in text:
                    bad.append(f)
    assert bad == []


def test_bench_refuses_more_than_one_gpu():
    """The packed-linear path has no collectives: `bench.py --gpus N` with N above 1 says so and exits before it
    touches a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU only" in r.stderr and r.stdout.strip() == ""


def test_fake_tensors_and_make_fx_go_through_the_registered_op():
    """Tracers other than dynamo (FakeTensorMode, make_fx) never reach a data pointer: ops.linear hands tensor
    subclasses to the registered op htr::linear, whose fake implementation gives the shape (the reference always
    dispatches the op, htr/ops.py:107-122)."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.proxy_tensor import make_fx
    from htr_amd import ops, wire
    w = wire.synth_linear(256, 384, 4, 1)
    with FakeTensorMode() as mode:
        y = ops.linear(torch.empty(3, 5, 384, dtype=torch.bfloat16), *[mode.from_tensor(t) for t in w])
        assert tuple(y.shape) == (3, 5, 256) and y.dtype == torch.bfloat16
    g = make_fx(lambda x, qw, sc, su, sv: ops.linear(x, qw, sc, su, sv), tracing_mode="fake")(torch.empty(2, 384, dtype=torch.bfloat16), *w)
    assert any("htr.linear" in str(n.target) for n in g.graph.nodes)
