"""Python entry points of the MI355X HTR-W1 packed-linear path + torch custom op htr::linear.

Same surface as htr/ops.py of the reference (linear(), the custom op and its fake, the
M-based dispatch of _linear_impl, htr/ops.py:69-122), but the body calls the gfx950 library
through its C ABI: tensors are passed as raw device pointers together with the current
torch stream; outputs and the workspace are allocated here with torch.
"""
import os

import torch

from . import _native, wire

CB = wire.cbscale()
_DTYPE_CODE = {torch.bfloat16: _native.BF16, torch.float16: _native.F16, torch.float32: _native.F32}

# One launch takes up to this many activation rows; longer inputs are cut into chunks that each
# re-read the packed weight (the reference does the same in 8-row chunks, htr/ops.py:77-88).
# HTR_GEMV_MAX_M lowers it (the reference's knob of that name is its rows per decode launch, 8 there: htr/ops.py:48).
LAUNCH_MAX_M = max(1, min(_native.MAX_BATCH, int(os.environ.get("HTR_GEMV_MAX_M", str(_native.MAX_BATCH)))))
GROUP_MAX_M = _native.MAX_GROUP_ROWS      # rows per entry of a grouped launch
# explicit chunk length (steps per workgroup) for experiments; 0 = library policy
NSPLIT = int(os.environ.get("HTR_NSPLIT", "0"))
# Above a number of activation rows the weight is dequantized once to the original basis (bf16) and a library GEMM does
# the product, as the reference does for prefill (HTR_PREFILL="w", htr/ops.py:52-54,89-93); up to it, fused launches
# run (the reference's HTR_GEMV_LOOP_MAX, htr/ops.py:59-61): up to 128 rows the batched decode kernel; beyond, the
# fused decode -> matrix-unit kernel in ONE launch (it re-decodes the weight once per 96 activation rows, so it pays while
# few such tiles cover the input).
# Measured on MI355X (K4, eager, us; one fused launch incl. its rotation launch / launches of 128 rows / dequantize + GEMM):
#   14336x4096: 160 rows 44 / 64 / 77, 192 rows 45 / 68 / 81, 256 rows 55 / 81 / 89, 384 rows 93 / 126 / 95, 512 rows 119 / 167 / 102
#   4096x14336: 160 rows 49 / 60 / 116, 192 rows 52 / 68 / 127, 256 rows 74 / 96 / 95, 384 rows 90 / 139 / 113, 512 rows 113 / 175 / 130
#   6144x4096:  160 rows 34 / 43 / 48, 192 rows 35 / 49 / 51, 256 rows 42 / 57 / 59, 384 rows 46 / 88 / 54, 512 rows 56 / 113 / 56
#   4096x4096:  160 rows 31 / 37 / 41, 192 rows 32 / 39 / 44, 256 rows 37 / 47 / 36, 384 rows 41 / 74 / 40, 512 rows 48 / 93 / 44
# So: one fused launch up to 384 rows on matrices from 4096x4096 up (512 rows where the rows are long, n >= 8192),
# dequantize beyond (and from 129 rows on smaller matrices, whose dequantization is cheap and which were not measured).
# HTR_GEMV_LOOP_MAX overrides the row limit for every shape (launches of LAUNCH_MAX_M rows up to it).
_LOOP_MAX_ENV = os.environ.get("HTR_GEMV_LOOP_MAX")
GEMV_LOOP_MAX = None if _LOOP_MAX_ENV is None else int(_LOOP_MAX_ENV)
ONE_LAUNCH = _native.MAX_BATCH
FUSED_GEMM_MAX_ROWS = 384
FUSED_GEMM_MIN_WEIGHTS = 4096 * 4096


def fused_rows_per_launch(m, n, M):
    """Rows per fused launch for M activation rows on an [m, n] linear; 0 = dequantize + library GEMM."""
    if GEMV_LOOP_MAX is not None:
        return LAUNCH_MAX_M if M <= GEMV_LOOP_MAX else 0
    if M <= _native.MAX_ROWS_PER_TILE:
        rows = _native.MAX_ROWS_PER_TILE
    else:
        rows = ONE_LAUNCH if (m * n >= FUSED_GEMM_MIN_WEIGHTS and M <= fused_max_rows(m, n)) else 0
    return min(rows, LAUNCH_MAX_M)


def fused_max_rows(m, n):
    """Activation rows up to which the fused kernels take an [m, n] linear; more rows go to dequantize + library GEMM."""
    if GEMV_LOOP_MAX is not None:
        return GEMV_LOOP_MAX
    if m * n < FUSED_GEMM_MIN_WEIGHTS:
        return _native.MAX_ROWS_PER_TILE
    return 512 if n >= 8192 else FUSED_GEMM_MAX_ROWS


# How inputs beyond GEMV_LOOP_MAX rows are multiplied (the reference's HTR_PREFILL, htr/ops.py:52-54): "w" = dequantize
# to the original basis and one library GEMM (default); "rot" = stay in the rotated basis: rotate the activations, GEMM
# against the dequantized Q, rotate the result (the reference's slower first-version path, htr/ops.py:101-104; here
# with float32 Q from htr_dequant_q and torch products, kept for cross-checks).
PREFILL = os.environ.get("HTR_PREFILL", "w")

class _Workspace:
    """One device buffer for split partials and pre-rotated activations, with its failure flag in pinned host memory."""
    __slots__ = ("buf", "flag", "stream")

    def __init__(self, buf, flag, stream):
        self.buf, self.flag, self.stream = buf, flag, stream


_WORKSPACES = {}      # (device index, stream), (device index, "capture", capture id) or (device index, "shared") -> _Workspace
_RETIRED = []         # buffers that a capture in progress has already recorded launches with: kept until released
_FLAG_POOLS = {}      # device index -> list of [pinned int32 tensor, its numpy view, next free word]
_FLAG_WORDS = 1024
# Captures that replay one after the other on one stream (the piecewise graphs of a serving stack: one per layer and batch
# size, thousands of them) may share ONE workspace per device instead of each holding its own: set this (or
# HTR_SHARE_CAPTURE_WS=1) before capturing.  Graphs that share it must never replay concurrently.
SHARE_CAPTURE_WORKSPACE = os.environ.get("HTR_SHARE_CAPTURE_WS", "0") not in ("", "0")


def share_capture_workspace(on=True):
    """Opt in to (or out of) one shared workspace per device for all HIP-graph captures: it is allocated and zeroed once,
    outside any capture (a warm-up call, or reserve_capture_workspace), so a capture neither allocates nor records a fill
    kernel, and thousands of captured pieces cost one buffer.  Only for graphs that replay serially."""
    global SHARE_CAPTURE_WORKSPACE
    SHARE_CAPTURE_WORKSPACE = bool(on)


def reserve_capture_workspace(device, nbytes):
    """Allocates (outside a capture) the shared capture workspace of `device` with room for `nbytes`."""
    device = torch.device(device)
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("reserve_capture_workspace must be called outside a capture")
    with torch.cuda.device(device):
        return _shared_workspace(device, _raw_stream(device.index), int(nbytes))


def release_capture_workspaces(device=None):
    """Drops the workspaces that captures on `device` (all devices if None) own.  Call it only after the graphs that
    recorded them have been destroyed: a graph replayed afterwards would write into freed memory."""
    dev = None if device is None else torch.device(device).index
    for key in [k for k in _WORKSPACES if len(k) == 3 and (dev is None or k[0] == dev)]:
        del _WORKSPACES[key]
    _RETIRED[:] = [w for w in _RETIRED if dev is not None and w.buf.device.index != dev]


def _flag_word(device):
    """A 4-byte word of pinned host memory (None while a capture is in progress and no room is left in the pools
    allocated so far: that workspace then works without a host-side flag)."""
    pools = _FLAG_POOLS.setdefault(device.index, [])
    if not pools or pools[-1][2] >= _FLAG_WORDS:
        if torch.cuda.is_current_stream_capturing():
            return None
        t = torch.zeros(_FLAG_WORDS, dtype=torch.int32).pin_memory()
        pools.append([t, t.numpy(), 0])
    pool = pools[-1]
    i = pool[2]
    pool[2] += 1
    return pool[1][i:i + 1], pool[0].data_ptr() + 4 * i


def _heal(ws, device):
    """A launch on this workspace gave up waiting (its host flag is set): drain the device, clear the workspace, raise."""
    torch.cuda.synchronize(device)
    ws.flag[0][0] = 0
    _native.check(_native.lib().htr_workspace_init(ws.buf.data_ptr(), ws.buf.numel(), ws.flag[1], ws.stream))
    torch.cuda.synchronize(device)
    raise RuntimeError("libhtr_gfx950: an earlier launch on this workspace gave up waiting for a partial result "
                       "(its outputs, and those of every launch after it, are NaN); the workspace has been cleared")


def check_status(device=None):
    """Raises if any launch so far gave up waiting on one of the workspaces of `device` (all devices if None), after
    clearing that workspace.  Eager calls check their own workspace by themselves; this is for graph replays."""
    for key, ws in list(_WORKSPACES.items()):
        if (device is None or key[0] == torch.device(device).index) and ws.flag is not None and ws.flag[0][0] != 0:
            _heal(ws, torch.device("cuda", key[0]))


def _new_workspace(key, device, stream_id, size):
    buf = torch.empty(size, dtype=torch.uint8, device=device)
    flag = _flag_word(device)
    ws = _WORKSPACES[key] = _Workspace(buf, flag, stream_id)
    _native.check(_native.lib().htr_workspace_init(buf.data_ptr(), size, None if flag is None else flag[1], stream_id))
    return ws


def _shared_workspace(device, stream_id, nbytes):
    key = (device.index, "shared")
    ws = _WORKSPACES.get(key)
    if ws is not None and ws.buf.numel() >= nbytes:
        return ws.buf
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError(f"libhtr_gfx950: the shared capture workspace of {device} holds "
                           f"{0 if ws is None else ws.buf.numel()} bytes, this launch needs {nbytes}; run the shapes once outside "
                           "the capture first, or call ops.reserve_capture_workspace")
    if ws is not None:
        _RETIRED.append(ws)        # graphs captured so far keep replaying against the old buffer
    return _new_workspace(key, device, stream_id, max(int(nbytes), 1 << 20)).buf


def workspace(device, stream_id, nbytes):
    """Scratch for split partials and pre-rotated activations: one per (device, stream), and one per HIP-graph capture.

    The reference keeps one counter tensor per device (htr/ops.py:24-28), which two streams
    would corrupt; keying by stream keeps concurrent streams apart.  Kernels leave the
    partial slots zero, so a buffer is cleared only when it is created (by the library's fill kernel).
    By default every capture gets buffers of its own (keyed by the runtime's capture id), allocated inside the capture,
    i.e. from the graph's memory pool, sized to what its launches need (no floor: a batch-1 layer takes tens of KB), and
    kept alive here until release_capture_workspaces: its address is part of the recorded launches, and the fill kernel
    of a NEW buffer is recorded with them.  A buffer that a capture has used is never replaced or freed; if a later call
    of the same capture needs more, a further buffer is added.  Eager calls never touch a capture's buffers.
    With SHARE_CAPTURE_WORKSPACE all captures of a device use one buffer that exists before they start (no allocation
    and no fill in any capture); that is only right for graphs that replay one after the other.
    """
    capturing = torch.cuda.is_current_stream_capturing()
    if capturing and SHARE_CAPTURE_WORKSPACE:
        return _shared_workspace(device, stream_id, nbytes)
    if not capturing and SHARE_CAPTURE_WORKSPACE:
        # eager calls (the warm-up before the captures) size the shared buffer; they run on their own stream's buffer
        _shared_workspace(device, stream_id, nbytes)
    cid = _native.lib().htr_stream_capture_id(stream_id) if capturing else 0
    key = (device.index, "capture", cid) if cid else (device.index, stream_id)
    ws = _WORKSPACES.get(key)
    if ws is not None and ws.buf.numel() >= nbytes:
        if ws.flag is not None and ws.flag[0][0] != 0 and not cid:
            _heal(ws, device)
        return ws.buf
    if ws is not None and cid:
        _RETIRED.append(ws)
    size = (int(nbytes) + 255) // 256 * 256 if cid else max(int(nbytes), 1 << 20)
    return _new_workspace(key, device, stream_id, size).buf


_NEED = {}       # workspace bytes per (m, n, K, M, nsplit)

# the current hipStream_t of a device as an integer; the direct accessor skips the construction of a Stream object
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda index: torch.cuda.current_stream(index).cuda_stream)


def _launch(x2, qweight, scales, su, sv, bias, y, m, n, K, out_code):
    L = _native.lib()
    M = x2.shape[0]
    key = (m, n, K, M, NSPLIT)
    need = _NEED.get(key)
    if need is None:
        need = _NEED[key] = L.htr_workspace_bytes(m, n, K, M, NSPLIT)
    if need == 0:
        raise RuntimeError("libhtr_gfx950: no launch plan for this shape / split")
    stream = _raw_stream(x2.device.index)
    ws = workspace(x2.device, stream, need)
    _native.check(L.htr_linear(qweight.data_ptr(), scales.data_ptr(), su.data_ptr(), sv.data_ptr(), x2.data_ptr(),
                               None if bias is None else bias.data_ptr(), y.data_ptr(), m, n, K, M,
                               _DTYPE_CODE[x2.dtype], out_code, NSPLIT, ws.data_ptr(), ws.numel(), stream))


def _linear_impl(x2, qweight, scales, su, sv, bias, out_dtype=None):
    m, n, K = wire.check_shapes(qweight, scales, su, sv)
    M = x2.shape[0]
    if x2.dim() != 2 or x2.shape[1] != n:
        raise RuntimeError(f"x has {x2.shape[-1]} input features, weight expects {n}")
    if x2.dtype not in _DTYPE_CODE:
        raise KeyError(x2.dtype)
    out_dtype = x2.dtype if out_dtype is None else out_dtype
    if M == 0:
        return x2.new_empty((0, m), dtype=out_dtype)
    if not x2.is_cuda:
        raise RuntimeError("htr::linear runs on a ROCm device only; move the tensors to the GPU")
    for t in (qweight, scales, su, sv):
        if t.device != x2.device or not t.is_contiguous():
            raise RuntimeError("HTR-W1 tensors must be contiguous and on the device of x")
    if bias is not None and (bias.dtype != out_dtype or bias.numel() != m or bias.device != x2.device):
        raise RuntimeError("bias must be [m] in the output dtype on the device of x")
    per_launch = fused_rows_per_launch(m, n, M)
    if per_launch == 0 and PREFILL == "rot":
        xr = wire.blk_had_cols_T(x2.float() * wire.unpack_signs(su, n).to(x2.device))
        yr = wire.blk_had_cols_T(xr @ dequant_q(qweight, scales).T) * wire.unpack_signs(sv, m).to(x2.device)
        if bias is not None:
            yr = yr + bias.float()
        return yr.to(out_dtype)
    if per_launch == 0:
        if PREFILL != "w":
            raise RuntimeError(f"HTR_PREFILL = {PREFILL!r}: expected 'w' or 'rot'")
        W = dequant_w(qweight, scales, su, sv)
        if x2.dtype != torch.bfloat16:
            W = W.to(x2.dtype)
        y = torch.nn.functional.linear(x2, W, None if bias is None else bias.to(x2.dtype))
        return y if y.dtype == out_dtype else y.to(out_dtype)
    y = torch.empty((M, m), dtype=out_dtype, device=x2.device)
    code = _DTYPE_CODE[out_dtype]
    with torch.cuda.device(x2.device):
        for r0 in range(0, M, per_launch):
            r1 = min(M, r0 + per_launch)
            _launch(x2[r0:r1], qweight, scales, su, sv, bias, y[r0:r1], m, n, K, code)
    return y


def linear_grouped(xs, weights, biases=None, out_dtype=None):
    """Many packed linears of one shape in one grouped launch: y_i = x_i @ W_i^T (+ bias_i).

    xs: list of [M_i, n] tensors (M_i may be 0); weights: list of (qweight, scales, su, sv) of identical shapes and K;
    returns the list of [M_i, m] results.  Routed experts are the use: the reference has no kernel for them and runs
    one linear per expert (docs/ADAPTERS.md:19 of the reference), which on this GPU is dominated by launch latency.
    Problems with more than GROUP_MAX_M rows are cut into several table entries.
    """
    if len(xs) != len(weights) or not xs:
        raise RuntimeError("linear_grouped wants as many activation tensors as weight tuples, at least one")
    m, n, K = wire.check_shapes(*weights[0])
    dev = xs[0].device
    if not xs[0].is_cuda:
        raise RuntimeError("htr::linear runs on a ROCm device only; move the tensors to the GPU")
    dt = xs[0].dtype
    if dt not in _DTYPE_CODE:
        raise KeyError(dt)
    out_dtype = dt if out_dtype is None else out_dtype
    rows = [int(x.shape[0]) for x in xs]
    total = sum(rows)
    y = torch.empty((total, m), dtype=out_dtype, device=dev)
    outs, entries, keep = [], [], []
    r = 0
    for i, (x, w) in enumerate(zip(xs, weights)):
        if wire.check_shapes(*w) != (m, n, K):
            raise RuntimeError("linear_grouped: every problem must have the same m, n and K")
        if x.dim() != 2 or x.shape[1] != n or x.dtype != dt or x.device != dev:
            raise RuntimeError("linear_grouped: activations must be [M, n] tensors of one dtype on one device")
        for t in w:
            if t.device != dev or not t.is_contiguous():
                raise RuntimeError("HTR-W1 tensors must be contiguous and on the device of x")
        b = None if biases is None else biases[i]
        if b is not None and (b.dtype != out_dtype or b.numel() != m or b.device != dev):
            raise RuntimeError("bias must be [m] in the output dtype on the device of x")
        xc = x.contiguous()
        keep.append(xc)
        outs.append(y[r:r + rows[i]])
        for r0 in range(0, rows[i], GROUP_MAX_M):
            mi = min(GROUP_MAX_M, rows[i] - r0)
            entries.append([w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(), w[3].data_ptr(),
                            xc[r0:r0 + mi].data_ptr(), 0 if b is None else b.data_ptr(), y[r + r0:r + r0 + mi].data_ptr(), mi])
        r += rows[i]
    if not entries:
        return outs
    if len(entries) > _native.MAX_GROUP:
        raise RuntimeError(f"linear_grouped: more than {_native.MAX_GROUP} table entries")
    max_m = max(e[7] for e in entries)
    L = _native.lib()
    need = L.htr_grouped_workspace_bytes(len(entries), m, n, K, max_m)
    if need == 0:
        raise RuntimeError("libhtr_gfx950: no launch plan for this grouped shape")
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev)
        table = torch.tensor(entries, dtype=torch.int64).to(dev, non_blocking=False)       # 8 x int64 = one 64-byte entry
        ws = workspace(dev, stream.cuda_stream, need)
        _native.check(L.htr_linear_grouped(table.data_ptr(), len(entries), m, n, K, max_m, _DTYPE_CODE[dt],
                                           _DTYPE_CODE[out_dtype], ws.data_ptr(), ws.numel(), stream.cuda_stream))
    return outs


def moe_experts(x, expert_ids, expert_weights, gate_up, down, activation=torch.nn.functional.silu):
    """Routed-expert MLP on packed weights: y_t = sum_j w_tj * Down_e( act(Gate_e x_t) * Up_e x_t ), e = ids[t, j].

    x [T, H]; expert_ids [T, top] integer; expert_weights [T, top]; gate_up[e] = HTR-W1 tuple of the fused [2F, H] matrix
    (gate rows first), down[e] = HTR-W1 tuple of [H, F].  Two grouped launches cover all active experts; the result is
    float32 [T, H].  The reference defines no such runtime (its experts are a composition of packed linears), so this
    is that composition, batched.
    """
    T, H = x.shape
    flat_e = expert_ids.reshape(-1)
    order = torch.argsort(flat_e, stable=True)
    tok = (order // expert_ids.shape[1])
    counts = torch.bincount(flat_e, minlength=len(gate_up)).tolist()
    xg = x[tok].contiguous()                                     # tokens grouped by expert
    act = [e for e, c in enumerate(counts) if c]
    offs, o = [], 0
    for e in act:
        offs.append(o)
        o += counts[e]
    h2 = linear_grouped([xg[o:o + counts[e]] for e, o in zip(act, offs)], [gate_up[e] for e in act], out_dtype=torch.float32)
    F = h2[0].shape[1] // 2
    hid = torch.cat(h2, 0)
    hid = (activation(hid[:, :F]) * hid[:, F:]).to(x.dtype).contiguous()
    out = linear_grouped([hid[o:o + counts[e]] for e, o in zip(act, offs)], [down[e] for e in act], out_dtype=torch.float32)
    wflat = expert_weights.reshape(-1)[order].to(torch.float32)
    y = torch.zeros((T, H), dtype=torch.float32, device=x.device)
    y.index_add_(0, tok, torch.cat(out, 0) * wflat[:, None])
    return y


@torch.library.custom_op("htr::linear", mutates_args=())
def htr_linear_op(x2: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor, su: torch.Tensor, sv: torch.Tensor,
                  bias: torch.Tensor | None) -> torch.Tensor:
    return _linear_impl(x2.contiguous(), qweight, scales, su, sv, bias)


@htr_linear_op.register_fake
def _(x2, qweight, scales, su, sv, bias):
    return x2.new_empty((x2.shape[0], qweight.shape[0] * 16))


def linear(x, qweight, scales, su, sv, bias=None):
    """y = x @ W^T (+bias) for an HTR-W1 weight. x [..., n] -> [..., m] in x.dtype.

    Under tracing (torch.compile) the call goes through the registered op `htr::linear`, as in the reference
    (htr/ops.py:107-122), and so do tensor subclasses (fake and functional tensors of other tracers); eager calls on
    plain tensors skip the dispatcher, which costs more host time than the launch itself."""
    shp = x.shape
    x2 = x.reshape(-1, shp[-1])
    if torch.compiler.is_compiling() or type(x2) is not torch.Tensor or type(qweight) not in (torch.Tensor, torch.nn.Parameter):
        y = htr_linear_op(x2, qweight, scales, su, sv, bias)      # tracing, fake or functional tensors: the registered op
    else:
        y = _linear_impl(x2.contiguous(), qweight, scales, su, sv, bias)
    return y.reshape(*shp[:-1], qweight.shape[0] * 16)


def linear_f32out(x, qweight, scales, su, sv, bias=None):
    """Same product with a float32 result (bias, if given, must be float32).  Used by accuracy checks."""
    shp = x.shape
    y = _linear_impl(x.reshape(-1, shp[-1]).contiguous(), qweight, scales, su, sv, bias, out_dtype=torch.float32)
    return y.reshape(*shp[:-1], qweight.shape[0] * 16)


def decode_raw(qweight):
    """int16 [ntiles, 256] of v(s) per weight in tile order (decode_raw of the reference extension)."""
    K = wire.bits_of(qweight)
    ntiles = qweight.numel() // (8 * K)
    if not qweight.is_cuda or not qweight.is_contiguous() or qweight.dtype != torch.int32:
        raise RuntimeError("decode_raw wants a contiguous int32 device tensor")
    out = torch.empty((ntiles, 256), dtype=torch.int16, device=qweight.device)
    with torch.cuda.device(qweight.device):
        st = torch.cuda.current_stream(qweight.device).cuda_stream
        _native.check(_native.lib().htr_decode_raw(qweight.data_ptr(), out.data_ptr(), ntiles, K, st))
    return out


def dequant_w(qweight, scales, su, sv):
    """Original-basis W bfloat16 [m, n] = Sv.Ho.Q.Hi.Su (dequant_w of the reference extension; wire.dequant on the CPU)."""
    m, n, K = wire.check_shapes(qweight, scales, su, sv)
    if not qweight.is_cuda or not all(t.is_contiguous() and t.device == qweight.device for t in (qweight, scales, su, sv)):
        raise RuntimeError("dequant_w wants contiguous tensors on one ROCm device")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=qweight.device)
    with torch.cuda.device(qweight.device):
        st = torch.cuda.current_stream(qweight.device).cuda_stream
        _native.check(_native.lib().htr_dequant_w(qweight.data_ptr(), scales.data_ptr(), su.data_ptr(), sv.data_ptr(),
                                                  out.data_ptr(), m, n, K, st))
    return out


def dequant_q(qweight, scales):
    """Rotated-domain Q float32 [m, n], bit-exact with the reference CPU decoder (wire.dequant_Q)."""
    mt, nt, W = qweight.shape
    if not qweight.is_cuda or not qweight.is_contiguous() or scales.dtype != torch.float16:
        raise RuntimeError("dequant_q wants contiguous device tensors (int32 qweight, float16 scales)")
    out = torch.empty((mt * 16, nt * 16), dtype=torch.float32, device=qweight.device)
    with torch.cuda.device(qweight.device):
        st = torch.cuda.current_stream(qweight.device).cuda_stream
        _native.check(_native.lib().htr_dequant_q(qweight.data_ptr(), scales.data_ptr(), out.data_ptr(), mt, nt, W // 8, st))
    return out
