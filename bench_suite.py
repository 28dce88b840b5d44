"""Timings of the packed-linear path beyond the headline layer: the other configurations the reference's baseline
names (K x shape x batch table, 8..128 activation rows, routed experts, lm_head) and the prefill path.

Every case cycles through a ring of distinct weight copies larger than the caches (>= 1 GB, or as many copies as
fit), replays the ring as one HIP graph and reads HIP events on the launch stream.  Used by `bench.py --suite`;
`python bench_suite.py [names]` prints the same dictionary as JSON; `one:MxNxKxROWS` times a single shape.
"""
import json
import sys

import torch

from htr_amd import _native, ops, wire

HBM_PEAK_GBS = 8000.0
SEED = 20261125


def _events_us(fn, reps):
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / reps


def _graph_of(calls):
    """Runs every call once eagerly, then captures them, in order, into one graph."""
    for c in calls:
        c()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for c in calls:
            c()
    g.replay()
    torch.cuda.synchronize()
    return g


def _weights(m, n, K, copies, dev, seed):
    """`copies` weight sets that share scales and signs (small) and differ in the packed streams (the bytes that count)."""
    _, sc, su, sv = wire.synth_linear(m, n, K, seed, dev)
    gen = torch.Generator(device=dev).manual_seed(seed)
    return [(torch.randint(-(2 ** 31), 2 ** 31, (m // 16, n // 16, 8 * K), dtype=torch.int32, device=dev, generator=gen),
             sc, su, sv) for _ in range(copies)]


def time_linear(m, n, K, M, dev, ring_bytes=1 << 30, launches=192):
    """us per htr_linear launch (library plan), bf16 in and out."""
    L = _native.lib()
    pb = wire.payload_bytes(m, n, K)
    copies = int(max(2, min(48, ring_bytes // pb)))
    sets = _weights(m, n, K, copies, dev, SEED + m + n + K)
    x = wire.synth_activation(M, n, SEED + 3, torch.bfloat16, dev)
    y = torch.empty(M, m, dtype=torch.bfloat16, device=dev)
    ws = torch.zeros(L.htr_workspace_bytes(m, n, K, M, 0), dtype=torch.uint8, device=dev)

    def call(s):
        def go():
            _native.check(L.htr_linear(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), s[3].data_ptr(), x.data_ptr(), None,
                                       y.data_ptr(), m, n, K, M, _native.BF16, _native.BF16, 0, ws.data_ptr(), ws.numel(),
                                       torch.cuda.current_stream().cuda_stream))
        return go

    g = _graph_of([call(s) for s in sets])
    runs = sorted(_events_us(g.replay, max(1, launches // copies)) / copies for _ in range(5))
    us = runs[2]                                   # median of five timed passes; the fastest is reported beside it
    return {"m": m, "n": n, "K": K, "M": M, "us": round(us, 2), "us_min": round(runs[0], 2), "GBps": round(pb / us / 1e3, 1),
            "pct_hbm": round(pb / us / 1e3 / HBM_PEAK_GBS * 100, 2)}


def table(dev):
    """K in 2..5 x {4096x4096, 14336x4096} x batch 1, 2, 4."""
    return [time_linear(m, n, K, M, dev) for (m, n) in ((4096, 4096), (14336, 4096)) for K in (2, 3, 4, 5) for M in (1, 2, 4)]


def batch(dev):
    """K3, K4 x 8 .. 128 activation rows x {14336x4096, 4096x14336}; also the rate in TFLOP/s (2 M m n)."""
    out = []
    for K in (3, 4):
        for M in (8, 16, 32, 64, 128):
            for (m, n) in ((14336, 4096), (4096, 14336)):
                r = time_linear(m, n, K, M, dev)
                r["TFLOPs"] = round(2.0 * M * m * n / r["us"] / 1e6, 1)
                out.append(r)
    return out


def layer_rows(dev):
    """The four fused linears of the 9B decoder layer (qkv, o, gate_up, down; K4) at 8 .. 128 activation rows: us per
    launch and their sum per layer, with the tokens/s that sum alone would allow (rows / layer time / 32 layers)."""
    shapes = (("qkv", 6144, 4096), ("o", 4096, 4096), ("gate_up", 28672, 4096), ("down", 4096, 14336))
    out = []
    for M in (8, 16, 32, 64, 128):
        per = {nm: time_linear(m, n, 4, M, dev)["us"] for nm, m, n in shapes}
        tot = sum(per.values())
        out.append({"M": M, "us": per, "us_per_layer": round(tot, 1), "rows_per_s_at_32_layers": round(M / (tot * 32e-6))})
    return out


def batch8_32(dev):
    """K3, K4 x 8, 16, 32 activation rows x {14336x4096, 4096x14336}, with the rate in TFLOP/s (2 M m n)."""
    out = []
    for K in (3, 4):
        for M in (8, 16, 32):
            for (m, n) in ((14336, 4096), (4096, 14336)):
                r = time_linear(m, n, K, M, dev)
                r["TFLOPs"] = round(2.0 * M * m * n / r["us"] / 1e6, 1)
                out.append(r)
    return out


def lm_head(dev):
    return time_linear(152064, 4096, 4, 1, dev, ring_bytes=1 << 30, launches=96)      # few launches leave the clocks unsettled


def moe(dev):
    """64 experts (gate_up 2816x2048 fused, down 2048x1408, K4), 16 tokens routed top-6: one MoE layer as two grouped
    launches against one launch per expert and matrix."""
    L = _native.lib()
    E, T, TOP, H, F, K, RING = 64, 16, 6, 2048, 1408, 4, 4
    g = torch.Generator().manual_seed(SEED + 5000)
    probs = torch.softmax(torch.randn(T, E, generator=g), dim=-1)
    _, ids = torch.topk(probs, TOP, dim=-1)
    counts = torch.bincount(ids.reshape(-1), minlength=E).tolist()
    act = [e for e, c in enumerate(counts) if c]
    offs, o = [], 0
    for e in act:
        offs.append(o)
        o += counts[e]
    maxm = max(counts)
    xg = torch.randn(o, H, generator=g).bfloat16().to(dev)
    hid = torch.randn(o, F, generator=g).bfloat16().to(dev)
    y1 = torch.empty(o, 2 * F, dtype=torch.float32, device=dev)
    y2 = torch.empty(o, H, dtype=torch.float32, device=dev)
    stacks = [(_weights(2 * F, H, K, E, dev, SEED + 7000 + r), _weights(H, F, K, E, dev, SEED + 7100 + r)) for r in range(RING)]

    def entries(wl, xin, yout):
        rows = []
        for e, of in zip(act, offs):
            q, c = wl[e], counts[e]
            rows.append([q[0].data_ptr(), q[1].data_ptr(), q[2].data_ptr(), q[3].data_ptr(), xin[of:of + c].data_ptr(), 0,
                         yout[of:of + c].data_ptr(), c])
        return torch.tensor(rows, dtype=torch.int64).to(dev)

    tabs = [(entries(gu, xg, y1), entries(dn, hid, y2)) for gu, dn in stacks]
    need = max(L.htr_grouped_workspace_bytes(len(act), 2 * F, H, K, maxm), L.htr_grouped_workspace_bytes(len(act), H, F, K, maxm))
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    st = lambda: torch.cuda.current_stream().cuda_stream

    def grouped(r):
        def go():
            t1, t2 = tabs[r]
            _native.check(L.htr_linear_grouped(t1.data_ptr(), len(act), 2 * F, H, K, maxm, _native.BF16, _native.F32,
                                               ws.data_ptr(), ws.numel(), st()))
            _native.check(L.htr_linear_grouped(t2.data_ptr(), len(act), H, F, K, maxm, _native.BF16, _native.F32,
                                               ws.data_ptr(), ws.numel(), st()))
        return go

    ws1 = torch.zeros(max(L.htr_workspace_bytes(2 * F, H, K, maxm, 0), L.htr_workspace_bytes(H, F, K, maxm, 0)),
                      dtype=torch.uint8, device=dev)

    def single(r):
        def go():
            gu, dn = stacks[r]
            for wl, xin, yout, m, n in ((gu, xg, y1, 2 * F, H), (dn, hid, y2, H, F)):
                for e, of in zip(act, offs):
                    q, c = wl[e], counts[e]
                    _native.check(L.htr_linear(q[0].data_ptr(), q[1].data_ptr(), q[2].data_ptr(), q[3].data_ptr(),
                                               xin[of:of + c].data_ptr(), None, yout[of:of + c].data_ptr(), m, n, K, c,
                                               _native.BF16, _native.F32, 0, ws1.data_ptr(), ws1.numel(), st()))
        return go

    active_bytes = len(act) * (wire.payload_bytes(2 * F, H, K) + wire.payload_bytes(H, F, K))
    res = {"experts": E, "active_experts": len(act), "tokens": T, "top_k": TOP, "max_tokens_per_expert": maxm,
           "active_packed_bytes": active_bytes}
    for name, fn in (("grouped", grouped), ("per_expert_launches", single)):
        gph = _graph_of([fn(r) for r in range(RING)])
        us = _events_us(gph.replay, 20) / RING
        res[name] = {"us_per_layer": round(us, 1), "GBps": round(active_bytes / us / 1e3, 1)}
    return res


def prefill(dev):
    """129 rows and more: dequant_w + library GEMM against ONE launch of the fused decode -> matrix-unit kernel (rotation
    launch included) and against fused launches of 128 rows; eager calls, events on the launch stream."""
    L = _native.lib()
    out = []
    for (m, n) in ((4096, 4096), (6144, 4096), (14336, 4096), (4096, 14336)):
        w = wire.synth_linear(m, n, 4, SEED + 11, dev)

        def eager(fn, reps=20):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            return _events_us(fn, reps)

        td = eager(lambda: ops.dequant_w(*w))
        W = ops.dequant_w(*w)
        row = {"m": m, "n": n, "K": 4, "dequant_w_us": round(td, 1),
               "dequant_w_written_GBps": round(2.0 * m * n / td / 1e3, 1), "rows": []}
        for M in (64, 128, 160, 192, 256, 384, 512):
            x = wire.synth_activation(M, n, SEED + 3, torch.bfloat16, dev)
            y = torch.empty(M, m, dtype=torch.bfloat16, device=dev)
            tg = eager(lambda: torch.nn.functional.linear(x, W))
            ws = torch.zeros(L.htr_workspace_bytes(m, n, 4, M, 0), dtype=torch.uint8, device=dev)

            def one_launch():
                _native.check(L.htr_linear(w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(), w[3].data_ptr(), x.data_ptr(), None,
                                           y.data_ptr(), m, n, 4, M, _native.BF16, _native.BF16, 0, ws.data_ptr(), ws.numel(),
                                           torch.cuda.current_stream().cuda_stream))

            t1 = eager(one_launch)
            rec = {"M": M, "gemm_us": round(tg, 1), "dequant_plus_gemm_us": round(td + tg, 1), "one_fused_launch_us": round(t1, 1),
                   "ops_rows_per_fused_launch": ops.fused_rows_per_launch(m, n, M)}       # 0: ops.linear dequantizes
            if M > 128:
                old_max, old_rows = ops.GEMV_LOOP_MAX, ops.LAUNCH_MAX_M
                ops.GEMV_LOOP_MAX, ops.LAUNCH_MAX_M = 10 ** 9, 128
                try:
                    rec["launches_of_128_rows_us"] = round(eager(lambda: ops.linear(x, *w), reps=5), 1)
                finally:
                    ops.GEMV_LOOP_MAX, ops.LAUNCH_MAX_M = old_max, old_rows
            row["rows"].append(rec)
        out.append(row)
    return out


CASES = {"table": table, "batch8_32": batch8_32, "moe": moe, "lm_head": lm_head, "batch": batch, "layer_rows": layer_rows,
         "prefill": prefill}
DEFAULT = ("table", "batch8_32", "moe", "lm_head")       # what bench.py reports by default: every baseline configuration


def one(spec, dev):
    """`one:MxNxKxROWS` - a single shape (for counter and trace runs of one kernel), e.g. one:14336x4096x4x192"""
    m, n, K, M = (int(v) for v in spec.lower().split("x"))
    return time_linear(m, n, K, M, dev)


def run(names, dev=None):
    dev = dev or torch.device("cuda:0")
    names = list(CASES) if not names or "all" in names else [c for nm in names for c in (DEFAULT if nm == "default" else (nm,))]
    res = {}
    for nm in names:
        res[nm] = one(nm[4:], dev) if nm.startswith("one:") else CASES[nm](dev)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    return res


if __name__ == "__main__":
    print(json.dumps(run(sys.argv[1:])))
