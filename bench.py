#!/usr/bin/env python3
"""Benchmark of the MI355X HTR-W1 packed-linear path.  Prints ONE JSON line.

Workload: the packed linears of one dense 9B-class decoder layer at K4, one bf16 activation row per linear.
A "step" is one layer: qkv (6144x4096, q/k/v fused along the output dim as the wire format allows),
o (4096x4096), gate_up (28672x4096, fused) and down (4096x14336): four launches through the C ABI.  Weights
cycle through a ring of distinct layer copies (>= 1 GB) so neither the per-XCD L2 nor the 256 MB Infinity
Cache can serve them.  value = packed W1 bytes of the layer / time per step.

Also reported: per-shape kernel rates for all seven unfused matrices, the roofline object of the dominant
kernel, and the CPU oracle's decode-then-matmul rate on the host cores as a baseline.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
K = 4
FUSED_LAYER = [("qkv", 6144, 4096), ("o", 4096, 4096), ("gate_up", 28672, 4096), ("down", 4096, 14336)]
UNFUSED_LAYER = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                 ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]
SEED = 20261125 + 1000 * 3


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--ring-gb", type=float, default=1.1, help="bytes of distinct packed weights cycled through")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample (0 = skip)")
    ap.add_argument("--shapes", action="store_true", help="also time every unfused shape on its own")
    ap.add_argument("--viterbi-tiles", type=int, default=0,
                    help="also time the encoder's trellis search on this many 256-weight tiles per K (0 = skip)")
    ap.add_argument("--suite", nargs="*", default=None, metavar="CASE",
                    help="also time the other baseline configurations (htr_amd/bench_suite.py): table, batch, layer_rows, lm_head, moe, "
                         "prefill; no names = all")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy, so a counter profile of this command holds a kernel of known traffic")
    return ap.parse_args()


class PackedLinear:
    """Device tensors of one synthetic HTR-W1 linear plus its launch closure."""

    def __init__(self, torch, wire, native, name, m, n, k, seed, dev, gen):
        self.name, self.m, self.n, self.k = name, m, n, k
        self.qw = torch.randint(-(2 ** 31), 2 ** 31, (m // 16, n // 16, 8 * k), dtype=torch.int32, device=dev, generator=gen)
        g = torch.Generator(device="cpu").manual_seed(seed)
        self.sc = torch.exp(0.25 * torch.randn(m, generator=g)).half().to(dev)
        self.su = torch.randint(0, 256, (n // 8,), dtype=torch.uint8, generator=g).to(dev)
        self.sv = torch.randint(0, 256, (m // 8,), dtype=torch.uint8, generator=g).to(dev)
        self.bytes = wire.payload_bytes(m, n, k)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives are part of the packed-linear path); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from htr_amd import _native, wire
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    L = _native.lib()      # raises if the HIP library is missing: there is no fallback path
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(SEED)

    layer_bytes = sum(wire.payload_bytes(m, n, K) for _, m, n in FUSED_LAYER)
    ring = max(2, int(args.ring_gb * 1e9 / layer_bytes + 0.999))
    layers = [[PackedLinear(torch, wire, _native, nm, m, n, K, SEED + 17 * i + j, dev, gen)
               for j, (nm, m, n) in enumerate(FUSED_LAYER)] for i in range(ring)]
    xs = {n: wire.synth_activation(1, n, SEED + 5, torch.bfloat16, dev) for n in (4096, 14336)}
    ys = {m: torch.empty(1, m, dtype=torch.bfloat16, device=dev) for m in (6144, 4096, 28672, 14336, 1024)}
    ws_bytes = max(L.htr_workspace_bytes(m, n, K, 1, 0) for _, m, n in FUSED_LAYER + UNFUSED_LAYER)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)

    def launch(p, M=1):
        st = torch.cuda.current_stream().cuda_stream
        rc = L.htr_linear(p.qw.data_ptr(), p.sc.data_ptr(), p.su.data_ptr(), p.sv.data_ptr(), xs[p.n].data_ptr(), None,
                          ys[p.m].data_ptr(), p.m, p.n, p.k, M, _native.BF16, _native.BF16, 0, ws.data_ptr(), ws.numel(), st)
        _native.check(rc)

    def step(i):
        for p in layers[i % ring]:
            launch(p)

    def make_runner(fn, count):
        """Returns run(n): executes fn(0), fn(1), ... fn(n-1) (indices mod count), eagerly or by replaying HIP graphs.

        One graph holds a whole pass over the ring (count calls of fn); single-call graphs serve the remainder, so
        exactly n calls run whatever n is and the host only issues one replay per ring pass.
        """
        if args.no_graph:
            def run_eager(n):
                for i in range(n):
                    fn(i)
            return run_eager
        full = torch.cuda.CUDAGraph()
        with torch.cuda.graph(full):
            for i in range(count):
                fn(i)
        singles = []
        for i in range(count):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                fn(i)
            singles.append(g)

        def run_graph(n):
            for _ in range(n // count):
                full.replay()
            for i in range(n % count):
                singles[i].replay()
        return run_graph

    for i in range(ring):      # touch everything once outside any capture
        step(i)
    torch.cuda.synchronize()
    run_step = make_runner(step, ring)

    run_step(args.warmup)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    run_step(args.steps)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    dev_ms_per_step = e0.elapsed_time(e1) / args.steps
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel (most bytes): k_linear<K=4> on the gate_up shape; average launch duration from HIP events
    # around back-to-back launches over the ring on the launch stream
    def time_shape(plist, reps):
        cnt = len(plist)
        runner = make_runner(lambda i: launch(plist[i % cnt]), cnt)
        runner(cnt)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        runner(reps)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / reps      # us per launch

    gate_up = [lay[2] for lay in layers]
    dom_us = time_shape(gate_up, max(100, args.steps))
    dom_bytes = gate_up[0].bytes
    achieved = dom_bytes / dom_us / 1e3            # GB/s
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "k_linear_K4_gate_up_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "kernel": "k_linear<K=4,MB=1> 28672x4096 (gate_up) batch 1", "us_per_launch": round(dom_us, 3),
                "algorithmic_bytes_per_launch": dom_bytes}

    # co-bound: the rate at which the SIMDs issue the decode's integer instructions.  Wave instructions per launch come
    # from the committed counter profile, the duration is the one measured above; peak = 256 CUs x 4 SIMDs x 16 lanes
    # per cycle at the 2.4 GHz peak engine clock.
    cpath = os.path.join(ROOT, "profiles", "k_linear_K4_gate_up_sq_counters.json")
    if os.path.exists(cpath):
        with open(cpath) as f:
            cj = json.load(f)
        lane_ops = (cj["valu_instructions_per_launch"] + cj["mfma_instructions_per_launch"]) * 64
        peak = 256 * 4 * 16 * 2.4e9 / 1e12
        roofline["co_bound"] = {"kind": "valu_issue", "unit": "T lane-ops/s", "achieved": round(lane_ops / dom_us / 1e6, 2),
                                "peak": round(peak, 2), "frac": round(lane_ops / dom_us / 1e6 / peak, 4),
                                "valu_instructions_per_weight": round(cj["valu_instructions_per_launch"] * 64 / cj["weights_per_launch"], 3)}

    if args.calibrate_copy:
        src = torch.randint(0, 256, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    shapes = None
    if args.shapes:
        shapes = []
        for nm, m, n in UNFUSED_LAYER[:2] + UNFUSED_LAYER[4:5] + UNFUSED_LAYER[6:]:
            b = wire.payload_bytes(m, n, K)
            cnt = max(2, min(64, int(1.1e9 / b)))
            plist = [PackedLinear(torch, wire, _native, nm, m, n, K, SEED + 99 + j, dev, gen) for j in range(cnt)]
            us = time_shape(plist, 4 * cnt)
            shapes.append({"name": nm, "m": m, "n": n, "K": K, "M": 1, "bytes": b, "us": round(us, 3),
                           "GBps": round(b / us / 1e3, 1), "pct_hbm": round(b / us / 1e3 / HBM_PEAK_GBS * 100, 2)})
            del plist

    # ---- CPU baseline: the oracle's decode-then-matmul (full float32 W, then x @ W^T) on the host cores, on a
    # bounded sample of the same workload (the q projection of the layer, repeated)
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import oracle
        m, n = 4096, 4096
        qw, sc, su, sv = wire.synth_linear(m, n, K, SEED)
        x = wire.synth_activation(1, n, SEED + 5).float().numpy()
        a = [t.numpy() for t in (qw, sc, su, sv)]
        oracle.c_decode_then_matmul_f32(x, *a)      # warm
        reps, t = 0, time.perf_counter()
        while True:
            oracle.c_decode_then_matmul_f32(x, *a)
            reps += 1
            el = time.perf_counter() - t
            if el >= args.cpu_seconds or reps >= 200:
                break
        # second shape of the same baseline: the factorised product (rotate x, decode rows on the fly, rotate y; float64),
        # which never materialises W
        oracle.c_linear(x, *a)
        freps, ft = 0, time.perf_counter()
        while True:
            oracle.c_linear(x, *a)
            freps += 1
            fel = time.perf_counter() - ft
            if fel >= args.cpu_seconds / 3 or freps >= 100:
                break
        b = wire.payload_bytes(m, n, K)
        cpu = {"value": round(b * reps / el / 1e9, 4), "unit": "GB/s", "cores": oracle.c_num_threads(), "kind": "port",
               "sample": f"{reps} x (4096x4096 K4 decode to float32 W + x@W^T, batch 1) in {el:.1f} s; "
                         f"host reports {os.cpu_count()} cpus", "ms_per_matrix": round(el / reps * 1e3, 2),
               "fused_decode_gemv_value": round(b * freps / fel / 1e9, 4), "fused_decode_gemv_ms_per_matrix": round(fel / freps * 1e3, 2)}

    # ---- optional: the encoder's tail-biting Viterbi (htr_viterbi), tiles per second per K, with the CPU oracle beside it
    search = None
    if args.viterbi_tiles > 0:
        from htr_amd import encode
        search = {}
        for k in (2, 3, 4, 5):
            g = torch.Generator().manual_seed(k)
            xv = torch.randn(args.viterbi_tiles, 256, generator=g)
            wv = torch.rand(args.viterbi_tiles, 256, generator=g) + 0.5
            xd, wd = xv.to(dev), wv.to(dev)
            encode.viterbi(xd[:32], wd[:32], None, k)
            torch.cuda.synchronize()
            t = time.perf_counter()
            encode.viterbi(xd, wd, None, k)
            torch.cuda.synchronize()
            el = time.perf_counter() - t
            search[f"K{k}"] = {"tiles": args.viterbi_tiles, "ms": round(el * 1e3, 2), "tiles_per_s": round(args.viterbi_tiles / el)}
            if args.cpu_seconds > 0:
                from oracle import oracle
                nt = 16
                t = time.perf_counter()
                oracle.c_viterbi(xv[:nt].numpy(), wv[:nt].numpy(), k)
                search[f"K{k}"]["cpu_port_tiles_per_s"] = round(nt / (time.perf_counter() - t), 1)

    suite = None
    if args.suite is not None:
        from htr_amd import bench_suite
        del layers, gate_up
        torch.cuda.empty_cache()
        suite = bench_suite.run(args.suite, dev)

    out = {
        "metric": "K4 GEMV packed-weight GB/s at batch 1 (% of 8 TB/s HBM); us per 9B decoder layer",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32 decode -> f16 x f16 MFMA, f32 accumulate", "data": "synthetic",
        "config": {"workload": "dense 9B decoder layer, K4 HTR-W1, batch 1, 4 launches/step: qkv 6144x4096 (fused), "
                               "o 4096x4096, gate_up 28672x4096 (fused), down 4096x14336; bf16 x~N(0,1)",
                   "K": K, "batch": 1, "packed_bytes_per_step": layer_bytes, "ring_layers": ring,
                   "ring_bytes": ring * layer_bytes, "launch": "eager" if args.no_graph else "hip-graph replay, one graph per pass over the ring"},
        "pct_hbm": round(value / HBM_PEAK_GBS * 100, 2),
        "us_per_layer": round(ms_per_step * 1e3, 2),
        "us_per_layer_device_events": round(dev_ms_per_step * 1e3, 2),
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if shapes is not None:
        out["shapes"] = shapes
    if search is not None:
        out["encoder_search"] = search
    if suite is not None:
        out["suite"] = suite
    print(json.dumps(out))


if __name__ == "__main__":
    main()
