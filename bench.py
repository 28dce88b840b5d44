#!/usr/bin/env python3
"""Benchmark of the MI355X HTR-W1 packed-linear path.  Prints ONE JSON line.

Workload: the packed linears of one dense 9B-class decoder layer at K4, one bf16 activation row per linear.
A "step" is one layer: qkv (6144x4096, q/k/v fused along the output dim as the wire format allows),
o (4096x4096), gate_up (28672x4096, fused) and down (4096x14336): four launches through the C ABI.  Weights
cycle through a ring of distinct layer copies (>= 1 GB) so neither the per-XCD L2 nor the 256 MB Infinity
Cache can serve them.  value = packed W1 bytes of the layer / time per step.

The timed region is ONE HIP graph that holds exactly `--steps` layers (graphs of at most 1024 layers each when more
are asked for), so the figure does not depend on how the step count divides the ring.

Also on the line: a parity check of the timed launches against the CPU oracle (before the timed region), the same
layer as seven unfused launches, every shape of the layer on its own (cold: ring larger than the caches; warm: one
weight replayed, labelled as such), the roofline object of the dominant kernel, and the CPU oracle's rate on the
host cores as a baseline.
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
# the unfused matrices as row ranges of the fused ones (concatenation along the output dim, shared input signs)
UNFUSED_LAYER = [("q", "qkv", 0, 4096), ("k", "qkv", 4096, 1024), ("v", "qkv", 5120, 1024), ("o", "o", 0, 4096),
                 ("gate", "gate_up", 0, 14336), ("up", "gate_up", 14336, 14336), ("down", "down", 0, 4096)]
SEED = 20261125 + 1000 * 3
GRAPH_MAX_LAYERS = 1024


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--ring-gb", type=float, default=1.1, help="bytes of distinct packed weights cycled through")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample (0 = skip)")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-shape table and the unfused layer")
    ap.add_argument("--viterbi-tiles", type=int, default=0,
                    help="also time the encoder's trellis search on this many 256-weight tiles per K (0 = skip)")
    ap.add_argument("--repeats", type=int, default=7, help="timed passes of the headline graph (median and min are reported)")
    ap.add_argument("--suite", nargs="*", default=["default"], metavar="CASE",
                    help="the other baseline configurations (bench_suite.py): default = table (K2..5 x 2 shapes x batch 1, 2, 4), "
                         "batch8_32 (K3, K4 x 8, 16, 32 rows x 2 shapes), moe, lm_head; further names: batch, layer_rows, prefill, "
                         "all; none = skip")
    ap.add_argument("--no-anchors", action="store_true", help="skip the timing anchors of the dominant kernel")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy, so a counter profile of this command holds a kernel of known traffic")
    return ap.parse_args()


class PackedLinear:
    """Device tensors of one synthetic HTR-W1 linear; `rows` cuts a row range out of it (an unfused member)."""

    def __init__(self, name, m, n, k, qw, sc, su, sv, nbytes):
        self.name, self.m, self.n, self.k, self.qw, self.sc, self.su, self.sv, self.bytes = name, m, n, k, qw, sc, su, sv, nbytes

    def rows(self, wire, name, r0, cnt):
        return PackedLinear(name, cnt, self.n, self.k, self.qw[r0 // 16:(r0 + cnt) // 16], self.sc[r0:r0 + cnt], self.su,
                            self.sv[r0 // 8:(r0 + cnt) // 8], wire.payload_bytes(cnt, self.n, self.k))


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

    def make_linear(name, m, n, seed):
        qw = torch.randint(-(2 ** 31), 2 ** 31, (m // 16, n // 16, 8 * K), dtype=torch.int32, device=dev, generator=gen)
        g = torch.Generator(device="cpu").manual_seed(seed)
        sc = torch.exp(0.25 * torch.randn(m, generator=g)).half().to(dev)
        su = torch.randint(0, 256, (n // 8,), dtype=torch.uint8, generator=g).to(dev)
        sv = torch.randint(0, 256, (m // 8,), dtype=torch.uint8, generator=g).to(dev)
        return PackedLinear(name, m, n, K, qw, sc, su, sv, wire.payload_bytes(m, n, K))

    layer_bytes = sum(wire.payload_bytes(m, n, K) for _, m, n in FUSED_LAYER)
    ring = max(2, int(args.ring_gb * 1e9 / layer_bytes + 0.999))
    layers = [{nm: make_linear(nm, m, n, SEED + 17 * i + j) for j, (nm, m, n) in enumerate(FUSED_LAYER)} for i in range(ring)]
    unfused = [[lay[src].rows(wire, nm, r0, cnt) for nm, src, r0, cnt in UNFUSED_LAYER] for lay in layers]
    xs = {n: wire.synth_activation(1, n, SEED + 5, torch.bfloat16, dev) for n in (4096, 14336)}
    ys = {m: torch.empty(1, m, dtype=torch.bfloat16, device=dev) for m in (6144, 4096, 28672, 14336, 1024)}
    all_shapes = {(p.m, p.n) for p in list(layers[0].values()) + unfused[0]}
    ws_bytes = max(L.htr_workspace_bytes(m, n, K, 1, 0) for m, n in all_shapes)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)

    def launch(p):
        st = torch.cuda.current_stream().cuda_stream
        rc = L.htr_linear(p.qw.data_ptr(), p.sc.data_ptr(), p.su.data_ptr(), p.sv.data_ptr(), xs[p.n].data_ptr(), None,
                          ys[p.m].data_ptr(), p.m, p.n, p.k, 1, _native.BF16, _native.BF16, 0, ws.data_ptr(), ws.numel(), st)
        _native.check(rc)

    def fused_step(i):
        for p in layers[i % ring].values():
            launch(p)

    def unfused_step(i):
        for p in unfused[i % ring]:
            launch(p)

    def make_runner(fn, n):
        """run() executes fn(0) .. fn(n - 1): eagerly, or as HIP graphs of at most GRAPH_MAX_LAYERS calls of fn each."""
        if args.no_graph:
            def run_eager():
                for i in range(n):
                    fn(i)
            return run_eager
        graphs = []
        for a in range(0, n, GRAPH_MAX_LAYERS):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(a, min(n, a + GRAPH_MAX_LAYERS)):
                    fn(i)
            graphs.append(g)

        def run_graphs():
            for g in graphs:
                g.replay()
        return run_graphs

    def timed(run, count):
        """us per call of what `run` executes `count` of: HIP events on the launch stream, and the host's clock."""
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        run()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e6 / count
        return e0.elapsed_time(e1) * 1e3 / count, wall

    for i in range(ring):      # touch everything once outside any capture
        fused_step(i)
        unfused_step(i)
    torch.cuda.synchronize()

    # ---- parity of what is about to be timed: every launch of layer 0, fused and unfused, against the CPU oracle
    # (float64 decode-then-matmul); bf16 outputs, so the bar is half a bf16 ulp of the largest output plus the 1e-3
    # the float32 path is held to
    verified = None
    if args.cpu_seconds > 0:
        from oracle import oracle
        worst, checked = 0.0, 0
        for p in list(layers[0].values()) + unfused[0]:
            launch(p)
            torch.cuda.synchronize()
            got = ys[p.m].float().cpu().numpy().astype("float64")
            ref = oracle.c_linear(xs[p.n].float().cpu().numpy(), p.qw.cpu().numpy(), p.sc.cpu().numpy(), p.su.cpu().numpy(),
                                  p.sv.cpu().numpy(), None)
            worst = max(worst, float(abs(got - ref).max() / abs(ref).max()))
            checked += 1
        tol = 2.0 ** -8 + 1e-3
        verified = {"ok": worst <= tol, "launches_checked": checked, "max_rel_err": round(worst, 6), "tolerance": round(tol, 6),
                    "against": "CPU oracle, float64 decode-then-matmul, same tensors; max|y - ref| / max|ref| of the bf16 outputs"}
        if not verified["ok"]:
            print(f"bench.py: parity check failed: {verified}", file=sys.stderr)
            sys.exit(1)

    # ---- the headline: `steps` fused layers, one graph
    if args.warmup > 0:
        make_runner(fused_step, args.warmup)()
    run_steps = make_runner(fused_step, args.steps)
    # untimed: the graph of the timed region itself, replayed until the device has been busy for 30 ms, so that a short
    # timed region (--steps 20 is one millisecond) does not measure the clocks ramping up
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.03:
        run_steps()
        torch.cuda.synchronize()
    passes = sorted((timed(run_steps, args.steps)[::-1] for _ in range(max(1, args.repeats))))      # (wall, device) pairs
    wall_us, dev_us = passes[len(passes) // 2]
    ms_per_step = wall_us * 1e-3
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel (most bytes): k_linear<K=4> on the gate_up shape; average launch duration from HIP events
    # around back-to-back launches over the ring on the launch stream
    def time_launches(plist, reps):
        cnt = len(plist)
        run = make_runner(lambda i: launch(plist[i % cnt]), reps)
        run()
        return timed(run, reps)[0]

    gate_up = [lay["gate_up"] for lay in layers]
    dom_us = time_launches(gate_up, max(110, min(args.steps, 440)))
    dom_bytes = gate_up[0].bytes
    achieved = dom_bytes / dom_us / 1e3            # GB/s
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": "k_linear<K=4,MB=1> 28672x4096 (gate_up) batch 1", "us_per_launch": round(dom_us, 3),
                "us_per_launch_source": "HIP events around back-to-back graph launches over the ring, this run",
                "algorithmic_bytes_per_launch": dom_bytes}
    # traffic and the instruction counts are NOT measured by this run: they come from committed counter profiles of
    # this command and say so
    tpath = os.path.join(ROOT, "profiles", "k_linear_K4_gate_up_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            tj = json.load(f)
        roofline["traffic"] = tj.get("hbm_bytes_per_launch")
        roofline["traffic_source"] = "profiles/k_linear_K4_gate_up_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, committed)"
        if "kernel_trace_us_per_launch" in tj:
            roofline["us_per_launch_kernel_trace"] = tj["kernel_trace_us_per_launch"]
            roofline["frac_kernel_trace"] = round(dom_bytes / tj["kernel_trace_us_per_launch"] / 1e3 / HBM_PEAK_GBS, 4)
    cpath = os.path.join(ROOT, "profiles", "k_linear_K4_gate_up_sq_counters.json")
    if os.path.exists(cpath):
        with open(cpath) as f:
            cj = json.load(f)
        lane_ops = (cj["valu_instructions_per_launch"] + cj["mfma_instructions_per_launch"]) * 64
        peak = 256 * 4 * 16 * 2.4e9 / 1e12
        roofline["co_bound"] = {"kind": "valu_issue", "unit": "T lane-ops/s", "achieved": round(lane_ops / dom_us / 1e6, 2),
                                "peak": round(peak, 2), "frac": round(lane_ops / dom_us / 1e6 / peak, 4),
                                "valu_instructions_per_weight": round(cj["valu_instructions_per_launch"] * 64 / cj["weights_per_launch"], 3),
                                "source": "instruction counts from profiles/k_linear_K4_gate_up_sq_counters.json (committed), duration from this run"}

    # ---- timing anchors of the dominant launch, same ring, same run: its bytes read and nothing else; the launch with
    # the decode compiled out; the decode loop on register data (shader clock).  They bound what the exact decode allows.
    if not args.no_anchors:
        def anchor_launcher(kind):
            def go(i):
                p = gate_up[i % len(gate_up)]
                st = torch.cuda.current_stream().cuda_stream
                _native.check(L.htr_anchor_linear(kind, p.qw.data_ptr(), p.sc.data_ptr(), p.su.data_ptr(), p.sv.data_ptr(),
                                                  xs[p.n].data_ptr(), ys[p.m].data_ptr(), p.m, p.n, p.k, _native.BF16, _native.BF16,
                                                  ws.data_ptr(), ws.numel(), st))
            return go
        reps = max(110, min(args.steps, 440))
        anchors = {}
        for name, kind in (("plain_read_us", 2), ("no_decode_us", 1)):
            run = make_runner(anchor_launcher(kind), reps)
            run()
            anchors[name] = round(sorted(timed(run, reps)[0] for _ in range(3))[1], 3)
        _native.check(L.htr_workspace_init(ws.data_ptr(), ws.numel(), None, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        iters, wgs = 4000, 256
        stamps = torch.zeros(wgs * 8 * 2, dtype=torch.int64, device=dev)
        for name, mf in (("decode_only", 0), ("decode_and_products", 1)):
            for _ in range(2):
                _native.check(L.htr_anchor_decode(K, mf, iters, wgs, stamps.data_ptr(), torch.cuda.current_stream().cuda_stream))
                torch.cuda.synchronize()
            t = stamps.view(wgs, 8, 2).double().cpu()
            # Two waves share a SIMD and the older one is served first, so a workgroup's first four waves run at the
            # single-wave rate and the other four get what is left: the SIMD is through when its slower wave is.
            # Per SIMD and wave-step = the slowest wave's cycles / (iterations x 2 waves); median over the workgroups.
            cyc = float(t[:, :, 0].max(dim=1).values.median()) / iters / 2.0
            ghz = float((t[:, :, 0] / (t[:, :, 1] * 10.0)).median())
            anchors[name + "_cycles_per_wave_step"] = round(cyc, 1)
            anchors[name + "_cycles_per_wave_step_first_wave_alone"] = round(float(t[:, :, 0].min(dim=1).values.median()) / iters, 1)
            anchors[name + "_shader_clock_GHz"] = round(ghz, 3)
            # all wave-steps of the launch spread over the chip's SIMDs (4 per CU) at that rate and clock
            simds = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
            us = (gate_up[0].m // 16) * (gate_up[0].n // 128) / simds * cyc / (ghz * 1e3)
            anchors[name + "_us"] = round(us, 3)
        roofline["anchors"] = anchors
        roofline["anchors_note"] = ("same ring and run as us_per_launch: plain_read_us = the launch's weight stream and nothing else; "
                                    "no_decode_us = the launch with the trellis decode compiled out; decode_*_cycles_per_wave_step = the "
                                    "decode (and the four matrix instructions) of 2048 weights on register data, per SIMD with two waves on it "
                                    "(from the slower wave of each pair; *_first_wave_alone = what the favoured wave of a pair needs per "
                                    "wave-step); *_us = all wave-steps of the launch over all SIMDs at that rate and clock")
        roofline["ceiling_frac"] = round(dom_bytes / anchors["decode_only_us"] / 1e3 / HBM_PEAK_GBS, 4)
        roofline["ceiling_frac_with_products"] = round(dom_bytes / anchors["decode_and_products_us"] / 1e3 / HBM_PEAK_GBS, 4)

    if args.calibrate_copy:
        src = torch.randint(0, 256, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- the same layer as seven unfused launches, and every shape on its own: cold (consecutive launches walk the
    # ring, >= 1 GB between two visits of a byte) and warm (one weight replayed: served by the 256 MB Infinity Cache)
    shapes = unfused_layer = None
    if not args.no_shapes:
        n_unf = min(args.steps, 220)
        run_unf = make_runner(unfused_step, n_unf)
        run_unf()
        du, wu = timed(run_unf, n_unf)
        unfused_layer = {"launches_per_layer": 7, "us_per_layer": round(wu, 2), "us_per_layer_device_events": round(du, 2),
                         "GBps": round(layer_bytes / wu / 1e3, 1), "pct_hbm": round(layer_bytes / wu / 1e3 / HBM_PEAK_GBS * 100, 2),
                         "layers_timed": n_unf}
        shapes = []
        # a pool of distinct random stream words of its own (>= 1 GB): the copies of a matrix are consecutive pieces of
        # it, as many as fit (at most 512), so that even the 2 MB k / v matrices walk >= 1 GB between two visits of a byte
        pool = torch.randint(-(2 ** 31), 2 ** 31, (int(args.ring_gb * 1e9) // 4,), dtype=torch.int32, device=dev, generator=gen)
        members = [(nm, unfused[0][j]) for j, (nm, _, _, _) in enumerate(UNFUSED_LAYER)]
        members += [(nm, layers[0][nm]) for nm in ("qkv", "gate_up")]
        for nm, p in members:
            words = p.qw.numel()
            copies = max(2, min(512, pool.numel() // words))
            plist = [PackedLinear(nm, p.m, p.n, K, pool[c * words:(c + 1) * words].view(p.m // 16, p.n // 16, 8 * K), p.sc, p.su, p.sv,
                                  p.bytes) for c in range(copies)]
            cold = time_launches(plist, 2 * copies)
            warm = time_launches([p], 44)
            shapes.append({"name": nm, "m": p.m, "n": p.n, "K": K, "M": 1, "bytes": p.bytes, "us": round(cold, 3),
                           "GBps": round(p.bytes / cold / 1e3, 1), "pct_hbm": round(p.bytes / cold / 1e3 / HBM_PEAK_GBS * 100, 2),
                           "ring_copies": copies, "us_warm_cache": round(warm, 3),
                           "pct_hbm_warm_cache": round(p.bytes / warm / 1e3 / HBM_PEAK_GBS * 100, 2)})
        del pool

    # ---- CPU baseline: the oracle on the host cores, on a bounded sample of the same workload (the q projection of
    # the layer, repeated).  value = its fused decode-GEMV (rotate x, decode rows on the fly, rotate y; float64), the
    # faster of its two forms; the reference-shaped form (decode to a float32 W, then x @ W^T) is beside it.
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import oracle
        m, n = 4096, 4096
        qw, sc, su, sv = wire.synth_linear(m, n, K, SEED)
        x = wire.synth_activation(1, n, SEED + 5).float().numpy()
        a = [t.numpy() for t in (qw, sc, su, sv)]

        def sample(fn, seconds, cap):
            fn(x, *a)      # warm
            reps, t = 0, time.perf_counter()
            while True:
                fn(x, *a)
                reps += 1
                el = time.perf_counter() - t
                if el >= seconds or reps >= cap:
                    return reps, el

        freps, fel = sample(oracle.c_linear, args.cpu_seconds * 0.6, 4000)
        reps, el = sample(oracle.c_decode_then_matmul_f32, args.cpu_seconds * 0.4, 200)
        b = wire.payload_bytes(m, n, K)
        cpu = {"value": round(b * freps / fel / 1e9, 4), "unit": "GB/s", "cores": oracle.c_num_threads(), "kind": "port",
               "sample": f"{freps} x (4096x4096 K4 fused decode-GEMV, batch 1, float64) in {fel:.1f} s on {oracle.c_num_threads()} "
                         f"OpenMP threads; host reports {os.cpu_count()} cpus",
               "ms_per_matrix": round(fel / freps * 1e3, 3),
               "decode_to_f32_W_then_matmul_value": round(b * reps / el / 1e9, 4),
               "decode_to_f32_W_then_matmul_ms_per_matrix": round(el / reps * 1e3, 2)}

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
    if args.suite and "none" not in args.suite:
        import bench_suite
        del layers, gate_up, unfused
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
                   "ring_bytes": ring * layer_bytes,
                   "launch": "eager" if args.no_graph else "one HIP graph of `steps` layers cycling the ring (cold caches)"},
        "pct_hbm": round(value / HBM_PEAK_GBS * 100, 2),
        "us_per_layer": round(ms_per_step * 1e3, 2),
        "us_per_layer_device_events": round(dev_us, 2),
        "timed_passes": {"count": len(passes), "of_steps_each": args.steps, "us_per_layer_wall_median": round(wall_us, 2),
                         "us_per_layer_wall_min": round(passes[0][0], 2), "us_per_layer_wall_max": round(passes[-1][0], 2),
                         "us_per_layer_device_events_min": round(min(p[1] for p in passes), 2)},
        "verified": verified,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if unfused_layer is not None:
        out["unfused_layer"] = unfused_layer
    if shapes is not None:
        out["shapes"] = shapes
        out["shapes_note"] = ("us / GBps / pct_hbm: cold, consecutive launches walk ring_copies distinct weights (>= 1 GB per pass); "
                              "*_warm_cache: one weight replayed out of the 256 MB Infinity Cache, LABELLED warm, not a roofline claim")
    if search is not None:
        out["encoder_search"] = search
    if suite is not None:
        out["suite"] = suite
    print(json.dumps(out))


if __name__ == "__main__":
    main()
