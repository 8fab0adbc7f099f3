#!/usr/bin/env python3
"""Benchmark of the quantized projection path on one MI355X.

A "step" is one decoded token's pass over the projections of a 32-layer 8B-class dense model in
Q4_K_M (the 8B decode configuration, repeated over 32 DISTINCT layers = 4.41 GB of weights so that
every step streams from HBM, not from the 256 MB Infinity Cache): per layer q/k/v (one launch),
o, gate/up (one launch) in Q4_K and down in Q6_K, each preceded by the activation quantizer, in
the ggml activation mode (the reference CPU path's arithmetic).  `value` is algorithmic GGUF bytes
per step / time.  Extra legs report the dominant kernel against the HBM roofline, the int8-MFMA
prefill GEMM (config 4), the MoE feed-forward (config 5) and the CPU oracle on the host cores.

    python bench.py --gpus 1 --steps 20 --warmup 3 [--legs step,roofline,verify,q8_0,prefill,moe,llama_bench,cpu]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0
Q4_K, Q6_K, Q8_0 = 12, 14, 8
D_MODEL, D_KV, D_FF = 4096, 1024, 14336


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gguf_bytes(qtype, n, k):
    return n * (k // (32 if qtype == Q8_0 else 256)) * {Q8_0: 34, Q4_K: 144, Q6_K: 210}[qtype]


def gemv_bytes(qtype, n, k, m=1):
    """algorithmic bytes of one projection: GGUF weight bytes + fp32 activations in + fp32 out"""
    return gguf_bytes(qtype, n, k) + m * k * 4 + m * n * 4


LAYER_TENSORS = [("q", Q4_K, D_MODEL, D_MODEL), ("k", Q4_K, D_KV, D_MODEL), ("v", Q4_K, D_KV, D_MODEL),
                 ("o", Q4_K, D_MODEL, D_MODEL), ("gate", Q4_K, D_FF, D_MODEL), ("up", Q4_K, D_FF, D_MODEL),
                 ("down", Q6_K, D_MODEL, D_FF)]
LAYER_BYTES = sum(gemv_bytes(t, n, k) for _, t, n, k in LAYER_TENSORS)
LAYER_WEIGHT_BYTES = sum(gguf_bytes(t, n, k) for _, t, n, k in LAYER_TENSORS)


class Timer:
    """HIP events on the stream the library launches on."""

    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream

    def time_ms(self, fn, iters):
        t = self.torch
        with t.cuda.stream(self.stream):
            a, b = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
            a.record(self.stream)
            for _ in range(iters):
                fn()
            b.record(self.stream)
        b.synchronize()
        return a.elapsed_time(b) / iters

    def samples_ms(self, fn, n):
        """n separately timed calls (an event pair around each), for records that keep raw samples"""
        t = self.torch
        evs = []
        with t.cuda.stream(self.stream):
            for _ in range(n):
                a, b = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
                a.record(self.stream)
                fn()
                b.record(self.stream)
                evs.append((a, b))
        evs[-1][1].synchronize()
        return [a.elapsed_time(b) for a, b in evs]


def median(samples):
    """the reference's median (inference/crates/icn-parity/src/compare.rs:757-766): mean of the two middle samples
    of an even count"""
    v = sorted(float(x) for x in samples)
    mid = len(v) // 2
    return (v[mid - 1] + v[mid]) / 2.0 if len(v) % 2 == 0 else v[mid]


def summarize(samples):
    """median and median absolute deviation of raw samples, as the reference's comparator summarizes a measurement
    (compare.rs:727-733), plus the count; `rel_mad` = MAD / median"""
    med = median(samples)
    mad = median([abs(float(x) - med) for x in samples])
    return {"median": med, "mad": mad, "rel_mad": mad / med if med > 0 else 0.0, "n": len(samples)}


MIN_SAMPLES, MIN_WARMUP = 30, 5      # every per-kernel figure: at least this many timed samples after this many warm-ups


def physical_cores():
    """(physical cores, logical CPUs) this process may run on: distinct (package, core) pairs over the CPUs of its
    affinity mask, from /sys/devices/system/cpu/cpuN/topology (the reference runs one thread a physical core:
    inference/parity/profiles/pr.toml:41)"""
    try:
        cpus = sorted(os.sched_getaffinity(0))
    except AttributeError:
        cpus = list(range(os.cpu_count() or 1))
    cores = set()
    for c in cpus:
        base = f"/sys/devices/system/cpu/cpu{c}/topology/"
        try:
            with open(base + "physical_package_id") as f:
                pkg = f.read().strip()
            with open(base + "core_id") as f:
                core = f.read().strip()
            cores.add((pkg, core))
        except OSError:
            cores.add(("?", str(c)))
    return len(cores), len(cpus)


def capture(torch, stream, fn):
    """Captures fn() (launches on `stream` only) into a HIP graph; returns replay() or None."""
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            fn()
        return g.replay
    except Exception as e:  # capture is an optimisation of the launch path, not of the kernels
        log(f"[bench] graph capture unavailable ({type(e).__name__}: {e}); timing eager launches")
        try:
            torch.cuda.synchronize()
        except Exception:
            pass
        return None


MAX_LINE_BYTES = 4000      # the final stdout line stays under this; everything else goes to the details file


def source_digest(*rel):
    """sha256 over the named source files (relative to the repository root), first 16 hex digits"""
    import hashlib
    h = hashlib.sha256()
    for r in rel:
        with open(os.path.join(ROOT, r), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


DECODE_KERNEL_SOURCES = ("magnitude_amd/csrc/kernels_decode.hip", "magnitude_amd/csrc/gemv_frags.h")


def measured_traffic(summary="decode_gate_up_q4k.txt"):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 counter summary (FETCH_SIZE +
    WRITE_SIZE, each scaled by a copy kernel of known size).  The summary names the digest of the kernel sources
    it was measured on; when the sources have changed since, the figure is withheld (None) and the source says so."""
    path = os.path.join(ROOT, "profiles", summary)
    traffic, digest = None, None
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                traffic = int(line.split(":")[1])
            if line.startswith("kernel_source_digest:"):
                digest = line.split(":")[1].strip()
    except OSError:
        return None, "not recorded"
    if traffic is None:
        return None, "not recorded"
    now = source_digest(*DECODE_KERNEL_SOURCES)
    if digest != now:
        return None, f"profiles/{summary} is stale (kernel sources {now}, summary measured on {digest})"
    return traffic, f"profiles/{summary} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, kernel sources {digest})"


def recorded_streaming_probe(summary="decode_gate_up_q4k.txt"):
    """[low, high] microseconds that a kernel of the decode kernel's grid which only streams the 66 MB of a gate+up
    launch was measured at (committed profile summary, line `streaming_probe_us: lo hi`); None when not recorded"""
    try:
        for line in open(os.path.join(ROOT, "profiles", summary)):
            if line.startswith("streaming_probe_us:"):
                return [float(v) for v in line.split(":")[1].split()]
    except (OSError, ValueError):
        pass
    return None


def _r(v, nd=4):
    return None if v is None else round(float(v), nd)


def compact_line(out, details_path=None):
    """The one JSON line the driver parses: the contract's fields, the roofline and CPU baseline objects and one
    headline figure per other leg.  Per-shape tables, raw samples and the reference-shaped evidence rows are in the
    details file (the reference keeps raw samples in evidence files too: inference/parity/README.md:110)."""
    keep = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data")
    line = {k: out.get(k) for k in keep}
    line["value"], line["ms_per_step"] = _r(out.get("value"), 2), _r(out.get("ms_per_step"), 5)
    cfg = out.get("config", {})
    line["config"] = {k: cfg[k] for k in ("workload", "layers", "act_mode", "launch_route") if k in cfg}
    for k in ("pct_hbm_peak", "tokens_per_s_projection_only"):
        if out.get(k) is not None:
            line[k] = _r(out[k], 2)
    if out.get("step_stats"):
        st = out["step_stats"]
        line["value_stats"] = {"statistic": "median + MAD over per-step samples", "median_ms": _r(st["median"], 5),
                               "mad_ms": _r(st["mad"], 5), "rel_mad": _r(st["rel_mad"], 4), "n": st["n"]}
    rf = out.get("roofline")
    if rf:
        line["roofline"] = {k: (_r(rf[k]) if isinstance(rf.get(k), float) else rf.get(k))
                            for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "traffic_source", "kernel",
                                      "bytes_per_launch", "us_per_launch", "mad_us", "rel_mad", "samples", "launches_timed",
                                      "launch_us", "streaming_probe_us")
                            if k in rf}
        line["decode_kernels_us"] = {k: _r(v["us_per_launch"], 2) for k, v in rf.get("other_kernels", {}).items()}
    cb = out.get("cpu_baseline")
    if cb:
        line["cpu_baseline"] = {k: (_r(cb[k]) if isinstance(cb.get(k), float) else cb.get(k))
                                for k in ("value", "unit", "cores", "kind", "sample", "host_cpus", "host_physical_cores",
                                          "thread_policy", "rel_mad", "one_thread_GBps", "isa")
                                if k in cb}
    if "verify" in out:
        line["verify_us"] = {f"M{r['M']}_{r['group']}": _r(r["us_per_launch"], 2) for r in out["verify"]["shapes"]}
        if all("us_rows_quantized_earlier" in r for r in out["verify"]["shapes"]):
            line["verify_us_rows_quantized_earlier"] = {f"M{r['M']}_{r['group']}": _r(r["us_rows_quantized_earlier"], 2)
                                                        for r in out["verify"]["shapes"]}
    if "q8_0" in out:
        line["q8_0_gemv"] = {"us": _r(out["q8_0"]["us_per_launch"], 2), "frac_hbm_peak": _r(out["q8_0"]["frac_hbm_peak"])}
    for key, tag in (("prefill", "prefill_q8x32"), ("prefill_ggml_acts", "prefill_q8k")):
        if key in out:
            pf = out[key]
            line[tag] = {"headline_tops": _r(pf["headline_tops"], 1), "frac_int8_peak": _r(pf["headline_frac_int8_peak"]),
                         "rel_mad": _r(pf.get("headline_rel_mad")), "samples": pf.get("samples_per_shape"),
                         "peak_tops": INT8_PEAK_TOPS, "shape": "M4096 K4096 N14336 Q4_K",
                         "tops": {f"{r.get('type', 'Q4_K')}_M{r['M']}_K{r['K']}_N{r['N']}": _r(r["gemm_tops"], 0)
                                  for r in pf["shapes"]}}
            for k in ("bound", "floor_tops", "floor"):
                if k in pf:
                    line[tag][k] = pf[k]
    if "moe" in out:
        line["moe_ffn"] = {f"B{r['B']}": {"us": _r(r["ms"] * 1e3, 1), "GBps": _r(r["GBps"], 0), "rel_mad": _r(r.get("rel_mad")),
                                          "MB_cycled": _r(r.get("bytes_cycled", 0) / 1e6, 0)}
                           for r in out["moe"]["batches"]}
    if "llama_bench" in out:
        med = median
        toks = {r["output"]["operation"].split(".")[1]: med(r["measurements"][1]["samples"]) for r in out["llama_bench"]}
        line["llama_bench_projections_only"] = {"pp512_tok_s": _r(toks.get("prompt-processing"), 0),
                                                "tg128_tok_s": _r(toks.get("token-generation"), 1)}
    if details_path:
        line["details"] = details_path
    text = json.dumps(line, separators=(",", ":"))
    if len(text) > MAX_LINE_BYTES:      # never lose the contract's fields to a long tail: drop the optional tables first
        for k in ("prefill_q8k", "prefill_q8x32", "verify_us", "moe_ffn", "decode_kernels_us"):
            if isinstance(line.get(k), dict) and "tops" in line[k]:
                line[k].pop("tops")
            else:
                line.pop(k, None)
            text = json.dumps(line, separators=(",", ":"))
            if len(text) <= MAX_LINE_BYTES:
                break
    assert len(text) <= MAX_LINE_BYTES, len(text)
    return text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--legs", default="step,roofline,verify,q8_0,norm,prefill,moe,llama_bench,cpu")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--split-quantize", action="store_true",
                    help="run the activation quantizer as a separate launch instead of inside the projection kernel")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (counter calibration for rocprofv3 --pmc)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--evidence-sql", default=None,
                    help="also write the per-kernel rows as test-backend-ops SQL INSERT lines to this file")
    ap.add_argument("--details-json", default=os.path.join("gpurun_out", "bench_details.json"),
                    help="per-shape tables, raw samples and the reference-shaped evidence rows go to this file "
                         "('' = nowhere); stdout carries one compact line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        return 2
    legs = set(args.legs.split(","))

    import torch

    from magnitude_amd import ACT_GGML, ACT_Q8X32, Context, evidence, synth

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    ctx = Context(0, stream=stream.cuda_stream)
    timer = Timer(torch, stream)
    props = torch.cuda.get_device_properties(0)
    log(f"[bench] device {props.name} ({getattr(props, 'gcnArchName', '?')}), {props.multi_processor_count} CUs")

    out = {
        "metric": "Q4_K GEMV achieved HBM GB/s (% peak) + prefill GEMM TOPS, 8B shapes",
        "value": None, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8",
        "dtype_note": "int8 activations x int4/int6/int8 weight codes -> int32 dots, fp32 scales (u8 bytes streamed)",
        "data": "synthetic: N(0,0.02) weights quantized to GGUF Q4_K/Q6_K on the device, N(0,1) fp32 activations",
        "config": {"workload": "configs[1]: Q4_K_M decode projections (q,k,v,o,gate,up Q4_K; down Q6_K), batch 1, "
                               f"d_model 4096, FFN 14336, {args.layers} distinct layers per step",
                   "layers": args.layers, "act_mode": "ggml (Q8_K activations, integer dots)",
                   "launches_per_layer": ("4 quantize + 4 projection" if args.split_quantize else
                                          "4 (q/k/v and gate/up share a launch; activations quantized in the kernel prologue)")},
    }

    # ------------------------------------------------------------------ weights
    L = args.layers
    layers = []
    need_layers = bool(legs & {"step", "roofline", "verify", "cpu", "llama_bench", "norm"})
    if need_layers:
        t0 = time.time()
        for l in range(L):
            lw = {}
            for i, (name, qt, n, k) in enumerate(LAYER_TENSORS):
                blocks = synth.random_weight(qt, n, k, seed=1000 * l + i, device=dev)
                lw[name] = ctx.upload_from_device(qt, k, n, blocks)
                del blocks
            layers.append(lw)
        torch.cuda.synchronize()
        log(f"[bench] {L} layers of weights ({L * LAYER_WEIGHT_BYTES / 1e9:.2f} GB) ready in {time.time() - t0:.1f}s")

    g = torch.Generator(device=dev).manual_seed(7)
    x_attn = torch.randn((1, D_MODEL), generator=g, device=dev)
    x_o = torch.randn((1, D_MODEL), generator=g, device=dev)
    x_ffn = torch.randn((1, D_MODEL), generator=g, device=dev)
    x_down = torch.randn((1, D_FF), generator=g, device=dev)
    lib = ctx.lib
    abuf = [torch.empty(int(lib.qproj_act_bytes(ACT_GGML, qt, 1, k)), dtype=torch.uint8, device=dev)
            for qt, k in ((Q4_K, D_MODEL), (Q4_K, D_MODEL), (Q4_K, D_MODEL), (Q6_K, D_FF))]
    y = {name: torch.empty((1, n), device=dev) for name, _, n, _ in LAYER_TENSORS}
    torch.cuda.synchronize()

    groups = [("qkv", ["q", "k", "v"], x_attn, 0), ("o", ["o"], x_o, 1), ("gate_up", ["gate", "up"], x_ffn, 2),
              ("down", ["down"], x_down, 3)]

    def launch(lw, grp, fused):
        _, names, x, ai = grp
        ws = [lw[n] for n in names]
        ys = [y[n] for n in names]
        if fused:      # one launch: the kernel quantizes the activation row in its prologue
            ctx.mul_mat_multi(ws, x, ACT_GGML, outs=ys, sync=False)
        else:          # activation quantizer as its own launch, then the projection
            ctx.quantize_activations_raw(x, ACT_GGML, ws[0].qtype, out=abuf[ai], sync=False)
            ctx.mul_mat_quantized(ws, abuf[ai], ACT_GGML, 1, ys, sync=False)

    def layer_pass(lw):
        for grp in groups:
            launch(lw, grp, not args.split_quantize)

    def step():
        for lw in layers:
            layer_pass(lw)

    # ------------------------------------------------------------------ step leg (headline)
    if "step" in legs:
        step()
        ctx.sync()
        def timed(run):
            """K steps between two synchronizations (the quoted time), with an event after every step on the library's
            stream so that the spread over the steps is known too"""
            for _ in range(args.warmup):
                run()
            torch.cuda.synchronize()
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
            with torch.cuda.stream(stream):
                t0 = time.perf_counter()
                evs[0].record(stream)
                for i in range(args.steps):
                    run()
                    evs[i + 1].record(stream)
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) / args.steps
            return dt, [evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps)]

        # The 128 launches of a step are issued either one by one or as a replay of a HIP graph; both are timed
        # (warmup + the same number of steps each) and the step is quoted on the faster route.  Issued one by
        # one the host stays ahead of the device here (a launch costs it about 6 us, the average kernel 9 us),
        # and the replay has measured 3 % slower than that on this runtime.
        runs = {"eager": timed(step)}
        replay = None if args.no_graph else capture(torch, stream, step)
        if replay is not None:
            runs["hip_graph"] = timed(replay)
        modes = {k: v[0] for k, v in runs.items()}
        best = min(modes, key=modes.get)
        dt = modes[best]
        out["step_stats"] = summarize(runs[best][1])          # ms per step, one sample a step (events)
        out["config"]["launch_route"] = best
        out["config"]["hip_graph"] = best == "hip_graph"
        out["ms_per_step_by_route"] = {k: v * 1e3 for k, v in modes.items()}
        bytes_step = L * LAYER_BYTES
        out["ms_per_step"] = dt * 1e3
        out["value"] = bytes_step / dt / 1e9
        out["pct_hbm_peak"] = 100.0 * out["value"] / HBM_PEAK_GBS
        out["tokens_per_s_projection_only"] = 1.0 / dt
        out["bytes_per_step"] = bytes_step
        log(f"[bench] step: {dt * 1e3:.3f} ms  {out['value']:.0f} GB/s ({out['pct_hbm_peak']:.1f}% of 8 TB/s)  "
            f"{1.0 / dt:.0f} tok/s (projections only)  [" +
            ", ".join(f"{k} {v * 1e3:.3f} ms" for k, v in modes.items()) + "]")

    # ------------------------------------------------------------------ fixed cost of a launch
    launch_us = None
    if legs & {"roofline", "moe"}:
        # the fixed cost of a launch, measured in this run from the smallest launch the library has (one 256 x 64 Q4_K
        # projection of one row: a single workgroup), 64 of them a graph replay; the calibration records below carry it
        # (launch_microseconds, inference/crates/icn-server/src/main.rs:1313-1325)
        tiny = ctx.upload_from_device(Q4_K, 256, 64, synth.random_weight(Q4_K, 64, 256, seed=3, device=dev))
        x_tiny, y_tiny = torch.randn((1, 256), generator=g, device=dev), torch.empty((1, 64), device=dev)

        def tiny_launches():
            for _ in range(64):
                ctx.mul_mat_multi([tiny], x_tiny, ACT_GGML, outs=[y_tiny], sync=False)
        tiny_launches()
        ctx.sync()
        run = (None if args.no_graph else capture(torch, stream, tiny_launches)) or tiny_launches
        for _ in range(MIN_WARMUP):
            run()
        torch.cuda.synchronize()
        launch_stats = summarize([s_ / 64 * 1e3 for s_ in timer.samples_ms(run, max(MIN_SAMPLES, args.steps))])
        launch_us = launch_stats["median"]
        out["launch_us"] = launch_stats
        log(f"[bench] smallest launch (one workgroup): {launch_us:.2f} us a launch (MAD {launch_stats['mad']:.3f})")
        tiny.free()

    # ------------------------------------------------------------------ roofline leg: dominant kernel
    ev_rows, ev_meas, ev_cal = [], [], []
    if "roofline" in legs:
        reps = max(MIN_SAMPLES, args.steps)
        per = {}
        for grp in groups:
            def all_layers(grp=grp):
                for lw in layers:
                    launch(lw, grp, not args.split_quantize)
            all_layers()
            ctx.sync()
            run = None if args.no_graph else capture(torch, stream, all_layers)
            run = run or all_layers
            for _ in range(MIN_WARMUP):
                run()
            torch.cuda.synchronize()
            samples = [s / L * 1e3 for s in timer.samples_ms(run, reps)]   # us per launch, one sample per replay
            st = summarize(samples)
            ms = st["median"] * 1e-3
            nbytes = sum(gemv_bytes(lw_t, n, k) for nm, lw_t, n, k in LAYER_TENSORS if nm in grp[1]) \
                - (len(grp[1]) - 1) * grp[2].numel() * 4      # the shared activation row is read once
            per[grp[0]] = {"us_per_launch": ms * 1e3, "mad_us": st["mad"], "rel_mad": st["rel_mad"], "samples": st["n"],
                           "bytes_per_launch": nbytes,
                           "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
            log(f"[bench] kernel {grp[0]:8s}: {ms * 1e3:7.2f} us  {per[grp[0]]['GBps']:6.0f} GB/s "
                f"({100 * per[grp[0]]['frac_hbm_peak']:.1f}% of peak)")
            qt0, rows, kk = [(t, sum(n for nm, _, n, _ in LAYER_TENSORS if nm in grp[1]), k)
                             for nm, t, n, k in LAYER_TENSORS if nm == grp[1][0]][0]
            ev_rows.append(evidence.backend_ops_row("MUL_MAT", evidence.mul_mat_params(qt0, rows, 1, kk), samples,
                                                    flops=2.0 * rows * kk, bytes_moved=nbytes,
                                                    memory_kb=nbytes // 1024, device=props.name))
            ev_meas.append(evidence.measurement(f"decode.{grp[0]}.launch", "us", samples))
            ev_cal.append(evidence.calibration_metric(qt0, False, nbytes, samples, launch_us=launch_us))
        dom = per["gate_up"]
        traffic, traffic_source = measured_traffic()
        out["roofline"] = {"bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": dom["frac_hbm_peak"], "traffic": traffic, "traffic_source": traffic_source,
                           "kernel": "gemv_decode_kernel<Q4_K, M=1>: gate+up (2 x 4096->14336) in one launch, "
                                     "activation quantized in the prologue",
                           "bytes_per_launch": dom["bytes_per_launch"], "us_per_launch": dom["us_per_launch"],
                           "statistic": "median of one sample per graph replay of the 32 layers' launches",
                           "mad_us": dom["mad_us"], "rel_mad": dom["rel_mad"], "samples": dom["samples"],
                           "launches_timed": reps * L, "launch_us": launch_us,
                           "other_kernels": {k: v for k, v in per.items() if k != "gate_up"}}
        probe = recorded_streaming_probe()
        if probe:
            out["roofline"]["streaming_probe_us"] = probe
        if args.calib_copy:
            # a plain elementwise kernel of known traffic (reads 256 MiB, writes 256 MiB) to scale the
            # FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this same command
            a = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
            b = torch.empty_like(a)
            with torch.cuda.stream(stream):
                for _ in range(5):
                    torch.add(a, 1, out=b)
            torch.cuda.synchronize()

    # ------------------------------------------------------------------ speculative-verify leg (config 3)
    if "verify" in legs:
        res = []
        for m in (2, 4, 8, 16):
            xs = {D_MODEL: torch.randn((m, D_MODEL), generator=g, device=dev),
                  D_FF: torch.randn((m, D_FF), generator=g, device=dev)}
            ys = {name: torch.empty((m, n), device=dev) for name, _, n, _ in LAYER_TENSORS}
            for gname, names in (("gate_up", ["gate", "up"]), ("down", ["down"])):
                k = {nm: kk for nm, _, _, kk in LAYER_TENSORS}[names[0]]

                def all_layers(names=names, k=k):
                    for lw in layers:
                        ctx.mul_mat_multi([lw[n] for n in names], xs[k], ACT_GGML, outs=[ys[n] for n in names], sync=False)
                def timed_layers(fn):
                    fn()
                    ctx.sync()
                    run = (None if args.no_graph else capture(torch, stream, fn)) or fn
                    for _ in range(MIN_WARMUP):
                        run()
                    torch.cuda.synchronize()
                    return summarize([s_ / L * 1e3 for s_ in timer.samples_ms(run, max(MIN_SAMPLES, args.steps))])
                st = timed_layers(all_layers)
                ms = st["median"] * 1e-3
                # the same projections through the entry point a graph reaches them by when the rows were quantized by
                # an earlier node (the norm in front writes the planes: qproj_rms_norm_quantize, then
                # qproj_mul_mat_quantized): no quantizer launch inside the timed call
                qt0 = {nm: t for nm, t, _, _ in LAYER_TENSORS}[names[0]]
                qb = torch.empty(int(lib.qproj_act_bytes(ACT_GGML, qt0, m, k)), dtype=torch.uint8, device=dev)
                ctx.quantize_activations_raw(xs[k], ACT_GGML, qt0, out=qb, sync=True)

                def all_layers_q(names=names, qb=qb):
                    for lw in layers:
                        ctx.mul_mat_quantized([lw[n] for n in names], qb, ACT_GGML, m, [ys[n] for n in names], sync=False)
                stq = timed_layers(all_layers_q)
                nbytes = sum(gemv_bytes(t, n, kk, m) for nm, t, n, kk in LAYER_TENSORS if nm in names) \
                    - (len(names) - 1) * m * k * 4
                res.append({"M": m, "group": gname, "us_per_launch": ms * 1e3, "mad_us": st["mad"], "samples": st["n"],
                            "us_rows_quantized_earlier": stq["median"], "mad_us_rows_quantized_earlier": stq["mad"],
                            "GBps": nbytes / (ms * 1e-3) / 1e9,
                            "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
                log(f"[bench] verify M={m:2d} {gname:8s}: {ms * 1e3:7.2f} us  {res[-1]['GBps']:6.0f} GB/s "
                    f"({100 * res[-1]['frac_hbm_peak']:.1f}% of peak); rows quantized by an earlier call: {stq['median']:.2f} us")
        out["verify"] = {"note": "weights read once for all M rows; ggml activation mode", "shapes": res}

    # ------------------------------------------------------------------ Q8_0 leg (config 1)
    if "q8_0" in legs:
        nrot = 24            # distinct 4096x4096 Q8_0 matrices (17.8 MB each) rotated through, > Infinity Cache
        ws = []
        for i in range(nrot):
            blocks = synth.random_weight(Q8_0, D_MODEL, D_MODEL, seed=9000 + i, device=dev)
            ws.append(ctx.upload_from_device(Q8_0, D_MODEL, D_MODEL, blocks))
            del blocks
        yq = torch.empty((1, D_MODEL), device=dev)

        def rot():
            for w in ws:
                ctx.mul_mat_multi([w], x_attn, ACT_GGML, outs=[yq], sync=False)
        rot()
        ctx.sync()
        run = (None if args.no_graph else capture(torch, stream, rot)) or rot
        for _ in range(MIN_WARMUP):
            run()
        torch.cuda.synchronize()
        stq8 = summarize([s_ / nrot * 1e3 for s_ in timer.samples_ms(run, max(MIN_SAMPLES, args.steps))])
        ms = stq8["median"] * 1e-3
        nbytes = gemv_bytes(Q8_0, D_MODEL, D_MODEL)
        out["q8_0"] = {"shape": "4096x4096, M=1", "us_per_launch": ms * 1e3, "mad_us": stq8["mad"], "samples": stq8["n"], "GBps": nbytes / (ms * 1e-3) / 1e9,
                       "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        log(f"[bench] q8_0 4096x4096 M=1: {ms * 1e3:.2f} us  {out['q8_0']['GBps']:.0f} GB/s")
        for w in ws:
            w.free()

    # ------------------------------------------------------------------ norm leg (fused neighbours of the path)
    if "norm" in legs:
        # RMS norm + norm weights in front of the gate/up projections of the 32 layers: three separate calls
        # (norm, then the projection call with its own quantizer) against the single entry point
        gamma = torch.ones(D_MODEL, device=dev) + 0.1 * torch.randn(D_MODEL, device=dev)
        res = {}
        for m in (1, 512):
            xn = torch.randn((m, D_MODEL), device=dev)
            xnormed = torch.empty_like(xn)
            yg = [torch.empty((m, D_FF), device=dev) for _ in range(2)]

            def separate():
                for lw in layers:
                    ctx.rms_norm(xn, gamma, 1e-5, out=xnormed, sync=False)
                    ctx.mul_mat_multi([lw["gate"], lw["up"]], xnormed, ACT_GGML, outs=yg, sync=False)

            def fused():
                for lw in layers:
                    ctx.rms_norm_mul_mat([lw["gate"], lw["up"]], xn, gamma, 1e-5, ACT_GGML, outs=yg, sync=False)

            hbuf = torch.empty((m, D_FF), device=dev)

            def separate_ffn():   # ... and the swiglu that joins gate and up, as one more elementwise launch
                for lw in layers:
                    ctx.rms_norm(xn, gamma, 1e-5, out=xnormed, sync=False)
                    ctx.mul_mat_multi([lw["gate"], lw["up"]], xnormed, ACT_GGML, outs=yg, sync=False)
                    torch.mul(torch.nn.functional.silu(yg[0]), yg[1], out=hbuf)

            def fused_ffn():
                for lw in layers:
                    ctx.ffn_gate_up(lw["gate"], lw["up"], xn, ACT_GGML, gamma=gamma, eps=1e-5, out=hbuf, sync=False)

            row = {}
            for name, f in (("separate", separate), ("fused", fused), ("separate_swiglu", separate_ffn), ("fused_swiglu", fused_ffn)):
                if name == "separate_swiglu" and not args.no_graph:
                    continue   # torch's elementwise launches are on torch's stream: only timed in eager mode
                f()
                ctx.sync()
                run = (None if args.no_graph else capture(torch, stream, f)) or f
                run()
                torch.cuda.synchronize()
                row[name + "_us"] = timer.time_ms(run, max(5, args.steps)) / len(layers) * 1e3
            res[f"M={m}"] = row
            log(f"[bench] norm + gate/up, M={m}: separate calls {row['separate_us']:.1f} us, one call {row['fused_us']:.1f} us per layer; "
                f"with swiglu in the same call {row['fused_swiglu_us']:.1f} us")
        out["norm"] = res

    # ------------------------------------------------------------------ prefill leg (config 4)
    if "prefill" in legs:
        res = []
        for (k, n) in ((4096, 14336), (14336, 4096), (4096, 4096)):
            blocks = synth.random_weight(Q4_K, n, k, seed=77 + n, device=dev)
            w = ctx.upload_from_device(Q4_K, k, n, blocks)
            del blocks
            for m in (512, 2048, 4096):
                x = torch.randn((m, k), generator=g, device=dev)
                cols = torch.randperm(k, generator=g, device=dev)[: k // 100]
                x[:, cols] *= 20.0
                yb = torch.empty((m, n), device=dev)
                qb = torch.empty(int(lib.qproj_act_bytes(ACT_Q8X32, Q4_K, m, k)), dtype=torch.uint8, device=dev)
                torch.cuda.synchronize()
                fq = lambda: ctx.quantize_activations_raw(x, ACT_Q8X32, Q4_K, out=qb, sync=False)
                fg = lambda: ctx.mul_mat_quantized([w], qb, ACT_Q8X32, m, [yb], sync=False)
                for _ in range(MIN_WARMUP):
                    fq(); fg()
                ctx.sync()
                tq = median(timer.samples_ms(fq, MIN_SAMPLES))
                sg = timer.samples_ms(fg, MIN_SAMPLES)
                stg = summarize(sg)
                tg = stg["median"]
                ops = 2.0 * m * n * k
                ev_rows.append(evidence.backend_ops_row("MUL_MAT", evidence.mul_mat_params(Q4_K, n, m, k) + ",act=q8x32",
                                                        [s * 1e3 for s in sg], flops=ops,
                                                        bytes_moved=gguf_bytes(Q4_K, n, k) + m * k + m * n * 4,
                                                        memory_kb=(gguf_bytes(Q4_K, n, k) + m * n * 4) // 1024,
                                                        device=props.name))
                res.append({"M": m, "K": k, "N": n, "gemm_ms": tg, "gemm_mad_ms": stg["mad"], "rel_mad": stg["rel_mad"], "quantize_ms": tq,
                            "gemm_tops": ops / (tg * 1e-3) / 1e12,
                            "end_to_end_tops": ops / ((tg + tq) * 1e-3) / 1e12,
                            "frac_int8_peak": ops / (tg * 1e-3) / 1e12 / INT8_PEAK_TOPS})
                log(f"[bench] prefill M={m} K={k} N={n}: gemm {tg:.3f} ms = {res[-1]['gemm_tops']:.1f} TOPS "
                    f"({100 * res[-1]['frac_int8_peak']:.1f}% of int8 peak), quantize {tq:.3f} ms")
                del x, yb, qb
            w.free()
        head = [r for r in res if (r["M"], r["K"], r["N"]) == (4096, 4096, 14336)][0]
        out["prefill"] = {"act_format": "per-32 int8 + fp32 scale", "mfma": "v_mfma_i32_32x32x32_i8",
                          "headline_tops": head["gemm_tops"], "headline_frac_int8_peak": head["frac_int8_peak"],
                          "headline_rel_mad": head["rel_mad"], "samples_per_shape": MIN_SAMPLES, "statistic": "median",
                          # What bounds this format (not the matrix cores): both operands change scale every 32 weights, so
                          # an int32 result is good for ONE matrix instruction and each of its 16 outputs a lane costs
                          # convert + scale product + fma on the vector ALU: 48 vector instructions behind every
                          # 32 x 32 x 32 product (52.8 measured with addresses and loads).  With a matrix instruction holding
                          # the issue port 16 of its 32 cycles and a vector instruction 4, the floor is
                          # 5000 TOPS x 32 / (16 + 4 x 52.8) = 704 TOPS (profiles/prefill_gemm_kernels.txt, section 2).
                          "bound": "valu", "floor_tops": 704.0,
                          "floor": "5000 x 32 / (16 + 4 x 52.8): 48 of 52.8 vector instr. per matrix instr. are the per-32 flush",
                          "peak_tops": INT8_PEAK_TOPS, "shapes": res}
        # the same shapes in the ggml activation format (Q8_K, one scale per 256): the reference's own arithmetic
        # (plus the layer's Q6_K down projection, which a Q4_K_M model runs through the same operator, and
        # config 1's Q8_0 matrix with ggml's Q8_0 activation blocks)
        resg = []
        for (qt, k, n) in ((Q4_K, 4096, 14336), (Q4_K, 14336, 4096), (Q4_K, 4096, 4096), (Q6_K, 14336, 4096),
                           (Q8_0, 4096, 4096)):
            blocks = synth.random_weight(qt, n, k, seed=77 + n, device=dev)
            w = ctx.upload_from_device(qt, k, n, blocks)
            del blocks
            for m in (512, 2048, 4096):
                x = torch.randn((m, k), generator=g, device=dev)
                yb = torch.empty((m, n), device=dev)
                qb = torch.empty(int(lib.qproj_act_bytes(ACT_GGML, qt, m, k)), dtype=torch.uint8, device=dev)
                torch.cuda.synchronize()
                fq = lambda: ctx.quantize_activations_raw(x, ACT_GGML, qt, out=qb, sync=False)
                fg = lambda: ctx.mul_mat_quantized([w], qb, ACT_GGML, m, [yb], sync=False)
                for _ in range(MIN_WARMUP):
                    fq(); fg()
                ctx.sync()
                tq = median(timer.samples_ms(fq, MIN_SAMPLES))
                sg = timer.samples_ms(fg, MIN_SAMPLES)
                stg = summarize(sg)
                tg = stg["median"]
                ops = 2.0 * m * n * k
                ev_rows.append(evidence.backend_ops_row("MUL_MAT", evidence.mul_mat_params(qt, n, m, k),
                                                        [s * 1e3 for s in sg], flops=ops,
                                                        bytes_moved=gguf_bytes(qt, n, k) + m * k * 4 + m * n * 4,
                                                        memory_kb=(gguf_bytes(qt, n, k) + m * n * 4) // 1024,
                                                        device=props.name))
                tname = {Q4_K: "Q4_K", Q6_K: "Q6_K", Q8_0: "Q8_0"}[qt]
                resg.append({"type": tname, "M": m, "K": k, "N": n, "gemm_ms": tg, "gemm_mad_ms": stg["mad"], "rel_mad": stg["rel_mad"], "quantize_ms": tq,
                             "gemm_tops": ops / (tg * 1e-3) / 1e12,
                             "frac_int8_peak": ops / (tg * 1e-3) / 1e12 / INT8_PEAK_TOPS})
                log(f"[bench] prefill(ggml acts) {tname} M={m} K={k} N={n}: gemm {tg:.3f} ms = {resg[-1]['gemm_tops']:.1f} TOPS "
                    f"({100 * resg[-1]['frac_int8_peak']:.1f}% of int8 peak), quantize {tq:.3f} ms")
                del x, yb, qb
            w.free()
        headg = [r for r in resg if (r["type"], r["M"], r["K"], r["N"]) == ("Q4_K", 4096, 4096, 14336)][0]
        out["prefill_ggml_acts"] = {"act_format": "ggml Q8_K (int8 + fp32 scale per 256, block sums)",
                                    "mfma": "Q4_K: 2 x v_mfma_i32_32x32x32_i8 per sub-block (scale split in base 8); "
                                            "Q6_K: v_mfma_i32_32x32x16_i8 per sub-block, integer scale on the vector ALU; "
                                            "Q8_0: v_mfma_i32_32x32x32_i8 per block, fp32 scales",
                                    "headline_tops": headg["gemm_tops"], "headline_frac_int8_peak": headg["frac_int8_peak"],
                                    "headline_rel_mad": headg["rel_mad"], "samples_per_shape": MIN_SAMPLES, "statistic": "median",
                                    "shapes": resg}

    # ------------------------------------------------------------------ MoE leg (config 5)
    if "moe" in legs:
        # Three distinct sets of expert weights (3 x 340 MB) and several draws of expert ids are rotated through, so
        # that more than a gigabyte of experts cycles between two uses of the same bytes: the 256 MB Infinity Cache
        # cannot hold them and the rate is an HBM rate.  One id draw replayed on one set (at most 340 MB, 21 MB at
        # B = 1) is reported beside it as the cache-resident figure.
        E, top, dm, dff, ncopy = 128, 8, 2048, 768, 3
        sets = []
        for c in range(ncopy):
            exps = {}
            for i, (name, n, k) in enumerate((("gate", dff, dm), ("up", dff, dm), ("down", dm, dff))):
                blocks = synth.random_weight(Q4_K, E * n, k, seed=500 + 10 * c + i, device=dev)
                exps[name] = ctx.upload_from_device(Q4_K, k, n, blocks, n_expert=E)
                del blocks
            sets.append(exps)
        per_expert = 2 * gguf_bytes(Q4_K, dff, dm) + gguf_bytes(Q4_K, dm, dff)
        res = []
        for B in (1, 8, 64):
            ndraw = {1: 16, 8: 4, 64: 2}[B]
            if B == 1:      # sixteen disjoint draws of eight experts cover all 128
                perm = torch.randperm(E, generator=g, device=dev).to(torch.int32)
                draws = [perm[top * d: top * (d + 1)].reshape(1, top).contiguous() for d in range(ndraw)]
            else:
                draws = [torch.stack([torch.randperm(E, generator=g, device=dev)[:top] for _ in range(B)]).to(torch.int32)
                         for _ in range(ndraw)]
            wts = torch.softmax(torch.randn((B, top), generator=g, device=dev), dim=1)
            x = torch.randn((B, dm), generator=g, device=dev)
            calls = [(c, d) for d in range(ndraw) for c in range(ncopy)]
            distinct = [int(torch.unique(draws[d]).numel()) for c, d in calls]
            cycled = ncopy * int(torch.unique(torch.cat([d.flatten() for d in draws])).numel()) * per_expert
            torch.cuda.synchronize()
            yb = torch.empty((B, dm), device=dev)

            def rotation():
                for c, d in calls:
                    ctx.moe_ffn(sets[c]["gate"], sets[c]["up"], sets[c]["down"], x, draws[d], wts, ACT_GGML, out=yb, sync=False)

            def resident():
                ctx.moe_ffn(sets[0]["gate"], sets[0]["up"], sets[0]["down"], x, draws[0], wts, ACT_GGML, out=yb, sync=False)

            rotation(); ctx.sync()
            run = (None if args.no_graph else capture(torch, stream, rotation)) or rotation
            run(); torch.cuda.synchronize()
            for _ in range(MIN_WARMUP - 1):
                run()
            torch.cuda.synchronize()
            sm_ = [s_ / len(calls) for s_ in timer.samples_ms(run, MIN_SAMPLES)]     # ms per call, one sample per rotation
            stm = summarize(sm_)
            ms = stm["median"]
            byts = sum(distinct) / len(calls) * per_expert + B * dm * 4 * 2  # mean distinct-expert bytes of a call
            run1 = (None if args.no_graph else capture(torch, stream, resident)) or resident
            run1(); torch.cuda.synchronize()
            ms1 = timer.time_ms(run1, 100)
            byts1 = distinct[0] * per_expert + B * dm * 4 * 2
            ev_rows.append(evidence.backend_ops_row("MUL_MAT_ID", evidence.mul_mat_id_params(Q4_K, dff, dm, E, top, B) +
                                                    ",fused=moe_ffn(gate,up,swiglu,down,combine)", [s_ * 1e3 for s_ in sm_],
                                                    flops=2.0 * B * top * 3 * dm * dff, bytes_moved=byts,
                                                    memory_kb=int(byts) // 1024, device=props.name))
            ev_cal.append(evidence.calibration_metric(Q4_K, True, byts, [s_ * 1e3 for s_ in sm_], launch_us=launch_us))
            res.append({"B": B, "distinct_experts_mean": sum(distinct) / len(calls), "calls_in_rotation": len(calls),
                        "bytes_cycled": cycled, "ms": ms, "mad_ms": stm["mad"], "rel_mad": stm["rel_mad"], "samples": stm["n"],
                        "GBps": byts / (ms * 1e-3) / 1e9,
                        "frac_hbm_peak": byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "cache_resident": {"ms": ms1, "GBps": byts1 / (ms1 * 1e-3) / 1e9, "bytes": byts1}})
            log(f"[bench] moe B={B}: {ms * 1e3:.1f} us a call over a rotation of {len(calls)} calls cycling {cycled / 1e6:.0f} MB "
                f"({res[-1]['GBps']:.0f} GB/s from HBM); one draw replayed: {ms1 * 1e3:.1f} us ({res[-1]['cache_resident']['GBps']:.0f} GB/s, "
                f"{byts1 / 1e6:.0f} MB, may sit in the Infinity Cache)")
        out["moe"] = {"experts": E, "top": top, "d_model": dm, "d_ff": dff, "batches": res,
                      "note": "2 launches per call up to 256 pairs (gate/up+SwiGLU, down+combine: an expert read per pair, rows "
                              "quantized in the prologue), else 5 (group+quantize, gate/up+SwiGLU, quantize, down, combine); "
                              "the rotation over three weight sets and several id draws is replayed as one "
                              "HIP graph; GBps counts the distinct experts of each call"}
        for exps in sets:
            for w in exps.values():
                w.free()

    # ------------------------------------------------------------------ CPU baseline (oracle, host cores)
    if "cpu" in legs:
        from oracle import oracle as orc
        import numpy as np
        orc.build()
        nl = L                       # every layer of the step: 4.4 GB of blocks on the host, far beyond its caches
        host = [[(qt, n, k, ctx.download(layers[l][name])) for name, qt, n, k in LAYER_TENSORS] for l in range(nl)]
        xs = {D_MODEL: x_attn.cpu().numpy(), D_FF: x_down.cpu().numpy()}
        # One thread a physical core, the reference's own policy (inference/parity/profiles/pr.toml:41), counted from
        # /sys over the CPUs this process may run on and capped by the 16 CPUs a one-GPU box gives a job.  AVX2 dot
        # products in the shape of ggml's x86 path when the oracle was built with them, the generic C loops otherwise.
        phys, logical = physical_cores()
        threads = max(1, min(phys, orc.max_threads(), 16))
        avx2 = orc.has_avx2()
        run_cpu = (lambda qt, blocks, k, th: orc.time_mul_mat_avx2(qt, blocks, k, xs[k], th, 1)) if avx2 else \
                  (lambda qt, blocks, k, th: orc.time_mul_mat(qt, blocks, k, xs[k], orc.ACT_GGML, th, 1))
        t_end = time.time() + args.cpu_seconds
        pass_s = []                                # seconds of arithmetic per pass over the layers
        while len(pass_s) < 2 or time.time() < t_end:
            t_pass = 0.0
            for lw in host:
                for qt, n, k, blocks in lw:
                    t_pass += run_cpu(qt, blocks, k, threads)
            pass_s.append(t_pass)
        passes, spent = len(pass_s), sum(pass_s)
        stc = summarize(pass_s)
        cpu_gbs = nl * LAYER_BYTES / stc["median"] / 1e9
        one = 0.0                                  # one thread, one layer
        for qt, n, k, blocks in host[0]:
            one += run_cpu(qt, blocks, k, 1)
        scalar_one = 0.0                           # the same with the generic C loops the parity tests use
        for qt, n, k, blocks in host[0]:
            scalar_one += orc.time_mul_mat(qt, blocks, k, xs[k], orc.ACT_GGML, 1, 1)
        out["cpu_baseline"] = {"value": cpu_gbs, "unit": "GB/s", "cores": threads, "kind": "port",
                               "sample": f"{passes} passes over the same {nl} layers (7 projections each, M=1, ggml activation "
                                         f"mode; median pass), {spent:.1f} s on the host",
                               "rel_mad": stc["rel_mad"], "thread_policy": "physical-cores, at most the box's 16-CPU share",
                               "host_physical_cores": phys, "host_logical_cpus": logical,
                               "isa": "AVX2 maddubs/madd dot products, OpenMP over rows" if avx2 else "generic C, OpenMP over rows",
                               "host_cpus": os.cpu_count(),
                               "one_thread_GBps": LAYER_BYTES / one / 1e9,
                               "one_thread_generic_c_GBps": LAYER_BYTES / scalar_one / 1e9}
        log(f"[bench] cpu baseline: {cpu_gbs:.2f} GB/s on {threads} threads ({phys} physical cores, {logical} logical CPUs usable)")

    # ------------------------------------------------------------------ llama-bench style leg
    # pp512 / tg128 over the projections of all layers (no attention, norms or sampling): the prompt
    # pass is one 512-token batch per layer tensor group, generation is 128 single-token steps.
    if "llama_bench" in legs:
        n_prompt, n_gen, reps = 512, 128, 10       # the reference's gate takes the median of 10 (generation-128.json:44-51)
        xs = {kk: torch.randn((n_prompt, kk), generator=g, device=dev) for kk in (D_MODEL, D_FF)}
        yp = {name: torch.empty((n_prompt, n), device=dev) for name, _, n, _ in LAYER_TENSORS}

        def prompt_pass():
            for lw in layers:
                for _, names, x1, _ in groups:
                    ctx.mul_mat_multi([lw[nm] for nm in names], xs[x1.shape[1]], ACT_GGML,
                                      outs=[yp[nm] for nm in names], sync=False)

        def timed(fn):
            fn(); ctx.sync(); torch.cuda.synchronize()
            t0 = time.perf_counter_ns()
            fn(); ctx.sync(); torch.cuda.synchronize()
            return time.perf_counter_ns() - t0

        def generate():
            for _ in range(n_gen):
                step()
                ctx.sync()            # llama-bench synchronizes after every generated token

        cfg = {"batch_size": n_prompt, "ubatch_size": n_prompt, "n_gpu_layers": L, "split_mode": "none", "main_gpu": 0,
               "flash_attention": False, "warmup": True, "actual_backends": ["qproj-hip"],
               "scope": "projection operators only (q,k,v,o,gate,up Q4_K; down Q6_K), ggml activation format"}
        devs = [{"name": props.name, "backend": "ROCm", "index": 0}]
        pp = [timed(prompt_pass) for _ in range(reps)]
        tg = [timed(generate) for _ in range(reps)]
        rec_pp = evidence.llama_bench_record("llama-bench.prompt-processing", n_prompt, 1, 0, 0, pp, cfg, devs)
        rec_tg = evidence.llama_bench_record("llama-bench.token-generation", 0, 0, n_gen, n_gen, tg, cfg, devs)
        out["llama_bench"] = [rec_pp, rec_tg]
        med = median
        log(f"[bench] llama-bench style, projections only: pp{n_prompt} {n_prompt * 1e9 / med(pp):.0f} tok/s "
            f"({med(pp) / 1e6:.2f} ms), tg{n_gen} {n_gen * 1e9 / med(tg):.0f} tok/s ({med(tg) / 1e6:.1f} ms)")

    if ev_rows:
        # the reference's own record shapes (test-backend-ops rows, parity measurements, fit calibration)
        out["evidence"] = {"backend_ops": ev_rows, "measurements": ev_meas, "calibration": ev_cal}
        if args.evidence_sql:
            with open(args.evidence_sql, "w") as f:
                f.write("\n".join(evidence.backend_ops_sql(r) for r in ev_rows) + "\n")
    details = None
    if args.details_json:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.details_json)), exist_ok=True)
            with open(args.details_json, "w") as f:
                json.dump(out, f, indent=1)
            details = args.details_json
        except OSError as e:
            log(f"[bench] details file not written: {e}")
    print(compact_line(out, details), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
