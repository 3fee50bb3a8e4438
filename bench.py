#!/usr/bin/env python3
"""Benchmark of the W4A16 GEMM path on one MI355X.

A "step" is one pass over the Llama-2-7B decode layer set: the four layer GEMMs
(qkv, o, gate_up + SiLU, down + residual) at each of T = 1, 4, 8, 16 tokens = 16 launches.
Every one of the 16 GEMMs of a step has its own copy of its weight matrix, and the steps rotate
through 12 such sets (48 copies per shape, about 5 GB of packed weights), so that no matrix is
read again before several GB of other traffic have passed: neither the L2s nor the 256 MB
Infinity Cache can serve the weights.  The headline value is the aggregate achieved bandwidth:
algorithmic bytes of all launches / elapsed time.

Also in the same JSON line: roofline objects for the dominant decode kernel (gate_up) and for the
one furthest below its roofline (o), per-shape tables for Llama-2-7B and Llama-2-70B (decode:
GB/s; T = 2048: TFLOP/s), the 32-layer decode step at M = 8 as one launch per GEMM and as
persistent launches, the socket power and engine clocks read while the prefill kernel runs for
four seconds (the part sits at its power limit and well below the 2.4 GHz of its quoted peak), what
plain library kernels reach on this GPU (streaming reads of 8 / 45 /
512 MiB, a device copy, a dense fp16 GEMM), and the CPU baseline (the oracle: unpack,
dequantise, torch fp32 matmul) timed on the host cores on bounded samples.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0    # MI355X dense fp16 matrix

# HBM bytes per launch of the two dominant kernels and of the o decode kernel, from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`
# runs of `bench.py --probe ...`, calibrated against an elementwise kernel of known size
# (profiles/decode_gate_up_hbm_traffic.md, profiles/prefill_gate_up_mfma_and_traffic.md).
N_LAYERS = 32          # Llama-2-7B
TRAFFIC_DECODE_GATE_UP = 49.36e6
TRAFFIC_DECODE_O = 10.02e6
TRAFFIC_PREFILL_GATE_UP = 567.5e6

# name, K, N (gate_up: both halves), epilogue
LAYER_7B = [("qkv", 4096, 12288, 0), ("o", 4096, 4096, 0), ("gate_up", 4096, 22016, 1), ("down", 11008, 4096, 2)]
LAYER_70B = [("qkv", 8192, 10240, 0), ("o", 8192, 8192, 0), ("gate_up", 8192, 57344, 1), ("down", 28672, 8192, 2)]
DECODE_T = (1, 4, 8, 16)
DECODE_T_70B = (1, 16)
PREFILL_T = 2048
BATCHED_T = (32, 64, 128, 256)   # reported per shape, outside the headline metric
GROUP = 128


def algorithmic_bytes(T, K, N, epi):
    """int4 weights + fp16 scales + int4 zeros + activations + output (+ residual)."""
    G = K // GROUP
    n_out = N // 2 if epi == 1 else N
    b = K * N // 2 + G * N * 2 + G * N // 2 + T * K * 2 + T * n_out * 2
    if epi == 2:
        b += T * N * 2
    return b


def flops(T, K, N):
    return 2 * T * K * N


def make_weights(tm, torch, gen, name, K, N):
    """One copy of a layer matrix in the library's layout, from synthetic AWQ tensors on the GPU."""
    G = K // GROUP
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, device="cuda", generator=gen)
    s = (torch.randn((G, N), device="cuda", generator=gen).abs() * 0.01 + 1e-3).half()
    if name == "gate_up":  # w1 and w3 (each [K, N/2]) interleaved by the repack path, as deploy does
        fused = torch.empty_like(qw)
        tm.fuse_w1_w3_s4_k_m8(qw.view(2 * K, N // 16), fused, N // 2, K)
        qw = fused
    A = torch.empty_like(qw)
    Q = torch.empty((G, N), dtype=torch.int32, device="cuda")
    tm.convert_s4_k_m8(A, Q, s, qw, s, qz, N, K, GROUP)
    return A, Q


def read_power_and_clocks():
    """Socket power and per-XCD engine clocks from `amd-smi metric --power --clock` (a sensor read; a child
    process, so that nothing is started in place of this one)."""
    import re
    import subprocess
    tool = "amd-smi metric --power --clock"
    try:
        out = subprocess.run(tool.split(), capture_output=True, text=True, timeout=30).stdout
    except (OSError, subprocess.SubprocessError) as e:
        return {"tool": tool, "error": str(e)[:200]}
    power = re.search(r"SOCKET_POWER:\s*(\d+)\s*W", out)
    clocks = [int(m) for m in re.findall(r"GFX_\d+:\s*\n\s*CLK:\s*(\d+)\s*MHz", out)]
    if not power and not clocks:
        return {"tool": tool, "error": "no power or clock figures in the tool's output"}
    return {"tool": tool, "socket_power_W": int(power.group(1)) if power else None, "gfx_clk_MHz": clocks,
            "mean_gfx_clk_MHz": round(sum(clocks) / len(clocks), 1) if clocks else None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=96)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--repeats", type=int, default=9,
                    help="the timed region of --steps steps is measured this many times in a row; the median is reported")
    ap.add_argument("--steps-per-graph", type=int, default=0,
                    help="steps captured into one HIP graph (must divide --steps; 0 = 4, or else 5, 3, 2 or 1, whichever "
                         "divides --steps first); a decode step of a whole model is one "
                         "graph of hundreds of launches, so what one graph launch costs is spread thinner there")
    ap.add_argument("--copies", type=int, default=12,
                    help="distinct sets of 16 weight matrices (one per GEMM of a step) the steps rotate through")
    ap.add_argument("--cold-gib", type=float, default=1.25,
                    help="per-shape measurements rotate through at least this many GiB of weight copies")
    ap.add_argument("--eager", action="store_true", help="launch from the host instead of replaying HIP graphs")
    ap.add_argument("--prefill-steps", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-per-shape", action="store_true")
    ap.add_argument("--no-70b", action="store_true")
    ap.add_argument("--no-sustained", action="store_true", help="skip the power / clock reading under a sustained prefill load")
    ap.add_argument("--sustained-seconds", type=float, default=4.0)
    ap.add_argument("--seconds", type=float, default=8.0, help="duration of the sustain-* probes")
    ap.add_argument("--probe", choices=["decode", "prefill", "decode-o", "decode-70b", "sustain-prefill",
                                        "sustain-decode", "sustain-dense"],
                    help="decode / prefill / decode-o: run only the named kernel (gate_up decode / gate_up at T=2048 / o "
                         "decode) plus a plain 256 MiB elementwise kernel, eagerly, for `rocprofv3 --pmc` (no JSON line).  "
                         "decode-70b: the same for the Llama-2-70B gate_up and down decode kernels at T=1 and T=16.  "
                         "sustain-prefill / sustain-decode / sustain-dense: "
                         "keep launching gate_up (T=2048 / T=8 / torch.matmul fp16 at T=2048) for --seconds and print the "
                         "rate once a second, so that the engine clock under that load can be read beside it "
                         "(`rocm-smi --showclocks`)")
    args = ap.parse_args()
    if args.steps_per_graph == 0:
        args.steps_per_graph = next(s for s in (4, 5, 3, 2, 1) if args.steps % s == 0)
    if args.steps < 1 or args.steps_per_graph < 1 or args.steps % args.steps_per_graph:
        print("bench.py: --steps-per-graph must divide --steps", file=sys.stderr)
        sys.exit(2)
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import lmdeploy_amd.turbomind as tm

    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(20240611)
    gemm = tm.GemmS4F16()
    stream = torch.cuda.Stream()          # default priority; graphs are captured and replayed on it
    shape = {name: (K, N, epi) for name, K, N, epi in LAYER_7B}
    n_sets = args.copies
    weights = {}
    for name, K, N, epi in LAYER_7B:
        per_copy = K * N // 2 + (K // GROUP) * N * 4
        n = max(len(DECODE_T) * n_sets, N_LAYERS, int(args.cold_gib * 2 ** 30 / per_copy) + 1)
        if args.probe == "decode-70b":
            n = 1
        elif args.probe:
            n = max(8, int(args.cold_gib * 2 ** 30 / per_copy) + 1) if name in ("gate_up", "o") else 1
        weights[name] = [make_weights(tm, torch, gen, name, K, N) for _ in range(n)]
    Tmax = max(max(DECODE_T), PREFILL_T)
    X = {K: torch.randn((Tmax, K), device="cuda", generator=gen).half() for K in (4096, 11008)}
    Res = torch.randn((Tmax, 4096), device="cuda", generator=gen).half()
    out = {name: torch.empty((Tmax, N // 2 if epi == 1 else N), dtype=torch.float16, device="cuda")
           for name, K, N, epi in LAYER_7B}
    # the kernels that split K need the handle's workspace, which cannot be allocated during graph capture
    gemm.Run(out["down"], *weights["down"][0][:1], X[11008], weights["down"][0][1], 4096, 64, 11008, GROUP, 2, -1,
             residual=Res)
    torch.cuda.synchronize()

    def launch(name, copy, T, st):
        K, N, epi = shape[name]
        A, Q = weights[name][copy % len(weights[name])]
        gemm.Run(out[name], A, X[K], Q, N, T, K, GROUP, epi, -1, residual=Res if epi == 2 else None, stream=st)

    def make_runner(work, fn=None):
        """work: list of launch lists; returns one callable per entry (a replayable HIP graph)."""
        fn = fn or (lambda w, st: [launch(n, c, T, st) for n, c, T in w])
        if args.eager:
            return [lambda w=w: fn(w, stream.cuda_stream) for w in work]
        runners = []
        for w in work:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                keep = fn(w, torch.cuda.current_stream().cuda_stream)
            runners.append(lambda g=g, keep=keep: g.replay())
        return runners

    def timed_all(runner, steps, warmup, repeats):
        """`warmup` untimed calls, then `repeats` timed regions of exactly `steps` calls each (HIP events on the
        stream the graphs replay on, a synchronisation on both sides of every region); ms per region."""
        out, n = [], 0
        with torch.cuda.stream(stream):
            for _ in range(warmup):
                runner[n % len(runner)]()
                n += 1
            for _ in range(repeats):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record(stream)
                for _ in range(steps):
                    runner[n % len(runner)]()
                    n += 1
                e1.record(stream)
                torch.cuda.synchronize()
                out.append(e0.elapsed_time(e1))
        return out

    def timed(runner, steps, warmup, repeats=1):
        """Median over `repeats` timed regions of `steps` calls, in ms per region."""
        ms = sorted(timed_all(runner, steps, warmup, repeats))
        return ms[len(ms) // 2]

    def kernel_clock(work, fn=None, steps=3):
        """The engine clock inside the kernels of `work` (a launch list as for make_runner): the graph is captured and
        replayed with the library's clock recording on, apart from the timed regions."""
        gemm.clock_begin(stream.cuda_stream)
        r = make_runner([work], fn)
        timed(r, steps, 1, 1)
        c = gemm.clock_end(stream.cuda_stream)
        return {"MHz": round(c["MHz"]), "kernel_us": round(c["us_per_launch"], 2)} if c["launches"] else None

    if args.probe and args.probe.startswith("sustain-"):
        K, N, _ = shape["gate_up"]
        T = 8 if args.probe == "sustain-decode" else PREFILL_T
        dense_w = torch.randn(K, N, device="cuda", generator=gen).half() if args.probe == "sustain-dense" else None
        dense_out = torch.empty(T, N, dtype=torch.float16, device="cuda") if dense_w is not None else None
        n, per = len(weights["gate_up"]), 2000 if T == 8 else 200
        t_end, t0, shown = time.time() + args.seconds, time.time(), -1
        while time.time() < t_end:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with torch.cuda.stream(stream):
                e0.record()
                for c in range(per):
                    if dense_w is not None:
                        torch.matmul(X[K][:T], dense_w, out=dense_out)
                    else:
                        launch("gate_up", c % n, T, stream.cuda_stream)
                e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / per
            if int(time.time() - t0) == shown:
                continue
            shown = int(time.time() - t0)
            print("%s t=%4.1fs  %7.1f us/launch  %6.0f TFLOP/s  %6.0f GB/s" % (
                args.probe, time.time() - t0, us, 2.0 * T * K * N / us / 1e6,
                algorithmic_bytes(T, K, N, 0 if dense_w is not None else 1) / us / 1e3), flush=True)
        return

    if args.probe == "decode-70b":
        # calibration kernel, then gate_up (strips of 7 tiles, SiLU) and down (strips of 2, residual) of Llama-2-70B,
        # every weight copy once at T = 1 and once at T = 16, cold
        src = torch.zeros(64 * 2 ** 20, dtype=torch.int32, device="cuda")   # 256 MiB
        dst = torch.empty_like(src)
        X70 = {K: torch.randn((16, K), device="cuda", generator=gen).half() for K in (8192, 28672)}
        Res70 = torch.randn((16, 8192), device="cuda", generator=gen).half()
        with torch.cuda.stream(stream):
            for _ in range(4):
                torch.add(src, 1, out=dst)
        done = []
        for name, K, N, epi in LAYER_70B:
            if name not in ("gate_up", "down"):
                continue
            n = max(3, int(args.cold_gib * 2 ** 30 / (K * N // 2 + (K // GROUP) * N * 4)) + 1)
            ws = [make_weights(tm, torch, gen, name, K, N) for _ in range(n)]
            C = torch.empty((16, N // 2 if epi == 1 else N), dtype=torch.float16, device="cuda")
            with torch.cuda.stream(stream):
                for T in (1, 16):
                    for A, Q in ws:
                        gemm.Run(C, A, X70[K], Q, N, T, K, GROUP, epi, -1, residual=Res70 if epi == 2 else None,
                                 stream=stream.cuda_stream)
            torch.cuda.synchronize()
            done.append("%d %s launches at T=1 and as many at T=16" % (n, name))
            del ws
        print("probe done: 4 add kernels over 268435456 bytes, " + ", ".join(done))
        return

    if args.probe:
        # a plain elementwise kernel of known size calibrates FETCH_SIZE / WRITE_SIZE, then the kernel on cold weights
        src = torch.zeros(64 * 2 ** 20, dtype=torch.int32, device="cuda")   # 256 MiB
        dst = torch.empty_like(src)
        name = "o" if args.probe == "decode-o" else "gate_up"
        with torch.cuda.stream(stream):
            for _ in range(4):
                torch.add(src, 1, out=dst)   # reads 256 MiB, writes 256 MiB
            n = len(weights[name])
            for rep in range(2):
                for c in range(n):
                    launch(name, c, PREFILL_T if args.probe == "prefill" else DECODE_T[c % len(DECODE_T)], stream.cuda_stream)
        torch.cuda.synchronize()
        print("probe done: 4 add kernels over 268435456 bytes, %d %s launches (%s)" % (2 * n, name, args.probe))
        return

    # ---- headline: the decode layer set; every GEMM of a step has its own weight copy ----------
    step_bytes = sum(algorithmic_bytes(T, K, N, epi) for T in DECODE_T for _, K, N, epi in LAYER_7B)
    def set_work(c):
        return [(name, len(DECODE_T) * c + ti, T) for ti, T in enumerate(DECODE_T) for name, _, _, _ in LAYER_7B]

    S = args.steps_per_graph
    runner = make_runner([sum((set_work((g * S + j) % n_sets) for j in range(S)), []) for g in range(n_sets)])
    # One timed region of `steps` steps lasts a few milliseconds and cannot resolve a 3 % change; the region is
    # therefore timed `--repeats` times in a row and the median region is the one reported.
    regions = sorted(timed_all(runner, args.steps // S, max(1, args.warmup // S), args.repeats))
    ms = regions[len(regions) // 2]
    ms_per_step = ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    timing = {"regions": args.repeats, "steps_per_region": args.steps, "reported": "median region",
              "min_ms_per_step": round(regions[0] / args.steps, 5), "max_ms_per_step": round(regions[-1] / args.steps, 5)}

    def per_launch_us(name, tokens, passes=3, repeats=3):
        """Average time of one launch of `name`, rotating through all of its copies (cold weights); median of
        `repeats` regions of `passes` rounds."""
        n = len(weights[name])
        r = make_runner([[(name, c, tokens[c % len(tokens)]) for c in range(n)]])
        return timed(r, passes, 1, repeats) * 1e3 / (passes * n)

    def decode_roofline(name, traffic, what):
        K, N, epi = shape[name]
        by = sum(algorithmic_bytes(T, K, N, epi) for T in DECODE_T) / len(DECODE_T)
        us = per_launch_us(name, DECODE_T, passes=4, repeats=7)
        ach = by / (us * 1e-6) / 1e9
        return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": traffic, "kernel": what,
                "bytes_per_launch": int(by), "us_per_launch": round(us, 3),
                "us_per_launch_is": "median of 7 regions of 4 rounds over all weight copies"}

    # ---- rooflines: the dominant decode kernel (gate_up) and the one furthest below its roofline (o) ----
    roofline = decode_roofline("gate_up", TRAFFIC_DECODE_GATE_UP,
                               "strip_kernel, gate_up K=4096 N=22016 +SiLU, T cycling over {1,4,8,16}")
    roofline_worst = decode_roofline("o", TRAFFIC_DECODE_O, "strip_kernel, o K=4096 N=4096, T cycling over {1,4,8,16}")

    # ---- per-shape decode table ----------------------------------------------------------------
    per_shape = []
    if not args.no_per_shape:
        for name, K, N, epi in LAYER_7B:
            for T in DECODE_T:
                us = per_launch_us(name, (T,))
                by = algorithmic_bytes(T, K, N, epi)
                per_shape.append({"shape": name, "T": T, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                                  "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 3)})
                if T in (1, 16):   # the engine clock inside the kernel and the life of one of its workgroups
                    per_shape[-1]["engine_clock"] = kernel_clock([(name, c, T) for c in range(len(weights[name]))])

    # ---- batched decode / short prompts: 32 .. 256 tokens (not part of `value`) ----------------
    batched = []
    if not args.no_per_shape:
        for name, K, N, epi in LAYER_7B:
            for T in BATCHED_T:
                us = per_launch_us(name, (T,), passes=2)
                batched.append({"shape": name, "T": T, "us": round(us, 2), "TFLOPs": round(flops(T, K, N) / us / 1e6, 1),
                                "GBps": round(algorithmic_bytes(T, K, N, epi) / us / 1e3, 1)})

    # ---- prefill: T = 2048 ---------------------------------------------------------------------
    prefill = None
    if not args.no_prefill:
        rows, tot_fl, tot_ms = [], 0.0, 0.0
        for name, K, N, epi in LAYER_7B:
            # four launches on four weight copies per graph: the gap between graph launches
            # (several microseconds) would otherwise count as kernel time
            r = make_runner([[(name, 4 * g + c, PREFILL_T) for c in range(4)] for g in range(2)])
            t_ms = timed(r, args.prefill_steps, 3, 5) / args.prefill_steps / 4
            fl = flops(PREFILL_T, K, N)
            rows.append({"shape": name, "ms": round(t_ms, 4), "TFLOPs": round(fl / t_ms / 1e9, 1),
                         "frac": round(fl / t_ms / 1e9 / MFMA_PEAK_TFLOPS, 4)})
            tot_fl += fl
            tot_ms += t_ms
        dom = max(rows, key=lambda x: x["ms"])
        prefill = {"T": PREFILL_T, "TFLOPs": round(tot_fl / tot_ms / 1e9, 1), "ms_per_layer": round(tot_ms, 4),
                   "per_shape": rows,
                   "roofline": {"bound": "mfma", "achieved": dom["TFLOPs"], "peak": MFMA_PEAK_TFLOPS,
                                "unit": "TFLOP/s", "frac": dom["frac"],
                                "traffic": TRAFFIC_PREFILL_GATE_UP if dom["shape"] == "gate_up" else None,
                                "kernel": "prefill_kernel, %s, T=2048" % dom["shape"]}}

        # The same kernel kept running for a few seconds, with the socket power and the engine clocks read beside
        # it: the 2.5 PFLOP/s peak is quoted at 2.4 GHz, and under a sustained matrix load the GPU sits at its
        # power limit and clocks lower.
        if not args.no_sustained:
            name = dom["shape"]
            r = make_runner([[(name, c, PREFILL_T) for c in range(4)]])
            reps = max(1, int(args.sustained_seconds * 1e3 / (dom["ms"] * 4)))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            sensors = {}
            # (a thread: enqueueing thousands of replays may block this one until most of them have run)
            reader = threading.Thread(target=lambda: (time.sleep(min(1.5, args.sustained_seconds / 3)),
                                                      sensors.update(read_power_and_clocks())))
            torch.cuda.synchronize()
            reader.start()
            e0.record(stream)
            with torch.cuda.stream(stream):
                for _ in range(reps):
                    r[0]()
            e1.record(stream)
            torch.cuda.synchronize()
            reader.join()
            fl = flops(PREFILL_T, *shape[name][:2])
            sensors.update(kernel="prefill_kernel, %s, T=2048" % name, seconds=round(e0.elapsed_time(e1) / 1e3, 2),
                           TFLOPs=round(4 * reps * fl / e0.elapsed_time(e1) / 1e9, 1))
            if sensors.get("mean_gfx_clk_MHz"):
                at_clock = MFMA_PEAK_TFLOPS * sensors["mean_gfx_clk_MHz"] / 2400.0
                sensors.update(mfma_peak_at_that_clock_TFLOPs=round(at_clock, 1),
                               frac_of_peak_at_that_clock=round(sensors["TFLOPs"] / at_clock, 4))
            prefill["under_sustained_load"] = sensors

    # ---- the full 32-layer GEMM sequence of one decode step at M = 8 (every layer its own weights) ----
    # as one launch per GEMM, and through w4a16_gemm_sequence as persistent launches (32 GEMMs each, every GEMM
    # behind a device-wide barrier as if it read its predecessor's output)
    seq_T = 8
    seq_bytes = N_LAYERS * sum(algorithmic_bytes(seq_T, K, N, epi) for _, K, N, epi in LAYER_7B)

    def layers32(ms_, launch_kind):
        return {"launch": launch_kind, "ms_per_decode_step": round(ms_, 4), "GBps": round(seq_bytes / ms_ / 1e6, 1),
                "frac": round(seq_bytes / ms_ / 1e6 / HBM_PEAK_GBS, 4)}

    seq_work = [[(name, layer, seq_T) for layer in range(N_LAYERS) for name, _, _, _ in LAYER_7B]]
    seq_ms = timed(make_runner(seq_work), 20, 5, 7) / 20

    def persistent(w, st):
        descs = []
        for i, (name, c, T) in enumerate(w):
            K, N, epi = shape[name]
            A, Q = weights[name][c % len(weights[name])]
            descs.append((out[name], A, X[K], Q, N, K, epi, Res if epi == 2 else None, i > 0))
        return gemm.sequence(descs, seq_T, persistent=True, stream=st)

    pers_ms = timed(make_runner(seq_work, persistent), 20, 5, 3) / 20
    gemm.sequence_status(stream.cuda_stream)
    layers32_m8 = dict(layers32(seq_ms, "one launch per GEMM (128 launches, one HIP graph)"), T=seq_T, layers=N_LAYERS,
                       gemms=4 * N_LAYERS,
                       weights_GB=round(N_LAYERS * sum(K * N // 2 + K // GROUP * N * 4 for _, K, N, _ in LAYER_7B) / 1e9, 2),
                       persistent=layers32(pers_ms, "w4a16_gemm_sequence, persistent: 4 launches of 32 dependent GEMMs"))

    # ---- what this machine reaches with plain kernels (context for the two peaks) ---------------
    # a streaming read launched like the decode kernels on 8 / 45 / 512 MiB (cold: rotating through >= 1.25 GiB),
    # a device copy (read + write), and hipBLASLt's fp16 GEMM on dense fp16 weights of the gate_up shape at
    # T = 2048 (what the reference's non-quantised LlamaLinear path would call)
    ceilings = None
    if not args.no_prefill:
        reads = {}
        # (workgroups per CU, 16-byte loads in flight per lane, hint: 1 = non-temporal) of w4a16_probe_stream; the
        # configurations that came out ahead in a full sweep (1, 2, 4 workgroups x 2, 4, 8, 16 loads x 3 hints)
        stream_configs = [(1, 4, 1), (1, 8, 1), (2, 2, 1), (1, 4, 0), (2, 8, 1), (2, 16, 1)]
        for mib in (8, 45, 244, 512):
            n = max(3, int(args.cold_gib * 1024 / mib) + 1)
            bufs = [torch.empty(mib << 20, dtype=torch.uint8, device="cuda") for _ in range(n)]
            for b in bufs:
                b.zero_()
            r = make_runner([bufs], lambda w, st: [gemm.probe_read(b, stream=st) for b in w])
            us = timed(r, 3, 1, 3) * 1e3 / (3 * n)
            row = {"us": round(us, 2), "GBps": round((mib << 20) / us / 1e3, 1),
                   "frac": round((mib << 20) / us / 1e3 / HBM_PEAK_GBS, 3)}
            swept = {}
            for wg, fl, hint in stream_configs:
                r = make_runner([bufs], lambda w, st: [gemm.probe_stream(b, wg, fl, hint, stream=st) for b in w])
                swept["wg%d_inflight%d_%s" % (wg, fl, "nt" if hint else "plain")] = round(timed(r, 3, 1, 3) * 1e3 / (3 * n), 2)
            best = min(swept, key=swept.get)
            row["counted_loads_us"] = swept
            row["best"] = {"config": best, "us": swept[best], "GBps": round((mib << 20) / swept[best] / 1e3, 1),
                           "frac": round((mib << 20) / swept[best] / 1e3 / HBM_PEAK_GBS, 3)}
            reads["read_%dMiB" % mib] = row
            del bufs, r
        with torch.cuda.stream(stream):
            src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
            dst = torch.empty_like(src)
            dst.copy_(src)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(10):
                dst.copy_(src)
            e1.record(stream)
            torch.cuda.synchronize()
            copy_gbs = 10 * 2 * src.numel() / e0.elapsed_time(e1) / 1e6
            del src, dst
            K, N = 4096, 22016
            Wd = [torch.randn((K, N), device="cuda", generator=gen).half() for _ in range(4)]
            Y = torch.empty((PREFILL_T, N), dtype=torch.float16, device="cuda")
            torch.matmul(X[K][:PREFILL_T], Wd[0], out=Y)
            torch.cuda.synchronize()
            e0.record(stream)
            for i in range(12):
                torch.matmul(X[K][:PREFILL_T], Wd[i % 4], out=Y)
            e1.record(stream)
            torch.cuda.synchronize()
            dense_tf = 12 * flops(PREFILL_T, K, N) / e0.elapsed_time(e1) / 1e9
            del Wd, Y
        barrier = {}
        with torch.cuda.stream(stream):
            for kind, tree in (("tree", True), ("single_counter", False)):
                gemm.probe_barrier(200, tree)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record(stream)
                gemm.probe_barrier(2000, tree)
                e1.record(stream)
                torch.cuda.synchronize()
                barrier[kind + "_us"] = round(e0.elapsed_time(e1) * 1e3 / 2000, 3)
        gemm.sequence_status(stream.cuda_stream)
        # the matrix pipes alone (w4a16_probe_mfma: nothing but MFMAs on registers) and the clock they run at
        mfma_loop = {}
        with torch.cuda.stream(stream):
            for waves in (8, 16):
                gemm.probe_mfma(waves, 2000)
                gemm.clock_begin(stream.cuda_stream)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record(stream)
                fl = sum(gemm.probe_mfma(waves, 40000) for _ in range(8))
                e1.record(stream)
                c = gemm.clock_end(stream.cuda_stream)
                tf = fl / e0.elapsed_time(e1) / 1e9
                mfma_loop["waves_per_cu_%d" % waves] = {"TFLOPs": round(tf, 1), "frac": round(tf / MFMA_PEAK_TFLOPS, 3),
                                                        "engine_clock_MHz": round(c["MHz"])}
        # what one more kernel costs in a chain: 200 launches of a read of 256 KiB (warm) in one graph
        tiny = torch.zeros(256 << 10, dtype=torch.uint8, device="cuda")
        r = make_runner([[tiny] * 200], lambda w, st: [gemm.probe_stream(b, 1, 2, 1, stream=st) for b in w])
        launch_floor_us = timed(r, 5, 1, 5) * 1e3 / (5 * 200)
        del tiny, r
        # the engine clock inside a streaming read and inside the decode kernel of gate_up
        bufs = [torch.zeros(45 << 20, dtype=torch.uint8, device="cuda") for _ in range(max(3, int(args.cold_gib * 1024 / 45) + 1))]
        clocks = {"read_45MiB_wg1_inflight4_nt": kernel_clock(bufs, lambda w, st: [gemm.probe_stream(b, 1, 4, 1, stream=st) for b in w])}
        del bufs
        for T in (1, 16):
            clocks["gate_up_T%d" % T] = kernel_clock([("gate_up", c, T) for c in range(len(weights["gate_up"]))])
        ceilings = dict(reads, device_wide_barrier=barrier, device_copy_512MiB_GBps=round(copy_gbs, 1),
                        mfma_loop=mfma_loop, engine_clock_in_kernel=clocks,
                        kernel_period_floor_in_graph_us=round(launch_floor_us, 2),
                        dense_fp16_gemm_gate_up_T2048_TFLOPs=round(dense_tf, 1),
                        note="read_*: w4a16_probe_read (plain streaming read, one launch per buffer in a HIP graph, cold buffers) and, "
                             "under counted_loads_us, w4a16_probe_stream (the GEMM kernels' load pipeline: wgN = workgroups of eight "
                             "waves per CU, inflightN = 16-byte loads per lane kept in flight, nt = non-temporal); "
                             "device_wide_barrier: w4a16_probe_barrier, one workgroup per CU, 2000 barriers in one launch; "
                             "torch copy_ (bytes read + written); torch.matmul fp16 (hipBLASLt); mfma_loop: w4a16_probe_mfma, "
                             "8 launches of 40000 x 4 MFMAs per wave; engine_clock_in_kernel (and llama70b rows): core-clock "
                             "cycles over constant-rate ticks between the first and last instruction of one wave per launch "
                             "(w4a16_probe_clock_begin / _end), kernel_us = those ticks per launch; kernel_period_floor_in_graph_us: "
                             "200 launches of a 256 KiB read in one graph, time per launch")

    # ---- Llama-2-70B layer shapes (BASELINE configs[3]) -----------------------------------------
    llama70b = None
    if not args.no_70b:
        rows70 = []
        X70 = {K: torch.randn((PREFILL_T, K), device="cuda", generator=gen).half() for K in (8192, 28672)}
        Res70 = torch.randn((PREFILL_T, 8192), device="cuda", generator=gen).half()
        copies_used = {}
        for name, K, N, epi in LAYER_70B:
            per_copy = K * N // 2 + (K // GROUP) * N * 4
            n = max(3, int(args.cold_gib * 2 ** 30 / per_copy) + 1)
            copies_used[name] = n
            ws = [make_weights(tm, torch, gen, name, K, N) for _ in range(n)]
            C = torch.empty((PREFILL_T, N // 2 if epi == 1 else N), dtype=torch.float16, device="cuda")

            def run70(w, st, K=K, N=N, epi=epi, C=C):
                for c, T in w:
                    gemm.Run(C, ws[c][0], X70[K], ws[c][1], N, T, K, GROUP, epi, -1, residual=Res70 if epi == 2 else None,
                             stream=st)
            for T in DECODE_T_70B:
                us = timed(make_runner([[(c, T) for c in range(n)]], run70), 3, 1, 5) * 1e3 / (3 * n)
                by = algorithmic_bytes(T, K, N, epi)
                rows70.append({"shape": name, "T": T, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                               "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 3),
                               "engine_clock": kernel_clock([(c, T) for c in range(n)], run70)})
            us = timed(make_runner([[(c, PREFILL_T) for c in range(n)]], run70), 2, 1, 3) * 1e3 / (2 * n)
            fl = flops(PREFILL_T, K, N)
            rows70.append({"shape": name, "T": PREFILL_T, "us": round(us, 1), "TFLOPs": round(fl / us / 1e6, 1),
                           "frac": round(fl / us / 1e6 / MFMA_PEAK_TFLOPS, 4)})
            del ws, C
            torch.cuda.empty_cache()
        llama70b = {"per_shape": rows70, "weight_copies_rotated": copies_used,
                    "note": "decode rows: frac of 8 TB/s; T=2048 rows: frac of 2.5 PFLOP/s; every launch reads a weight copy "
                            "that was last touched >= %.2f GiB of traffic ago" % args.cold_gib}

    # ---- CPU baselines: the oracle on the host cores ---------------------------------------------
    cpu = None
    cpu_prefill = None
    if not args.no_cpu:
        from oracle import w4a16_oracle as O
        T, reps = 8, 5
        t_deq = t_mm = t_mm1 = 0.0
        by = 0
        for i, (name, K, N, epi) in enumerate(LAYER_7B):
            d = O.make_inputs(77 + i, T, K, N, GROUP, residual=(epi == 2))
            deq, mm = [], []
            for _ in range(reps):   # median of five passes per GEMM, both halves timed separately
                t0 = time.perf_counter()
                W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], GROUP)
                t1 = time.perf_counter()
                O.epilogue(O.gemm_acc(d["X"], W), epi, d.get("R"))
                t2 = time.perf_counter()
                deq.append(t1 - t0)
                mm.append(t2 - t1)
            t_deq += sorted(deq)[reps // 2]
            t_mm += sorted(mm)[reps // 2]
            by += algorithmic_bytes(T, K, N, epi)
            nthreads = torch.get_num_threads()   # the same matmul once on a single thread, for scale
            torch.set_num_threads(1)
            t1 = time.perf_counter()
            O.epilogue(O.gemm_acc(d["X"], W), epi, d.get("R"))
            t_mm1 += time.perf_counter() - t1
            torch.set_num_threads(nthreads)
            if name == "o" and not args.no_prefill:
                # beside the T = 2048 figure: the same path on the o shape (68.7 GFLOP), dequantised weights reused
                dp = O.make_inputs(99, PREFILL_T, K, N, GROUP)
                tp = []
                for _ in range(3):
                    t1 = time.perf_counter()
                    O.epilogue(O.gemm_acc(dp["X"], W), epi)
                    tp.append(time.perf_counter() - t1)
                tpm = sorted(tp)[1]
                cpu_prefill = {"value": round(flops(PREFILL_T, K, N) / tpm / 1e12, 4), "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "o shape (K=4096, N=4096) at T=2048, torch fp32 matmul + epilogue on already dequantised "
                                         "weights, median of 3: %.3f s; unpack+dequantise of the matrix adds %.2f s (numpy, 1 thread)"
                                         % (tpm, sorted(deq)[reps // 2])}
        cpu = {"value": round(by / (t_deq + t_mm) / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(),
               "sample": "one Llama-2-7B layer (qkv, o, gate_up+SiLU, down+residual) at T=8, median of %d passes per "
                         "GEMM: numpy unpack+dequantise %.2f s (1 thread) + torch fp32 matmul+epilogue %.3f s "
                         "(%d threads; %.3f s on 1 thread)" % (reps, t_deq, t_mm, torch.get_num_threads(), t_mm1),
               "prefill": cpu_prefill}

    line = {
        "metric": "W4A16 GEMM achieved HBM GB/s (M=1..16) + TFLOP/s (M=2048), % of roofline",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "timing": timing, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Llama-2-7B decode layer set (qkv 4096x12288, o 4096x4096, gate_up 4096x22016 +SiLU, "
                               "down 11008x4096 +residual) at T in {1,4,8,16}, group 128: 16 GEMMs per step, each on its own "
                               "weight copy, %d rotating sets of 16" % n_sets,
                   "launch": "eager" if args.eager else "hipgraph replays, %d steps (%d launches) per graph" % (S, 16 * S),
                   "bytes_per_step": step_bytes},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": roofline, "roofline_worst_decode_kernel": roofline_worst, "cpu_baseline": cpu,
        "decode_per_shape": per_shape, "batched_decode_per_shape": batched,
        "prefill": prefill, "llama70b": llama70b,
        "layers32_m8": layers32_m8, "library_ceilings": ceilings,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
