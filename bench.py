#!/usr/bin/env python3
"""Benchmark of the INT4 AWQ dequantise+GEMV hot path on one MI355X.

A "step" is one pass over the seven Qwen3-8B decoder projections at M = 1 (q, k, v, o, gate, up,
down; group 128, fp16 scales, int4 zero points, bf16 activations), each a separate launch of the
fused kernel through the C ABI.  Weights are cold: consecutive steps walk through WEIGHT_SETS
distinct copies of every tensor (> 1 GiB in total, more than L2 + Infinity Cache hold), so no
launch finds its weights in a cache.  All inputs are resident in HBM before the timed region.

Prints one JSON line:  value = algorithmic bytes of a step / time of a step, in GB/s.
  roofline      dominant kernel (the fused AWQ GEMV): algorithmic bytes per launch over the average
                launch duration seen by HIP events on the launch stream (back-to-back launches, so
                the figure includes the dispatch gap between kernels), against 8 TB/s
  cpu_baseline  the oracle's single-threaded fp32 restatement, timed on this host on a bounded
                number of passes over the same seven shapes
  per_shape     each projection shape on its own, cold weights, same event timing: median / p10 / p90 of the
                per-launch time over 20 graph replays of 60 launches, and beside it the streaming floor of the
                same tensors (a kernel that only reads them, mykuiperllama_amd/probe/kx_stream_probe.hip, same
                rotation, same replay) with the GEMV's distance to it
  validated     after the timed region the outputs the last timed step left behind are compared with the CPU
                oracle (fp64 evaluation rounded to bf16) on the same weight set: relative L2 per shape
  kernel_variants  five shapes at M = 1 under the two forced kernel policies (1 = vector-ALU kernel, 2 = one-shot
                MFMA kernel, both with the K tiles meeting through partial sums in memory), microseconds per launch;
                per_shape holds the product's own launch (vector kernel, K tiles meeting in 64-bit fixed point)
  small_batch   configs[2]: M in {1, 2, 4, 8, 16} on three shapes, microseconds per launch of the
                vector-ALU kernel and of the MFMA kernel (cold weights, same event timing)
  decode        configs[3] and configs[4]: tokens/s of a full decode step (Qwen3-8B, Qwen3-32B-shaped); under the
                8B entry, small_batch_decode: 2, 8 and 16 sequences decoded together (--decode-batches), each at
                the same position of its own KV cache, tokens/s summed over the sequences, with the GEMVs'
                prologues and epilogues (seven launches per layer) and from stand-alone operators
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
WEIGHT_SETS = 12           # x 100.4 MB per set = 1.2 GB of cold weights
ORDER = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
METRIC = "INT4 AWQ GEMV achieved HBM GB/s (% of 8 TB/s); Qwen3-8B decode tok/s"
# HBM bytes per launch of the dominant kernel (average over the seven launches of a step) from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --probe`, each counter scaled by what it
# reads for a 256 MiB copy (profiles/awq_gemv_qwen3_8b_projections_hbm_counters.md).  Counters cannot be
# read from inside this process, so the figure is carried over from that profile and named as such.
TRAFFIC_BYTES_PER_LAUNCH = 15349775
TRAFFIC_SOURCE = "profiles/awq_gemv_qwen3_8b_projections_hbm_counters.md"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=600)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--eager", action="store_true", help="launch from the host loop instead of a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-passes", type=int, default=150)
    ap.add_argument("--no-per-shape", action="store_true")
    ap.add_argument("--no-small-batch", action="store_true", help="skip the M = 1..16 vector/MFMA kernel table")
    ap.add_argument("--no-decode", action="store_true", help="skip the Qwen3-8B decode-step measurement")
    ap.add_argument("--no-decode-32b", action="store_true", help="skip the Qwen3-32B-shaped decode step")
    ap.add_argument("--decode-32b", action="store_true", help="kept for older command lines: the step runs by default")
    ap.add_argument("--decode-steps", type=int, default=60)
    ap.add_argument("--decode-batches", default="2,8,16",
                    help="numbers of sequences decoded together in the small_batch_decode leg (Qwen3-8B); '' skips it")
    ap.add_argument("--lib", default=None,
                    help="time another build of the HIP library (e.g. lib/libkx_hip_ablate1.so from "
                         "`python -m mykuiperllama_amd.build --ablate 1`); its numbers attribute time, its results "
                         "are wrong by construction, so validation and the small-batch table are skipped")
    ap.add_argument("--probe", action="store_true",
                    help="counter-collection workload: one 256 MiB device copy (known traffic, for scaling the "
                         "counters) followed by a few cold launches per projection shape; prints no metric")
    return ap.parse_args()


class WeightSet:
    """One cold copy of the seven projections' packed tensors, generated on the device."""

    def __init__(self, torch, shapes, group, gen):
        self.t = {}
        for name, (K, N) in shapes.items():
            qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
            qz = torch.randint(-2**31, 2**31 - 1, (K // group, N // 8), dtype=torch.int32, device="cuda", generator=gen)
            sc = (torch.rand((K // group, N), device="cuda", generator=gen) * 0.019 + 0.001).half()
            self.t[name] = (qw, sc, qz)


def timed_region(torch, launch_steps, steps, warmup, eager, steps_per_graph):
    """Run `warmup` untimed steps, then exactly `steps` timed ones; returns seconds (events)."""
    torch.cuda.synchronize()  # tensors were initialised on the default stream; the launches below use another
    stream = torch.cuda.current_stream()
    if eager:
        launch_steps(0, warmup)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        launch_steps(warmup, steps)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    def capture(first, count):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            launch_steps(first, count)
        return g

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        launch_steps(0, min(warmup, 4))  # load the code objects outside capture
        side.synchronize()
        full = capture(0, steps_per_graph)
        rem = steps % steps_per_graph
        tail = capture(0, rem) if rem else None
        for _ in range(max(1, warmup // steps_per_graph)):
            full.replay()
        side.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(side)
        for _ in range(steps // steps_per_graph):
            full.replay()
        if tail is not None:
            tail.replay()
        e1.record(side)
        side.synchronize()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3


def replay_times(torch, launch_steps, steps_per_graph, replays):
    """Per-launch-step microseconds of each of `replays` replays of one captured graph of `steps_per_graph` steps."""
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        launch_steps(0, min(steps_per_graph, 4))
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            launch_steps(0, steps_per_graph)
        g.replay()
        side.synchronize()
        events = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
        events[0].record(side)
        for i in range(replays):
            g.replay()
            events[i + 1].record(side)
        side.synchronize()
    torch.cuda.synchronize()
    return [events[i].elapsed_time(events[i + 1]) * 1e3 / steps_per_graph for i in range(replays)]


def spread(us):
    """median / p10 / p90 of a list of per-launch microseconds."""
    v = sorted(us)

    def q(f):
        return v[min(len(v) - 1, max(0, int(round(f * (len(v) - 1)))))]
    return {"us": round(q(0.5), 3), "p10_us": round(q(0.1), 3), "p90_us": round(q(0.9), 3)}


def shape_report(torch, capi, synth, K, N, group, tensor_sets, x, y, ws):
    """One projection shape on its own: the GEMV and the streaming floor over the same cold tensors."""
    nsets = len(tensor_sets)
    b = synth.awq_gemv_bytes(1, K, N)

    def launch_gemv(first, count):
        for s in range(first, first + count):
            qw, sc, qz = tensor_sets[s % nsets]
            capi.gemv_awq_bf16(x, qw, sc, qz, y, group, ws)

    def launch_floor(first, count):
        for s in range(first, first + count):
            capi.probe_stream_read(tensor_sets[s % nsets])

    rep = spread(replay_times(torch, launch_gemv, 5 * nsets, 20))
    floor = spread(replay_times(torch, launch_floor, 5 * nsets, 20))
    rep.update({"GB/s": round(b / rep["us"] / 1e3, 1), "pct_of_8TBps": round(b / rep["us"] / 1e3 / HBM_PEAK_GBPS * 100, 2),
                "bytes": b, "stream_floor_us": floor["us"], "stream_floor_pct_of_8TBps":
                round(b / floor["us"] / 1e3 / HBM_PEAK_GBPS * 100, 2),
                "frac_of_floor": round(floor["us"] / rep["us"], 3)})
    return rep


def validate_outputs(torch, sets, last_set, xs, ys, shapes, group):
    """The outputs the last timed step left in `ys` against the CPU oracle on the same weight set."""
    import numpy as np
    from oracle import oracle
    out = {}
    worst = 0.0
    for n in ORDER:
        K, N = shapes[n]
        qw, sc, qz = sets[last_set].t[n]
        xb = xs[K].cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
        ref64 = oracle.gemv_awq_f64(xb, qw.cpu().numpy(), sc.cpu().contiguous().view(torch.int16).numpy().view(np.uint16),
                                    qz.cpu().numpy(), group)
        ref = oracle.bf16_to_f32(oracle.f32_to_bf16(ref64.astype(np.float32))).astype(np.float64)
        got = ys[n].float().cpu().numpy().astype(np.float64)
        err = float(np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()))
        out[n] = float(f"{err:.3e}")
        worst = max(worst, err)
    return {"validated": bool(worst <= 1e-3), "tolerance_rel_l2": 1e-3, "weight_set": last_set, "rel_l2": out,
            "checker": "oracle/kx_oracle.c kxo_gemv_awq_f64 rounded to bf16, outside the timed region"}


def cpu_baseline(passes):
    """Single-threaded oracle (fp32 evaluation of w = (q - z) * s) over the seven shapes."""
    import numpy as np
    from mykuiperllama_amd import synth
    from oracle import oracle
    probs = [synth.make_awq_problem(f"bench_cpu_{n}", 1, *synth.QWEN3_8B[n]) for n in ORDER]
    step_bytes = sum(synth.awq_gemv_bytes(1, p["K"], p["N"]) for p in probs)
    for p in probs[:1]:
        oracle.gemv_awq_f32(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"])
    t0 = time.perf_counter()
    for _ in range(passes):
        for p in probs:
            oracle.gemv_awq_f32(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"])
    dt = time.perf_counter() - t0
    del np
    out = {"value": round(step_bytes * passes / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
           "ms_per_step": round(dt / passes * 1e3, 2),
           "sample": f"{passes} passes over the seven Qwen3-8B projections at M=1 (seeded inputs), "
                     f"oracle/kx_oracle.c kxo_gemv_awq_f32, gcc -O3 -march=x86-64-v3 (the library is built "
                     f"where there is no GPU and travels to this host, so it cannot be tuned to this host's CPU "
                     f"with -march=native), one thread, host has {os.cpu_count()} logical cpus"}
    # the same arithmetic spread over the host's cores (columns split across threads), as a second figure
    threads = min(os.cpu_count() or 1, 16)
    if threads > 1:
        mt_passes = max(10, passes // 3)
        t0 = time.perf_counter()
        for _ in range(mt_passes):
            for p in probs:
                oracle.gemv_awq_f32_threads(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"], threads)
        dt = time.perf_counter() - t0
        out["all_cores"] = {"value": round(step_bytes * mt_passes / dt / 1e9, 4), "unit": "GB/s", "cores": threads,
                            "ms_per_step": round(dt / mt_passes * 1e3, 2),
                            "sample": f"{mt_passes} passes, kxo_gemv_awq_f32_range over {threads} threads"}
    # configs[0]: the single Qwen3-0.6B q_proj GEMV (M=1, K=1024, N=2048), the case the CPU path is quoted on
    K0, N0 = synth.QWEN3_0P6B["q_proj"]
    p0 = synth.make_awq_problem("bench_cpu_config0", 1, K0, N0)
    b0 = synth.awq_gemv_bytes(1, K0, N0)
    n0 = max(200, passes * 10)
    oracle.gemv_awq_f32(p0["x"], p0["qweight"], p0["scales"], p0["qzeros"], p0["group"])
    t0 = time.perf_counter()
    for _ in range(n0):
        oracle.gemv_awq_f32(p0["x"], p0["qweight"], p0["scales"], p0["qzeros"], p0["group"])
    dt = time.perf_counter() - t0
    cfg0 = {"workload": "configs[0]: Qwen3-0.6B q_proj 1024->2048, M=1", "bytes": b0, "cores": 1,
            "us_per_gemv": round(dt / n0 * 1e6, 1), "GB/s": round(b0 * n0 / dt / 1e9, 4), "calls": n0}
    if threads > 1:
        t0 = time.perf_counter()
        for _ in range(n0):
            oracle.gemv_awq_f32_threads(p0["x"], p0["qweight"], p0["scales"], p0["qzeros"], p0["group"], threads)
        dt = time.perf_counter() - t0
        cfg0["all_cores"] = {"cores": threads, "us_per_gemv": round(dt / n0 * 1e6, 1),
                             "GB/s": round(b0 * n0 / dt / 1e9, 4)}
    out["config0"] = cfg0
    return out


def decode_benchmark(torch, cfg_name, ctx, steps, warmup, eager, batches=()):
    """Tokens/s of a full random-init decode step (batch 1, KV cache pre-filled at `ctx`)."""
    from mykuiperllama_amd import decode
    cfg = {"qwen3-8b": decode.QWEN3_8B, "qwen3-32b": decode.QWEN3_32B}[cfg_name]
    model = decode.DecodeModel(cfg, max_positions=ctx + 128)
    model.prefill_cache_random(ctx)
    model.set_input(1, ctx)  # every timed step decodes position `ctx` against ctx cached positions
    out = {"model": cfg_name, "context": ctx, "steps": steps, "launch": "eager" if eager else "hipGraph replay",
           "weights": "random-init INT4 AWQ group 128 (q/k/v and gate/up fused along N), bf16 embedding and lm_head",
           "fusion": "add+RMSNorm and SwiGLU in the prologue of the consuming GEMV, QK-norm+RoPE+KV append in the epilogue of the q/k/v GEMV"}
    for with_head in (True, False):
        def launch(first, count, with_head=with_head):
            for _ in range(count):
                model.step(with_lm_head=with_head)
        sec = timed_region(torch, launch, steps, warmup, eager, 4)
        key = "with_lm_head" if with_head else "without_lm_head"
        nbytes = decode.step_bytes(cfg, ctx, with_head)
        out[key] = {"tokens_per_s": round(steps / sec, 1), "ms_per_token": round(sec / steps * 1e3, 4),
                    "algorithmic_GB_per_token": round(nbytes / 1e9, 3),
                    "GB/s": round(nbytes / (sec / steps) / 1e9, 1),
                    "pct_of_8TBps": round(nbytes / (sec / steps) / 1e9 / HBM_PEAK_GBPS * 100, 2),
                    "launches_per_token": model.launches_per_step(with_head)}
    torch.cuda.synchronize()
    out["next_token_finite"] = bool(torch.isfinite(model.logits.float()).all().item())
    if batches:
        # several sequences decoded together, every one of them at position `ctx` of its own cache: the GEMVs
        # read the weights once for all rows, the attention reads one cache per sequence
        rows = {}
        for B in batches:
            bm = decode.BatchDecodeModel(model, B)
            bm.prefill_cache_random(ctx)
            bm.set_input([1 + b for b in range(B)], [ctx] * B)
            cell = {}
            for label, fused in (("fused", True), ("unfused", False)):
                def launch(first, count, fused=fused):
                    for _ in range(count):
                        bm.step(fused=fused)
                n = max(8, steps // 3)
                sec = timed_region(torch, launch, n, 4, eager, 4)
                cell[label] = {"ms_per_step": round(sec / n * 1e3, 4), "tokens_per_s": round(B * n / sec, 1),
                               "launches_per_step": bm.launches_per_step(True, fused)}
            torch.cuda.synchronize()
            cell["finite"] = bool(torch.isfinite(bm.logits.float()).all().item())
            rows[f"B={B}"] = cell
            del bm
            torch.cuda.empty_cache()
        out["small_batch_decode"] = rows
    del model
    torch.cuda.empty_cache()
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no multi-GPU part in this build "
              "(run with --gpus 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    from mykuiperllama_amd import capi, synth
    capi.load(args.lib)  # raises if the HIP library is missing: there is no fallback path
    profiling_build = args.lib is not None
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    shapes = synth.QWEN3_8B
    group = synth.GROUP
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.BASE_SEED)

    sets = [WeightSet(torch, shapes, group, gen) for _ in range(WEIGHT_SETS)]
    xs = {K: torch.randn((1, K), device="cuda", generator=gen).bfloat16() for K in {k for k, _ in shapes.values()}}
    ys = {n: torch.empty((1, shapes[n][1]), dtype=torch.bfloat16, device="cuda") for n in ORDER}
    ws = capi.make_workspace(1, max(k for k, _ in shapes.values()), max(n for _, n in shapes.values()))
    step_bytes = sum(synth.awq_gemv_bytes(1, *shapes[n]) for n in ORDER)

    def launch_steps(first, count):
        for s in range(first, first + count):
            wset = sets[s % WEIGHT_SETS]
            for n in ORDER:
                qw, sc, qz = wset.t[n]
                capi.gemv_awq_bf16(xs[shapes[n][0]], qw, sc, qz, ys[n], group, ws)

    if args.probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        launch_steps(0, WEIGHT_SETS)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "copy 268435456 B, then %d steps of 7 launches" % WEIGHT_SETS}))
        return

    seconds = timed_region(torch, launch_steps, args.steps, args.warmup, args.eager, WEIGHT_SETS)
    # which weight set the last timed step walked over (its outputs are what ys holds now)
    if args.eager:
        last_set = (args.warmup + args.steps - 1) % WEIGHT_SETS
    else:
        rem = args.steps % WEIGHT_SETS
        last_set = (rem - 1) if rem else (WEIGHT_SETS - 1)
    validation = None if profiling_build else validate_outputs(torch, sets, last_set, xs, ys, shapes, group)
    ms_per_step = seconds / args.steps * 1e3
    value = step_bytes / (seconds / args.steps) / 1e9
    launches = args.steps * len(ORDER)
    avg_launch_us = seconds / launches * 1e6
    bytes_per_launch = step_bytes / len(ORDER)
    achieved = bytes_per_launch / (avg_launch_us * 1e-6) / 1e9

    per_shape = None
    if not args.no_per_shape:
        per_shape = {"protocol": "each shape alone, cold weights (12 rotating sets), 20 replays of a 60-launch HIP graph, "
                                 "events on the launch stream; us = median per-launch time over the replays; "
                                 "stream_floor_us = the same for a kernel that only reads the shape's three packed "
                                 "tensors (mykuiperllama_amd/probe/kx_stream_probe.hip)"}
        # what a launch costs before it has done anything: workgroups of 512 threads that return at once
        def launch_empty(blocks):
            def body(first, count):
                for _ in range(count):
                    capi.probe_empty_launch(blocks)
            return body
        per_shape["empty_launch_us"] = {str(b): spread(replay_times(torch, launch_empty(b), 60, 20))["us"]
                                        for b in (64, 256, 768, 2000)}
        for n in ["k_proj", "q_proj", "gate_proj", "down_proj"]:
            K, N = shapes[n]
            per_shape[f"{n} {K}x{N}"] = shape_report(torch, capi, synth, K, N, group, [st.t[n] for st in sets],
                                                     xs[K], ys[n], ws)

        # The launches a decode step fuses along N, and the launches of the Qwen3-32B-shaped step: same
        # cold-weight protocol, one shape at a time (the largest is 131 MB per copy).
        more_shapes = {"qkv fused": (4096, 6144), "gate+up fused": (4096, 24576),
                       "32B qkv fused": (5120, 10240), "32B o_proj": (8192, 5120),
                       "32B gate+up fused": (5120, 51200), "32B down_proj": (25600, 5120)}
        for n, (K, N) in more_shapes.items():
            fsets = [WeightSet(torch, {n: (K, N)}, group, gen).t[n] for _ in range(WEIGHT_SETS)]
            xf = xs[K] if K in xs else torch.randn((1, K), device="cuda", generator=gen).bfloat16()
            yf = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
            wsf = capi.make_workspace(1, K, N)
            per_shape[f"{n} {K}x{N}"] = shape_report(torch, capi, synth, K, N, group, fsets, xf, yf, wsf)
            del fsets
            torch.cuda.empty_cache()

    kernel_variants = None
    if not args.no_per_shape:
        kernel_variants = {"unit": "us per launch, M = 1, cold weights, median of 10 replays of a 60-launch graph",
                           "kernels": {"vector": "policy 1", "mfma": "policy 2 (one-shot MFMA)"}}
        for label, (K, N) in {"q_proj": (4096, 4096), "gate_proj": (4096, 12288), "gate+up fused": (4096, 24576),
                              "32B down_proj": (25600, 5120), "32B gate+up fused": (5120, 51200)}.items():
            vsets = [WeightSet(torch, {label: (K, N)}, group, gen).t[label] for _ in range(WEIGHT_SETS)]
            xv = xs[K] if K in xs else torch.randn((1, K), device="cuda", generator=gen).bfloat16()
            yv = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
            wsv = capi.make_workspace(1, K, N)
            row = {}
            for name, policy in (("vector", 1), ("mfma", 2)):
                capi.set_awq_kernel_policy(policy)

                def launch_v(first, count, vsets=vsets, xv=xv, yv=yv, wsv=wsv):
                    for s_ in range(first, first + count):
                        qw, sc, qz = vsets[s_ % WEIGHT_SETS]
                        capi.gemv_awq_bf16(xv, qw, sc, qz, yv, group, wsv)

                row[name] = spread(replay_times(torch, launch_v, 5 * WEIGHT_SETS, 10))["us"]
            capi.set_awq_kernel_policy(0)
            kernel_variants[f"{label} {K}x{N}"] = row
            del vsets
            torch.cuda.empty_cache()

    small_batch = None
    if not args.no_small_batch and not profiling_build:
        small_batch = {"unit": "us per launch", "kernels": {"vector": "VALU kernel, bf16 dot2", "mfma": "16x16x32 bf16 MFMA"}}
        for n in ["q_proj", "gate_proj", "down_proj"]:
            K, N = shapes[n]
            row = {}
            for M in (1, 2, 4, 8, 16):
                xm = torch.randn((M, K), device="cuda", generator=gen).bfloat16()
                ym = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
                wsm = capi.make_workspace(M, K, N)
                cell = {}
                for label, policy in (("vector", 1), ("mfma", 2)):
                    capi.set_awq_kernel_policy(policy)

                    def launch_m(first, count, n=n, xm=xm, ym=ym, wsm=wsm):
                        for s in range(first, first + count):
                            qw, sc, qz = sets[s % WEIGHT_SETS].t[n]
                            capi.gemv_awq_bf16(xm, qw, sc, qz, ym, group, wsm)

                    reps = 10 * WEIGHT_SETS
                    sec = timed_region(torch, launch_m, reps, WEIGHT_SETS, args.eager, WEIGHT_SETS)
                    cell[label] = round(sec / reps * 1e6, 2)
                capi.set_awq_kernel_policy(0)
                cell["GB/s_best"] = round(synth.awq_gemv_bytes(M, K, N) / min(cell["vector"], cell["mfma"]) / 1e3, 1)
                row[f"M={M}"] = cell
            small_batch[f"{n} {K}x{N}"] = row

    out = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int4 weights x bf16 activations, fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": "configs[1]: the seven Qwen3-8B decoder projections at M=1, INT4 AWQ group 128, "
                               f"cold weights ({WEIGHT_SETS} rotating sets, {WEIGHT_SETS * step_bytes / 1e9:.2f} GB)",
                   "launch": "eager" if args.eager else "hipGraph replay",
                   "bytes_per_step": step_bytes, "launches_per_step": len(ORDER),
                   "weights": f"torch.randint / torch.rand on the device, torch.Generator(cuda) seeded {synth.BASE_SEED} "
                              "(uniform int4 codes and zero points, fp16 scales U(0.001, 0.02)), activations "
                              "bf16 N(0,1) from the same generator",
                   "library": args.lib or "mykuiperllama_amd/lib/libkx_hip.so"},
        "pct_of_8TBps": round(value / HBM_PEAK_GBPS * 100, 2),
        "decode_tok_s": None,
        "roofline": {"bound": "hbm", "kernel": "kx::awq_gemv_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": TRAFFIC_BYTES_PER_LAUNCH, "traffic_source": TRAFFIC_SOURCE,
                     "bytes_per_launch": round(bytes_per_launch),
                     "avg_launch_us": round(avg_launch_us, 3)},
    }
    if validation is not None:
        out["validated"] = validation["validated"]
        out["validation"] = validation
    if per_shape is not None:
        out["per_shape"] = per_shape
    if kernel_variants is not None:
        out["kernel_variants"] = kernel_variants
    if small_batch is not None:
        out["small_batch"] = small_batch
    if not args.no_decode:  # also with --lib: the builds that cut the first attention stage short are timed here
        del sets
        torch.cuda.empty_cache()
        d8 = decode_benchmark(torch, "qwen3-8b", 4096, args.decode_steps, 8, args.eager,
                              batches=tuple(int(b) for b in args.decode_batches.split(",") if b.strip()))
        out["decode_tok_s"] = d8["with_lm_head"]["tokens_per_s"]
        out["decode"] = {"qwen3-8b ctx4096": d8}
        if not args.no_decode_32b:
            out["decode"]["qwen3-32b ctx8192"] = decode_benchmark(torch, "qwen3-32b", 8192, args.decode_steps, 8,
                                                                  args.eager)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_passes)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
