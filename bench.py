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
  per_shape     each projection shape on its own, cold weights, same event timing
  small_batch   configs[2]: M in {1, 2, 4, 8, 16} on three shapes, microseconds per launch of the
                vector-ALU kernel and of the MFMA kernel (cold weights, same event timing)
  decode        configs[3] and configs[4]: tokens/s of a full decode step (Qwen3-8B, Qwen3-32B-shaped)
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
# reads for a 256 MiB copy (profiles/awq_gemv_qwen3_8b_projections_hbm_counters.md).
TRAFFIC_BYTES_PER_LAUNCH = 15288300


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
                     f"oracle/kx_oracle.c kxo_gemv_awq_f32, gcc -O3 -march=x86-64-v3, one thread, "
                     f"host has {os.cpu_count()} logical cpus"}
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
    return out


def decode_benchmark(torch, cfg_name, ctx, steps, warmup, eager):
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
    capi.load()  # raises if the HIP library is missing: there is no fallback path
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
    ms_per_step = seconds / args.steps * 1e3
    value = step_bytes / (seconds / args.steps) / 1e9
    launches = args.steps * len(ORDER)
    avg_launch_us = seconds / launches * 1e6
    bytes_per_launch = step_bytes / len(ORDER)
    achieved = bytes_per_launch / (avg_launch_us * 1e-6) / 1e9

    per_shape = None
    if not args.no_per_shape:
        per_shape = {}
        for n in ["k_proj", "q_proj", "gate_proj", "down_proj"]:
            K, N = shapes[n]
            b = synth.awq_gemv_bytes(1, K, N)
            reps = max(WEIGHT_SETS, 240 // WEIGHT_SETS * WEIGHT_SETS)

            def launch_one(first, count, n=n):
                for s in range(first, first + count):
                    qw, sc, qz = sets[s % WEIGHT_SETS].t[n]
                    capi.gemv_awq_bf16(xs[shapes[n][0]], qw, sc, qz, ys[n], group, ws)

            sec = timed_region(torch, launch_one, reps, WEIGHT_SETS, args.eager, WEIGHT_SETS)
            us = sec / reps * 1e6
            per_shape[f"{n} {K}x{N}"] = {"us": round(us, 3), "GB/s": round(b / us / 1e3, 1),
                                         "pct_of_8TBps": round(b / us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                                         "bytes": b}

        # The launches a decode step fuses along N, and the launches of the Qwen3-32B-shaped step: same
        # cold-weight protocol, one shape at a time (the largest is 131 MB per copy).
        more_shapes = {"qkv fused": (4096, 6144), "gate+up fused": (4096, 24576),
                       "32B qkv fused": (5120, 10240), "32B o_proj": (8192, 5120),
                       "32B gate+up fused": (5120, 51200), "32B down_proj": (25600, 5120)}
        for n, (K, N) in more_shapes.items():
            fsets = [WeightSet(torch, {n: (K, N)}, group, gen) for _ in range(WEIGHT_SETS)]
            b = synth.awq_gemv_bytes(1, K, N)
            xf = xs[K] if K in xs else torch.randn((1, K), device="cuda", generator=gen).bfloat16()
            yf = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
            wsf = capi.make_workspace(1, K, N)
            reps = 240 // WEIGHT_SETS * WEIGHT_SETS

            def launch_f(first, count, n=n, xf=xf, yf=yf, wsf=wsf, fsets=fsets):
                for s in range(first, first + count):
                    qw, sc, qz = fsets[s % WEIGHT_SETS].t[n]
                    capi.gemv_awq_bf16(xf, qw, sc, qz, yf, group, wsf)

            sec = timed_region(torch, launch_f, reps, WEIGHT_SETS, args.eager, WEIGHT_SETS)
            us = sec / reps * 1e6
            per_shape[f"{n} {K}x{N}"] = {"us": round(us, 3), "GB/s": round(b / us / 1e3, 1),
                                         "pct_of_8TBps": round(b / us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                                         "bytes": b}
            del fsets, launch_f
            torch.cuda.empty_cache()

    small_batch = None
    if not args.no_small_batch:
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
                   "bytes_per_step": step_bytes, "launches_per_step": len(ORDER)},
        "pct_of_8TBps": round(value / HBM_PEAK_GBPS * 100, 2),
        "decode_tok_s": None,
        "roofline": {"bound": "hbm", "kernel": "kx::awq_gemv_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": TRAFFIC_BYTES_PER_LAUNCH, "bytes_per_launch": round(bytes_per_launch),
                     "avg_launch_us": round(avg_launch_us, 3)},
    }
    if per_shape is not None:
        out["per_shape"] = per_shape
    if small_batch is not None:
        out["small_batch"] = small_batch
    if not args.no_decode:
        del sets
        torch.cuda.empty_cache()
        d8 = decode_benchmark(torch, "qwen3-8b", 4096, args.decode_steps, 8, args.eager)
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
