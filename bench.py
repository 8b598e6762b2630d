#!/usr/bin/env python3
"""Benchmark of the fused W8A8 MoE operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--M 64] [--shape ds]

A "step" is one call of torch.ops.alpha_moe.fused_moe_w8a8_up_down on a DeepSeek-V3-like single-GPU TP shard
(E=257 incl. the fused shared expert, top_k=9, K=7168, I=256, FP8 e4m3 with 128x128 block scales) with all inputs
resident in HBM.  The headline is M=64 decode against the HBM roofline; the same run also measures the other batch
sizes of that shard (decode M = 1, 4, 16 and prefill M = 512, 2048, 8192, reported under "per_M" with both the HBM and
the FP8 MFMA fraction) and the Qwen3-Next-like and Qwen3-30B-like shards ("other_configs").
Consecutive steps rotate through several copies of the weights and several routings so that a step never finds its
weights in the 256 MiB Infinity Cache; where that rotation touches less than 1 GiB (small M), every timed call is
preceded by a 512 MiB fill that evicts L2 and the Infinity Cache, and the figure is the mean of the per-call device
times ("cold": true).  `out` is not re-zeroed inside the timed region (the operator adds into it).
Every reported size is also checked against the CPU oracle on a sample of its tokens ("parity_sample").

Prints ONE JSON line: the driver's contract fields plus
  "roofline":     algorithmic HBM bytes per launch / average launch duration (HIP events on the launch stream)
  "cpu_baseline": the CPU oracle (oracle/moe_oracle.py, a port of the reference maths) timed on the host cores
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "alpha-moe_amd"))
sys.path.insert(0, ROOT)

# HBM bytes per call from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy of known size; all kernels of a
# call) live in profiles/traffic.json together with the library version they were measured on: a build of another
# version reports null instead of a stale figure.
def load_measured_traffic(library_version):
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        return {}
    if doc.get("library_version") != library_version:
        return {}
    return {tuple(k.split("/")[:1]) + (int(k.split("/")[1]),): float(v) for k, v in doc.get("bytes_per_call", {}).items()}


HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP8_PEAK_TFLOPS = 5000.0     # MI355X dense FP8 MFMA, published
DEFAULT_KNOBS = {"block_m": 16, "block_n": 32, "warp_n": 8, "stages": 5}
# batch sizes of the other benchmark configurations
DS_OTHER_M = (1, 4, 16, 64, 512, 2048, 8192)
OTHER_CONFIGS = {"qn": (1, 32, 256, 4096), "q3": (64, 1024, 8192)}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--shape", default="ds", choices=["ds", "qn", "q3", "c1"])
    ap.add_argument("--M", type=int, default=64, help="tokens of the headline measurement")
    ap.add_argument("--also-M", type=int, nargs="*", default=None, help="other token counts reported under per_M")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the Qwen3-Next / Qwen3-30B shards")
    ap.add_argument("--replicas", type=int, default=6, help="copies of the weights rotated through")
    ap.add_argument("--config", default=None, help="tuning table (JSON of jit_moe.py); default: shipped table or built-in knobs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity-samples", action="store_true", help="skip the oracle check of every reported size")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy three times: a kernel of known traffic to scale "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings by")
    return ap.parse_args()


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this operator is a single-GPU kernel on one tensor-parallel shard and has no "
              f"multi-GPU path (asked for --gpus {args.gpus}).", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    import alpha_moe  # fails loudly if the HIP libraries are not built
    MEASURED_TRAFFIC_BYTES = load_measured_traffic(alpha_moe.__version__)
    from alpha_moe_python.utils import get_best_config
    from alpha_moe_python.workloads import SHAPES, Weights, make_problem, make_weights

    dev = "cuda:0"
    torch.cuda.set_device(0)
    n_routings = 8

    flush_buf = torch.empty((512 << 20) // 4, dtype=torch.int32, device=dev)
    deferred_parity = []   # (result row, check) pairs run once every size has been timed

    def flush_caches(i):
        flush_buf.fill_(i)   # 512 MiB written: nothing of an earlier call is left in L2 or the Infinity Cache

    class Bench:
        """Weights of one shape (rotated copies) and the measurement of one batch size on them."""

        def __init__(self, name, cfg_path=None):
            self.shape = SHAPES[name]
            s = self.shape
            self.cfg_path = cfg_path or os.path.join(ROOT, "alpha-moe_amd", "configs", f"moe_jit_{s.E}_{s.N}_{s.K}.json")
            self.W0 = make_weights(s, device=dev, seed=0)
            self.replicas = [self.W0]
            for _ in range(max(1, args.replicas) - 1):
                W0 = self.W0
                self.replicas.append(Weights(s, W0.w1.clone(), W0.w1_scale.clone(), W0.w2.clone(), W0.w2_scale.clone()))

        def knobs_for(self, M):
            if os.path.exists(self.cfg_path):
                return dict(get_best_config(self.cfg_path, M)), os.path.relpath(self.cfg_path, ROOT)
            return dict(DEFAULT_KNOBS), "built-in"

        def prepare(self, M):
            """Problems (routing + activations) for M tokens, one per routing seed, each bound to one weight replica."""
            s = self.shape
            knobs, src = self.knobs_for(M)
            n_prob = n_routings if M <= 1024 else 3
            calls, byts, flops = [], [], []
            for i in range(n_prob):
                W = self.replicas[i % len(self.replicas)]
                P = make_problem(W, M, seed=i)
                s_ids, e_ids, total = P.align(knobs["block_m"])
                out = torch.zeros((M, s.K), dtype=torch.bfloat16, device=dev)
                byts.append(P.algorithmic_bytes())
                flops.append(P.algorithmic_flops())

                def call(P=P, W=W, s_ids=s_ids, e_ids=e_ids, total=total, out=out):
                    torch.ops.alpha_moe.fused_moe_w8a8_up_down(
                        P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total, P.topk_weights, out,
                        s.top_k, knobs["block_m"], knobs["block_n"], knobs["warp_n"], knobs["stages"], s.scaling_factor)
                calls.append(call)
            self.last = (P, W, s_ids, e_ids, total, out, knobs)
            return calls, statistics.mean(byts), statistics.mean(flops), knobs, src

        def parity_sample(self, ctx, n=12):
            """The last prepared problem's output rows for a sample of its tokens against the CPU oracle on those tokens
            alone (a token's result depends only on its own row, routing and the weights)."""
            from oracle import moe_oracle as O
            from alpha_moe_python.workloads import Problem
            P, W, s_ids, e_ids, total, out, knobs = ctx
            s = self.shape
            out.zero_()
            torch.ops.alpha_moe.fused_moe_w8a8_up_down(
                P.x, P.x_scale, W.w1, W.w1_scale, W.w2, W.w2_scale, s_ids, e_ids, total, P.topk_weights, out,
                s.top_k, knobs["block_m"], knobs["block_n"], knobs["warp_n"], knobs["stages"], s.scaling_factor)
            torch.cuda.synchronize()
            idx = torch.randperm(P.M, generator=torch.Generator().manual_seed(5))[:n].sort().values
            sub = Problem(W, len(idx), P.x[idx.to(dev)].contiguous(), P.x_scale[idx.to(dev)].contiguous(),
                          P.topk_ids[idx.to(dev)].contiguous(), P.topk_weights[idx.to(dev)].contiguous())
            ids = sub.align(16)
            # only the sample's experts cross to the host
            used = torch.unique(sub.topk_ids).long()
            remap = torch.full((s.E,), -1, dtype=torch.int32, device=dev)
            remap[used] = torch.arange(len(used), dtype=torch.int32, device=dev)
            e_sub = torch.where(ids[1] >= 0, remap[ids[1].clamp(min=0).long()], ids[1])
            ref = O.fused_moe_oracle(sub.x.cpu(), sub.x_scale.cpu(), W.w1[used].cpu(), W.w1_scale[used].cpu(),
                                     W.w2[used].cpu(), W.w2_scale[used].cpu(), ids[0].cpu(), e_sub.cpu(), ids[2].cpu(),
                                     sub.topk_weights.cpu(), torch.zeros((len(idx), s.K), dtype=torch.bfloat16),
                                     s.top_k, 16, s.scaling_factor)
            m = O.error_metrics(out[idx.to(dev)], ref)
            return {"tokens": len(idx), "max_abs_over_max_ref": round(m["max_abs_over_max_ref"], 5),
                    "cosine": round(m["cosine"], 7),
                    "ok": bool(m["max_abs_over_max_ref"] <= 1e-2 and m["cosine"] >= 0.9999)}

        def measure(self, M, steps, warmup):
            calls, B, F, knobs, src = self.prepare(M)
            # does the rotation alone keep a step's weights out of the 256 MiB Infinity Cache?
            cold = B * len(calls) < (1 << 30)
            # W untimed steps, and at least 30 ms of them: the sizes are measured back to back with host work in
            # between (building problems, the CPU oracle), and a GPU that has idled needs that long to clock up again
            t_w = time.perf_counter()
            i = 0
            while i < warmup or time.perf_counter() - t_w < 0.03:
                calls[i % len(calls)]()
                i += 1
                if i % 8 == 0:
                    torch.cuda.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(steps):
                calls[i % len(calls)]()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3 / steps
            # per-launch device time: HIP events on the launch stream (torch's current stream) around every call
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
            for i in range(steps):
                if cold:
                    flush_caches(i)
                evs[i][0].record()
                calls[i % len(calls)]()
                evs[i][1].record()
            torch.cuda.synchronize()
            dev_ms = [a.elapsed_time(b) for a, b in evs]
            r = {"M": M, "shape": self.shape.name, "ms_per_step": wall_ms, "launch_us_mean": statistics.mean(dev_ms) * 1e3,
                 "launch_us_median": statistics.median(dev_ms) * 1e3, "launch_us_min": min(dev_ms) * 1e3,
                 "bytes": B, "flops": F, "knobs": knobs, "knobs_from": src, "cold": cold}
            if not args.no_parity_samples:
                # checked after ALL timing is done: the CPU oracle takes a while, and a GPU that has idled meanwhile
                # runs the next size's short measurement at lower clocks
                ctx = self.last
                deferred_parity.append((r, lambda ctx=ctx: self.parity_sample(ctx)))
            return r

    def run_deferred_parity():
        for r, check in deferred_parity:
            r["summary"]["parity_sample"] = check()
        deferred_parity.clear()

    def summarise(r):
        t_us = r["launch_us_mean"]
        # cold rows: the wall-clock rotation may find its weights in the Infinity Cache, the flushed launches do not
        us_layer = t_us if r["cold"] else r["ms_per_step"] * 1e3
        extra = {"cold": r["cold"]}
        if r["cold"]:
            extra["us_per_layer_rotation_only"] = round(r["ms_per_step"] * 1e3, 2)
        if (r["shape"], r["M"]) in MEASURED_TRAFFIC_BYTES:
            extra["traffic_MB"] = round(MEASURED_TRAFFIC_BYTES[(r["shape"], r["M"])] / 1e6, 1)
        r["summary"] = {"us_per_layer": round(us_layer, 2), "launch_us_mean": round(t_us, 2), **extra,
                "launch_us_median": round(r["launch_us_median"], 2),
                "algorithmic_MB": round(r["bytes"] / 1e6, 1), "GB_per_s": round(r["bytes"] / t_us / 1e3, 1),
                "hbm_frac": round(r["bytes"] / t_us / 1e3 / HBM_PEAK_GBS, 4),
                "TFLOP_per_s": round(r["flops"] / t_us / 1e6, 2),
                "mfma_frac": round(r["flops"] / t_us / 1e6 / FP8_PEAK_TFLOPS, 5), "knobs": r["knobs"]}
        return r["summary"]

    def steps_for(M):
        return max(10, min(args.steps, args.steps * 64 // max(M, 64) * 2))

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.int32, device=dev)   # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    bench = Bench(args.shape, args.config)
    shape = bench.shape
    head = bench.measure(args.M, args.steps, args.warmup)
    default_others = DS_OTHER_M if args.shape == "ds" else OTHER_CONFIGS.get(args.shape, ())
    others = args.also_M if args.also_M is not None else [m for m in default_others if m != args.M]
    per_M = {str(args.M): summarise(head)}
    for m in others:
        per_M[str(m)] = summarise(bench.measure(m, steps_for(m), min(args.warmup, 5) if m > 64 else args.warmup))
    per_M = dict(sorted(per_M.items(), key=lambda kv: int(kv[0])))

    achieved = head["bytes"] / head["launch_us_mean"] / 1e3   # GB/s

    def kernel_of(knobs):
        if knobs["block_m"] <= 32:
            return "moe_stream_kernel"
        return "moe_wide_kernel" if knobs["warp_n"] == 8 else "moe_tile_kernel"
    if args.M >= 4096:   # prefill: the contraction is the bound (the weights stream once; from M ~ 8k the matrix time exceeds the HBM time)
        tflops = head["flops"] / head["launch_us_mean"] / 1e6
        roofline = {"bound": "mfma", "achieved": round(tflops, 1), "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(tflops / FP8_PEAK_TFLOPS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES.get((args.shape, args.M)),
                    "kernel": kernel_of(head["knobs"]),
                    "algorithmic_flops_per_launch": int(head["flops"]),
                    "launch_us_mean": round(head["launch_us_mean"], 2)}
    else:
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES.get((args.shape, args.M)),
                    "kernel": kernel_of(head["knobs"]),
                    "algorithmic_bytes_per_launch": int(head["bytes"]),
                    "launch_us_mean": round(head["launch_us_mean"], 2)}
    result = {
        "metric": "us_per_fused_moe_layer",
        "value": round(head["ms_per_step"] * 1e3, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {"workload": f"{shape.name}_{'prefill' if args.M >= 512 else 'decode'}_M{args.M}: E={shape.E} top_k={shape.top_k} K={shape.K} I={shape.I} "
                               f"fp8 e4m3 128x128 block scales, {len(bench.replicas)} weight copies x {n_routings} routings rotated",
                   "M": args.M, "knobs": head["knobs"], "knobs_from": head["knobs_from"]},
        "roofline": roofline,
        "per_M": per_M,
    }
    # the other half of the metric: the largest prefill size against the FP8 matrix peak (and against the binding bound:
    # the larger of the algorithmic HBM time and the algorithmic matrix time over the measured time)
    big = str(max(int(k) for k in per_M))
    if int(big) >= 4096 and int(big) != args.M:
        r = per_M[big]
        t_us = r["launch_us_mean"]
        t_hbm = r["algorithmic_MB"] * 1e6 / (HBM_PEAK_GBS * 1e9) * 1e6
        t_mfma = r["TFLOP_per_s"] * t_us / FP8_PEAK_TFLOPS
        result["roofline_prefill"] = {
            "workload": f"{shape.name}_prefill_M{big}", "bound": "mfma", "achieved": r["TFLOP_per_s"],
            "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": r["mfma_frac"], "hbm_frac": r["hbm_frac"],
            "binding_frac": round(max(t_hbm, t_mfma) / t_us, 4), "traffic": MEASURED_TRAFFIC_BYTES.get((args.shape, int(big))),
            "kernel": kernel_of(r["knobs"]), "launch_us_mean": t_us}

    if not args.no_cpu_baseline:
        # the CPU port of the reference maths on the same bits, on this box's host cores (checker, not product)
        from oracle import moe_oracle as O
        torch.set_num_threads(os.cpu_count() or 1)
        W0 = bench.W0
        Wc = Weights(shape, W0.w1.cpu(), W0.w1_scale.cpu(), W0.w2.cpu(), W0.w2_scale.cpu())
        P = make_problem(W0, args.M, seed=0)
        knobs = head["knobs"]
        s_ids, e_ids, total = P.align(knobs["block_m"])
        out = torch.zeros((args.M, shape.K), dtype=torch.bfloat16, device=dev)
        torch.ops.alpha_moe.fused_moe_w8a8_up_down(P.x, P.x_scale, W0.w1, W0.w1_scale, W0.w2, W0.w2_scale, s_ids, e_ids, total,
                                                   P.topk_weights, out, shape.top_k, knobs["block_m"], knobs["block_n"],
                                                   knobs["warp_n"], knobs["stages"], shape.scaling_factor)
        torch.cuda.synchronize()
        cpu_args = [t.cpu() for t in (P.x, P.x_scale)] + [Wc.w1, Wc.w1_scale, Wc.w2, Wc.w2_scale] + \
                   [t.cpu() for t in (s_ids, e_ids, total, P.topk_weights)]
        zero = torch.zeros((args.M, shape.K), dtype=torch.bfloat16)
        times = []
        ref = None
        t_budget = time.perf_counter()
        for _ in range(3):
            t0 = time.perf_counter()
            ref = O.fused_moe_oracle(*cpu_args, zero, shape.top_k, knobs["block_m"], shape.scaling_factor)
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - t_budget > 30:
                break
        result["cpu_baseline"] = {"value": round(statistics.median(times) * 1e6, 1), "unit": "us", "cores": torch.get_num_threads(),
                                  "kind": "port", "sample": f"same call as the headline (M={args.M}, routing seed 0), "
                                                            f"median of {len(times)} runs of oracle/moe_oracle.py (torch fp32)"}
        result["parity"] = O.error_metrics(out, ref)
        del Wc

    run_deferred_parity()
    if not args.no_other_configs and args.shape == "ds":
        del bench
        torch.cuda.empty_cache()
        other = {}
        for name, Ms in OTHER_CONFIGS.items():
            b = Bench(name)
            other[name] = {"shape": f"E={b.shape.E} top_k={b.shape.top_k} K={b.shape.K} I={b.shape.I}",
                           "per_M": {str(m): summarise(b.measure(m, steps_for(m), min(args.warmup, 5))) for m in Ms}}
            run_deferred_parity()
            del b
            torch.cuda.empty_cache()
        result["other_configs"] = other

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
