#!/usr/bin/env python3
"""Benchmark of the fused-encoder hot path on one MI355X.

Default workload (the metric of BASELINE.json): the BERT-base 12-layer encoder at B=1,
S=128, fp16, one persistent launch per forward pass (a plain launch of a co-resident grid; the
cooperative launch is timed beside it).  A step is one forward
pass over one synthetic input; the timed passes rotate through several distinct weight
sets (> 512 MB in total) so that the weight stream comes from HBM, not from the 256 MB
Infinity Cache.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload encoder|layer|encoder_s384|encoder_b32|lstm|swin|swin_merge|se|mbconv]
"""
import argparse
import json
import re
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "souffle-models_amd"))

HBM_PEAK_GBS = 8000.0            # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0    # MI355X published dense fp16 MFMA peak

# algorithmic HBM bytes / flops of one encoder layer (weights once + biases + LN vectors + x in + y out)
def layer_bytes(M):
    return 7077888 * 2 + 13824 + 6144 + 2 * M * 768 * 2


def layer_flops(B, S):
    return 2.0 * B * S * 7077888 + 4.0 * B * S * S * 768


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="encoder")
    p.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU-baseline sample")
    p.add_argument("--no-cpu", action="store_true")
    p.add_argument("--no-sub", action="store_true", help="skip the sub-results of the default workload (S=384, B=32, LSTM, Swin, SE, MBConv)")
    p.add_argument("--no-coop", action="store_true", help="skip the cooperative-launch timing of the encoder workloads")
    p.add_argument("--no-strict", action="store_true", help="skip the strict-fence timing of the encoder workloads")
    p.add_argument("--weight-sets", type=int, default=4)
    p.add_argument("--no-pack", action="store_true", help="encoders keep the [K][N] FC2 matrices only (split-K FC2) instead of packing them once")
    return p.parse_args()


def host_threads():
    """The cores this process may run on (its affinity mask; every one of them is used)."""
    try:
        return len(os.sched_getaffinity(0))
    except Exception:
        return os.cpu_count() or 1


def cpu_baseline_encoder(layers_np, x_np, B, S, budget_s):
    """The CPU oracle (a port: the reference has no CPU path) timed on the host cores."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle
    threads = host_threads()
    print("cpu_baseline: %d cores in the affinity mask (os.cpu_count() = %s), %d OpenMP threads" % (threads, os.cpu_count(), threads),
          file=sys.stderr)
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    oracle.bert_encoder(x_np, layers_np[:1], B, S, threads=threads)       # warm up
    n, t0 = 0, time.perf_counter()
    ref = None
    while True:
        ref = oracle.bert_encoder(x_np, layers_np, B, S, threads=threads)
        n += 1
        if time.perf_counter() - t0 > budget_s or n >= 50:
            break
    dt = (time.perf_counter() - t0) / n
    return ref, {"value": dt * 1e6, "unit": "us", "cores": threads, "kind": "port",
                 "sample": "%d passes of the %d-layer encoder B=%d S=%d through oracle/bert_oracle.c (OpenMP fp32)" % (n, len(layers_np), B, S)}


def traffic_from_profile(name):
    """HBM bytes per launch from the tracked counter summary profiles/<name> (a line
    'traffic_bytes_per_launch: <number>' written when the summary was made), None if there is none."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", f.read(), re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def encoder_sub_result(args, B, S, L=12):
    """One more shape of the same encoder for the default line: parity against the oracle (unless --no-cpu), then
    the event-timed launch and its place under the roofline that bounds it."""
    import numpy as np
    import torch
    import bert_binding
    import synth
    dev = torch.device("cuda:0")
    layers_np = [synth.bert_layer_weights(2, l) for l in range(L)]
    x_np = synth.bert_input(2, B, S)
    enc = bert_binding.Encoder([{k: torch.from_numpy(v).to(dev) for k, v in w.items()} for w in layers_np], B, S, pack=not args.no_pack)
    x = torch.from_numpy(x_np).to(dev)
    out = torch.empty((B * S, 768), dtype=torch.float16, device=dev)
    y = enc(x, out=out).float().cpu().numpy()
    parity = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
        ref = oracle.bert_encoder(x_np, layers_np, B, S, threads=host_threads())
        d = np.abs(y - ref)
        if not (np.isfinite(y).all() and d.max() <= 2e-2 and d.mean() <= 2e-3):
            print("PARITY FAILURE (B=%d S=%d): max-abs %.4g mean-abs %.4g" % (B, S, d.max(), d.mean()), file=sys.stderr)
            sys.exit(1)
        parity = {"max_abs": float(d.max()), "mean_abs": float(d.mean())}
    _, ev = time_steps(lambda i: enc(x, out=out), max(20, args.steps // 4), MIN_WARMUP)
    flops, bytes_alg = L * layer_flops(B, S), L * layer_bytes(B * S)
    tf, gbs = flops / (ev * 1e-3) / 1e12, bytes_alg / (ev * 1e-3) / 1e9
    return {"us": ev * 1e3, "parity": parity, "TFLOPs": tf, "mfma_frac": tf / MFMA_F16_PEAK_TFLOPS, "GBps": gbs,
            "hbm_frac": gbs / HBM_PEAK_GBS, "bound": "mfma" if flops / (MFMA_F16_PEAK_TFLOPS * 1e12) > bytes_alg / (HBM_PEAK_GBS * 1e9) else "hbm"}


# The few-rows encoder decides in the first 8 launches on a workspace which copy of its hand-over words every XCD polls
# (each of those launches ends with a 3 us vote) and keeps its wait masks there from the first launch on: at least this
# many untimed launches go in front of every timed region of an encoder, whatever --warmup says.
MIN_WARMUP = 10


def time_steps(launch, steps, warmup):
    """W untimed steps, then exactly K timed steps bracketed by synchronize on both sides;
    HIP events on the launch stream give the average launch duration."""
    import torch
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        launch(i)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps
    return wall_ms, ev_ms


def bench_encoder(args, B, S, L, name):
    import numpy as np
    import torch
    import bert_binding
    import souffle_hip as sh
    import synth

    dev = torch.device("cuda:0")
    to_dev = lambda w: {k: torch.from_numpy(v).to(dev) for k, v in w.items()}
    layers_np = [synth.bert_layer_weights(2, l) for l in range(L)]
    x_np = synth.bert_input(2, B, S)
    x = torch.from_numpy(x_np).to(dev)
    M = B * S
    # distinct weight sets for the cold-cache rotation (set 0 is the checked one; the others
    # are shuffled copies: same sizes and value distribution, different addresses)
    sets = [[to_dev(w) for w in layers_np]]
    for s in range(1, max(1, args.weight_sets)):
        sets.append([{k: v.clone() for k, v in sets[0][(l + s) % L].items()} for l in range(L)])
    encs = [bert_binding.Encoder(ls, B, S, pack=not args.no_pack) for ls in sets]
    out = torch.empty((M, 768), dtype=torch.float16, device=dev)

    # parity gate
    cpu = None
    y = encs[0](x, out=out).float().cpu().numpy()
    if not args.no_cpu:
        ref, cpu = cpu_baseline_encoder(layers_np, x_np, B, S, args.cpu_seconds)
        d = np.abs(y - ref)
        if not (np.isfinite(y).all() and d.max() <= 2e-2 and d.mean() <= 2e-3):
            print("PARITY FAILURE: max-abs %.4g mean-abs %.4g" % (d.max(), d.mean()), file=sys.stderr)
            sys.exit(1)
        parity = {"max_abs": float(d.max()), "mean_abs": float(d.mean())}
    else:
        parity = None

    wu = max(args.warmup, MIN_WARMUP)
    cold_wall, cold_ev = time_steps(lambda i: encs[i % len(encs)](x, out=out), args.steps, wu)
    warm_wall, warm_ev = time_steps(lambda i: encs[0](x, out=out), args.steps, wu)
    unf_wall, unf_ev = time_steps(lambda i: encs[i % len(encs)](x, out=out, fused=False), max(10, args.steps // 4), 5)
    # the per-op chain again as one HIP graph (no launch gaps): the strongest form of the unfused baseline
    graph_ev = None
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            encs[0](x, out=out, fused=False)
        _, graph_ev = time_steps(lambda i: g.replay(), max(10, args.steps // 4), 5)
    except Exception as e:                      # a capture failure must not cost the headline number
        print("graph capture of the per-op chain failed: %s" % e, file=sys.stderr)
    # the reference's own timing rule (min over rounds of the mean of repeated event-timed launches)
    mn, med = sh.bench_us(lambda: encs[0](x, out=out), warmup=10, rounds=5, repeat=max(10, args.steps // 5))

    bytes_alg = L * layer_bytes(M)
    flops = L * layer_flops(B, S)
    mfma_bound = flops / (MFMA_F16_PEAK_TFLOPS * 1e12) > bytes_alg / (HBM_PEAK_GBS * 1e9)
    if mfma_bound:
        ach = flops / (cold_ev * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / MFMA_F16_PEAK_TFLOPS, "traffic": None}
    else:
        ach = bytes_alg / (cold_ev * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS,
                "traffic": None}
    few_rows = M <= 1024 or (M < 1536 and M % 256 != 0)       # (the library's own rule: many_rows() in csrc/bert.hip)
    if (B, S, L) == (1, 128, 12):
        # L2<->fabric bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a device copy of
        # known size: read from the tracked summary, so the figure cannot outlive the kernel it was measured on
        roof["traffic"] = traffic_from_profile("k_encoder_small_bert_encoder_b1_s128_hbm_traffic.txt")
    roof["kernel"] = "%s (one launch = %d layers)" % ("k_encoder_small" if few_rows else "k_encoder_mega", L)
    roof["algorithmic_bytes_per_launch"] = bytes_alg
    roof["algorithmic_flops_per_launch"] = flops
    roof["avg_launch_us"] = cold_ev * 1e3
    # `achieved` and `frac` are over the kernel's average launch duration (HIP events around the timed region, on the
    # launch stream); `value` is the wall clock per step, which also holds the host's launch cost: the same fraction over it
    roof["clock"] = "HIP events around the %d timed launches" % args.steps
    roof["frac_over_wall_clock_value"] = (flops / (cold_wall * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS) if mfma_bound else (bytes_alg / (cold_wall * 1e-3) / 1e9 / HBM_PEAK_GBS)
    res = {
        "metric": "bert_base_encoder_latency_us", "value": cold_wall * 1e3, "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": cold_wall, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": name, "batch": B, "seq_len": S, "layers": L, "hidden": 768, "heads": 12, "ffn": 3072,
                   "weights": "random N(0,0.02) fp16, %d rotating sets" % len(encs)},
        "roofline": roof,
        "extra": {"per_layer_us_cold": cold_ev * 1e3 / L, "warm_cache_us": warm_ev * 1e3, "per_layer_us_warm": warm_ev * 1e3 / L,
                  "unfused_per_op_us": unf_ev * 1e3, "fused_speedup_vs_unfused": unf_ev / cold_ev,
                  "unfused_per_op_hip_graph_us": None if graph_ev is None else graph_ev * 1e3,
                  "min_of_means_us_warm": mn, "median_us_warm": med, "parity": parity,
                  "launches_fused": 1, "launches_unfused": 5 * L + 1 if few_rows else 7 * L},
    }
    # empirical ceilings of this device beside the published ones: device-to-device copy and an MFMA-only loop
    try:
        copy_gbs, mfma_tflops = sh.measured_ceilings()
        roof["measured_copy_GBps"] = copy_gbs
        roof["measured_mfma_f16_TFLOPs"] = mfma_tflops
        roof["measured_l2_to_lds_GBps"] = sh.measured_l2_stream_gbs()     # all CUs streaming L2-resident operands
        roof["frac_of_measured"] = ach / (mfma_tflops if mfma_bound else copy_gbs)
        if (B, S) == (1, 384):            # mixed shape: both fractions
            roof["mfma_frac"] = flops / (cold_ev * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS
        if few_rows:
            # Five phases per layer (QKV, attention, out-projection, FC1, FC2 with the split-K sum finished by the last
            # of a tile's four workgroups) and the final LayerNorm follow one another through flag hand-overs among the
            # workgroups that exchange data; no grid barrier.  The yardstick beside it: a chain of as many grid-wide
            # stages with no arithmetic at all.
            nst = 5 * L + 1
            bar_us, floor_us = sh.stage_floor_us(nst)
            res["extra"]["stages_per_launch"] = nst
            res["extra"]["grid_barriers_per_launch"] = 0
            res["extra"]["barriers_only_us"] = bar_us
            res["extra"]["stage_chain_floor_us"] = floor_us
            res["extra"]["frac_of_stage_chain_floor"] = floor_us / (cold_ev * 1e3)
    except sh.SouffleError as e:
        roof["measured_ceilings_error"] = str(e)
    # the same launch as a cooperative one (hipLaunchCooperativeKernel): the co-residency the hand-overs need is then
    # guaranteed by the runtime instead of checked with the occupancy query
    try:
        if args.no_coop:
            raise sh.SouffleError(0, "skipped (--no-coop)")
        sh.set_cooperative_launch(1)
        _, coop_ev = time_steps(lambda i: encs[i % len(encs)](x, out=out), max(20, args.steps // 2), 5)
        res["extra"]["cooperative_launch_us"] = coop_ev * 1e3
    except sh.SouffleError as e:
        res["extra"]["cooperative_launch_error"] = str(e)
    finally:
        sh.set_cooperative_launch(0)
    # the same launch with the memory model's release / acquire fences around every hand-over (souffle_set_strict_fences):
    # the by-the-book form, same bits (tests/test_strict_fences.py), kept as a fallback
    try:
        if args.no_strict:
            raise sh.SouffleError(0, "skipped (--no-strict)")
        sh.set_strict_fences(True)
        _, strict_ev = time_steps(lambda i: encs[i % len(encs)](x, out=out), max(10, args.steps // 4), 3)
        res["extra"]["strict_fences_us"] = strict_ev * 1e3
    except sh.SouffleError as e:
        res["extra"]["strict_fences_error"] = str(e)
    finally:
        sh.set_strict_fences(False)
    if cpu:
        res["cpu_baseline"] = cpu
        res["extra"]["gpu_speedup_vs_cpu"] = cpu["value"] / (cold_ev * 1e3)
    return res


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("no GPU available", file=sys.stderr)
        sys.exit(3)
    if args.workload == "encoder":
        sub = {}
        if not args.no_sub:
            import bench_extra
            sub = {"encoder_s384": encoder_sub_result(args, 1, 384), "encoder_b32": encoder_sub_result(args, 32, 128)}
            sub.update(bench_extra.sub_results(args))
        res = bench_encoder(args, 1, 128, 12, "BERT-base 12-layer encoder, B=1, S=128, fp16 (BASELINE configs[2], first shape)")
        res["extra"].update(sub)
    elif args.workload == "layer":
        res = bench_encoder(args, 1, 128, 1, "single BERT-base encoder layer, B=1, S=128, fp16 (BASELINE configs[0])")
    elif args.workload == "encoder_s384":
        res = bench_encoder(args, 1, 384, 12, "BERT-base 12-layer encoder, B=1, S=384, fp16")
    elif args.workload == "encoder_b32":
        args.weight_sets = 1
        res = bench_encoder(args, 32, 128, 12, "BERT-base 12-layer encoder, B=32, S=128, fp16 (MFMA-bound shape)")
    elif re.fullmatch(r"encoder_b(\d+)_s(\d+)", args.workload):
        # any other shape of the 12-layer encoder (development aid: the bench lines of record are the named workloads)
        B, S = (int(v) for v in re.fullmatch(r"encoder_b(\d+)_s(\d+)", args.workload).groups())
        res = bench_encoder(args, B, S, 12, "BERT-base 12-layer encoder, B=%d, S=%d, fp16" % (B, S))
    elif args.workload == "copy":
        # A plain device copy of known size: the calibration run for the FETCH_SIZE / WRITE_SIZE
        # counters (counter reading per byte actually read / written).
        n = 256 << 20
        a = torch.empty(n, dtype=torch.uint8, device="cuda:0").fill_(1)
        b = torch.empty_like(a)
        for _ in range(max(1, args.steps // 20)):
            b.copy_(a)
        torch.cuda.synchronize()
        res = {"workload": "copy", "bytes_read_per_copy": n, "bytes_written_per_copy": n, "copies": max(1, args.steps // 20)}
    else:
        import bench_extra
        res = bench_extra.run(args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
