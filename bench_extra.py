"""Secondary bench workloads selected with bench.py --workload {lstm,swin,swin_merge,se,mbconv}.
Each prints the same JSON shape as the default workload."""
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


def _cpu_time(fn, budget_s):
    fn()
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        if time.perf_counter() - t0 > budget_s or n >= 50:
            break
    return (time.perf_counter() - t0) / n * 1e6, n


def _threads():
    from bench import host_threads
    return host_threads()


def _kernel_us(launch, args):
    """(min over rounds of the mean, median) of `launch()` in us, HIP events on the launch stream, the reference's
    timing rule (cpp/souffle_utils/cuda_utils.h:102-136).  `launch` is a bare C-ABI call on preallocated buffers."""
    import souffle_hip as sh
    return sh.bench_us(launch, warmup=min(20, max(2, args.warmup)), rounds=5, repeat=max(10, min(100, args.steps)))


def _floor(extra, stages, launch_us):
    """What `stages` dependent grid-wide stages cost with no arithmetic at all, beside the measured launch."""
    import souffle_hip as sh
    try:
        bar_us, floor_us = sh.stage_floor_us(stages)
        extra.update({"stages_per_launch": stages, "barriers_only_us": bar_us, "stage_chain_floor_us": floor_us,
                      "frac_of_stage_chain_floor": floor_us / launch_us})
    except sh.SouffleError as e:
        extra["stage_floor_error"] = str(e)


def _base(metric, value_us, args, workload, dtype, roof, extra):
    return {"metric": metric, "value": value_us, "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": value_us / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": {"workload": workload}, "roofline": roof, "extra": extra}


def bench_lstm(args):
    import numpy as np
    import torch
    import lstm_binding
    import synth
    from bench import time_steps
    w_ih, w_hh, x = synth.lstm_tensors(1)
    d = lambda a, t: torch.from_numpy(a).to("cuda:0", dtype=t).contiguous()
    dx, dwi, dwh = d(x, torch.float32).view(1, 100, 256), d(w_ih, torch.float16), d(w_hh, torch.float16)
    y = lstm_binding.fused_lstm(dx, dwi, dwh)[0].cpu().numpy()
    res_cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
        ref = oracle.lstm(x, w_ih, w_hh)
        dd = np.abs(y - ref)
        if not (dd.max() <= 2e-2 and dd.mean() <= 2e-3):
            print("PARITY FAILURE (lstm): %g %g" % (dd.max(), dd.mean()), file=sys.stderr)
            sys.exit(1)
        us, n = _cpu_time(lambda: oracle.lstm(x, w_ih, w_hh), min(args.cpu_seconds, 8.0))
        res_cpu = {"value": us, "unit": "us", "cores": 1, "kind": "port",
                   "sample": "%d passes of the 10x256 T=100 stack through oracle/lstm_oracle.c (scalar fp32)" % n}
    wall, ev = time_steps(lambda i: lstm_binding.fused_lstm(dx, dwi, dwh), args.steps, args.warmup)
    bytes_alg = 5242880 * 2 + 2 * 51200 * 2
    ach = bytes_alg / (ev * 1e-3) / 1e9
    roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None,
            "kernel": "k_lstm", "algorithmic_bytes_per_launch": bytes_alg, "avg_launch_us": ev * 1e3,
            "note": "109 dependent wavefront steps bound the latency, not the one-time 10.5 MB weight stream"}
    extra = {"us_per_wavefront_step": ev * 1e3 / 109}
    _floor(extra, 109, ev * 1e3)
    res = _base("lstm_stack_latency_us", wall * 1e3, args, "stacked LSTM 10x256, T=100, batch 1 (BASELINE configs[1])", "f16",
                roof, extra)
    if res_cpu:
        res["cpu_baseline"] = res_cpu
    return res


def bench_swin(args):
    import numpy as np
    import torch
    import swin_transformer_binding as sb
    import synth
    from bench import time_steps
    ws = [synth.swin_block_weights(3, b) for b in range(2)]
    x = synth.swin_input(3)
    dw = [{k: torch.from_numpy(v).cuda() for k, v in w.items()} for w in ws]
    dx = torch.from_numpy(x).cuda()
    y = sb.swin_block_pair(dx, dw[0], dw[1]).float().cpu().numpy()
    res_cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
        ref = oracle.swin_block_pair(x, ws)
        dd = np.abs(y - ref)
        if not (dd.max() <= 2e-2 and dd.mean() <= 2e-3):
            print("PARITY FAILURE (swin): %g %g" % (dd.max(), dd.mean()), file=sys.stderr)
            sys.exit(1)
        thr = _threads()
        us, n = _cpu_time(lambda: oracle.swin_block_pair(x, ws, threads=thr), min(args.cpu_seconds, 8.0))
        res_cpu = {"value": us, "unit": "us", "cores": thr, "kind": "port",
                   "sample": "%d passes of the 56x56x128 block pair through oracle/swin_oracle.c (OpenMP fp32)" % n}
    launch = sb.block_pair_launcher(dx, dw[0], dw[1], torch.empty_like(dx))       # bare C-ABI call, output preallocated
    wall, ev = time_steps(lambda i: launch(), args.steps, args.warmup)
    mn, med = _kernel_us(launch, args)
    flops = 2 * (2.0 * 3136 * 196608 + 4.0 * 64 * 4 * 49 * 49 * 32)
    ach = flops / (ev * 1e-3) / 1e12
    roof = {"bound": "mfma", "achieved": ach, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": ach / MFMA_F16_PEAK_TFLOPS,
            "traffic": None, "kernel": "k_block_pair", "algorithmic_flops_per_launch": flops, "avg_launch_us": ev * 1e3}
    extra = {"kernel_us_min_of_means": mn, "kernel_us_median": med}
    _floor(extra, sb.BLOCK_PAIR_GRID_STAGES, ev * 1e3)
    res = _base("swin_block_pair_latency_us", wall * 1e3, args,
                "Swin-Base stage-1 block pair 56x56, C=128, 4 heads, window 7, shift 3 (BASELINE configs[3])", "f16", roof, extra)
    if res_cpu:
        res["cpu_baseline"] = res_cpu
    return res


def bench_se(args):
    import torch
    import efficientnet_se_module_binding as eb
    from bench import time_steps
    shapes = [(32, 112, 8), (96, 56, 4), (144, 56, 6), (144, 28, 6), (240, 28, 10), (240, 14, 10), (480, 14, 20),
              (672, 14, 28), (672, 7, 28), (1152, 7, 48)]
    a100 = [23.33, 14.14, 15.65, 12.48, 12.86, 12.03, 12.86, 13.86, 13.28, 15.36]   # cpp/efficientnet/scripts/efficientnet-se_module_v2-max-block.xlsx, column "Duration [usecond]", A100
    rows = []
    for (Cc, Hh, R), ref_us in zip(shapes, a100):
        x = torch.rand((1, Cc, Hh, Hh), device="cuda:0")
        wr, we = torch.randn((R, Cc), device="cuda:0") * 0.3, torch.randn((Cc, R), device="cuda:0") * 0.3
        print("se shape C=%d H=%d R=%d" % (Cc, Hh, R), file=sys.stderr, flush=True)
        launch = eb.se_launcher(x, wr, we, torch.empty_like(x), torch.empty((1, Cc), device="cuda:0"), combine="add")
        wall, ev = time_steps(lambda i: launch(), args.steps, args.warmup)
        mn, med = _kernel_us(launch, args)
        rows.append({"C": Cc, "H": Hh, "R": R, "us": ev * 1e3, "kernel_us_min_of_means": mn, "reference_a100_us": ref_us,
                     "vs_reference_a100": ref_us / mn, "GBps": 2.0 * Cc * Hh * Hh * 4 / (mn * 1e-6) / 1e9})
    tot = sum(r["us"] for r in rows)
    byt = sum(2.0 * r["C"] * r["H"] ** 2 * 4 for r in rows)
    ach = byt / (tot * 1e-6) / 1e9
    roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None,
            "kernel": "k_se", "avg_launch_us": tot / len(rows)}
    extra = {"per_shape": rows, "reference_a100_sum_us": sum(a100), "kernel_us_min_of_means_sum": sum(r["kernel_us_min_of_means"] for r in rows)}
    _floor(extra, 2, tot / len(rows))          # pool -> (grid barrier) -> gate and combine
    return _base("se_module_latency_us_sum_of_10_shapes", tot, args, "EfficientNet-B0 SE module, the reference's 10 shapes, fp32", "f32",
                 roof, extra)


def bench_mbconv(args):
    import numpy as np
    import torch
    import efficientnet_binding as eb
    import synth
    from bench import time_steps
    blocks = synth.mbconv_stack_weights()
    x = synth.mbconv_input()

    def up(v):
        return torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v
    stack = eb.MBConvStack([{k: up(v) for k, v in b.items()} for b in blocks])
    dx = torch.from_numpy(x).cuda()
    y = stack(dx).float().cpu().numpy()
    res_cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
        thr = _threads()
        ref = oracle.mbconv_stack(x, blocks, threads=thr)
        dd = np.abs(y - ref)
        if not (dd.max() <= 2e-2 and dd.mean() <= 2e-3):
            print("PARITY FAILURE (mbconv): %g %g" % (dd.max(), dd.mean()), file=sys.stderr)
            sys.exit(1)
        us, n = _cpu_time(lambda: oracle.mbconv_stack(x, blocks, threads=thr), min(args.cpu_seconds, 8.0))
        res_cpu = {"value": us, "unit": "us", "cores": thr, "kind": "port",
                   "sample": "%d passes of the 16-block stack through oracle/mbconv_oracle.c (OpenMP fp32)" % n}
    wall_u, ev_u = time_steps(lambda i: stack(dx, fused=False), max(10, args.steps // 4), args.warmup)
    wall, ev = time_steps(lambda i: stack(dx), args.steps, args.warmup)
    # algorithmic bytes: every weight tensor once, the input image and the result
    wbytes = sum(v.nbytes for b in blocks for v in b.values() if isinstance(v, np.ndarray))
    bytes_alg = wbytes + x.nbytes + y.size * 2
    flops = 0.0
    for b in blocks:
        hw, oh = b["in_h"] * b["in_w"], ((b["in_h"] - 1) // b["stride"] + 1) ** 2
        flops += 2.0 * hw * b["in_c"] * b["expand_c"] * (b["expand_w"] is not None) + 2.0 * oh * b["kernel"] ** 2 * b["expand_c"] + \
            2.0 * oh * b["expand_c"] * b["out_c"]
    ach = bytes_alg / (ev * 1e-3) / 1e9
    # barrier-separated steps of the launch: expand (where a block has one), depthwise, gate, project
    stages = sum(4 if b["expand_w"] is not None else 3 for b in blocks)
    roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None,
            "kernel": "k_mbconv", "algorithmic_bytes_per_launch": bytes_alg, "algorithmic_flops_per_launch": flops,
            "avg_launch_us": ev * 1e3,
            "note": "%d dependent barrier-separated steps bound the latency, not the %.1f MB of weights and activations" % (stages, bytes_alg / 1e6)}
    extra = {"unfused_per_op_us": ev_u * 1e3, "stages": stages, "us_per_stage": ev * 1e3 / stages}
    _floor(extra, stages, ev * 1e3)
    res = _base("mbconv_stack_latency_us", wall * 1e3, args,
                "EfficientNet-B0 MBConv stack (16 blocks), 112x112x32 -> 7x7x320, batch 1, fp16 (BASELINE configs[4])", "f16", roof,
                extra)
    if res_cpu:
        res["cpu_baseline"] = res_cpu
    return res


def bench_swin_merge(args):
    import numpy as np
    import torch
    import swin_transformer_binding as sb
    import synth
    from bench import time_steps
    H = W = 56
    Cc = 128
    x = synth.swin_input(3)
    w = synth.f16(synth.normal(synth.seed_of(3, 200), (4 * Cc, 2 * Cc), 0.02))
    g = synth.f16(1.0 + synth.normal(synth.seed_of(3, 201), (4 * Cc,), 0.1))
    b = synth.f16(synth.normal(synth.seed_of(3, 202), (4 * Cc,), 0.1))
    dx, dw, dg, db = [torch.from_numpy(a).cuda() for a in (x, w, g, b)]
    y = sb.patch_merging(dx, H, W, dg, db, dw).float().cpu().numpy()
    res_cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
        thr = _threads()
        ref = oracle.swin_patch_merge(x, H, W, g, b, w, threads=thr)
        dd = np.abs(y - ref)
        if not (dd.max() <= 2e-2 and dd.mean() <= 2e-3):
            print("PARITY FAILURE (swin_merge): %g %g" % (dd.max(), dd.mean()), file=sys.stderr)
            sys.exit(1)
        us, n = _cpu_time(lambda: oracle.swin_patch_merge(x, H, W, g, b, w, threads=thr), min(args.cpu_seconds, 5.0))
        res_cpu = {"value": us, "unit": "us", "cores": thr, "kind": "port",
                   "sample": "%d passes of the 56x56x128 patch merge through oracle/swin_oracle.c (OpenMP fp32)" % n}
    launch = sb.patch_merge_launcher(dx, H, W, dg, db, dw, torch.empty((H // 2 * (W // 2), 2 * Cc), dtype=torch.float16, device="cuda:0"))
    wall, ev = time_steps(lambda i: launch(), args.steps, args.warmup)
    mn, med = _kernel_us(launch, args)
    bytes_alg = x.nbytes + w.nbytes + g.nbytes + b.nbytes + y.size * 2
    ach = bytes_alg / (ev * 1e-3) / 1e9
    roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None,
            "kernel": "k_patch_merge", "algorithmic_bytes_per_launch": bytes_alg,
            "algorithmic_flops_per_launch": 2.0 * 784 * 512 * 256, "avg_launch_us": ev * 1e3,
            "note": "one launch of 1.5 MB and 0.2 GFLOP: launch and memory latency, not bandwidth"}
    res = _base("swin_patch_merge_latency_us", wall * 1e3, args, "Swin patch merging 56x56x128 -> 28x28x256, fp16", "f16", roof,
                {"kernel_us_min_of_means": mn, "kernel_us_median": med})
    if res_cpu:
        res["cpu_baseline"] = res_cpu
    return res


def _parity(name, got, ref, max_abs=2e-2, mean_abs=2e-3):
    import numpy as np
    d = np.abs(np.asarray(got, np.float32).reshape(-1) - np.asarray(ref, np.float32).reshape(-1))
    if not (np.isfinite(got).all() and d.max() <= max_abs and d.mean() <= mean_abs):
        print("PARITY FAILURE (%s): max-abs %.4g mean-abs %.4g" % (name, d.max(), d.mean()), file=sys.stderr)
        sys.exit(1)
    return {"max_abs": float(d.max()), "mean_abs": float(d.mean())}


def sub_results(args):
    """The other BASELINE configurations as short sub-results of the default line: each checked against the CPU oracle
    first (unless --no-cpu) and then timed as bare C-ABI launches on preallocated outputs (HIP events on the launch
    stream, min over rounds of the mean: the reference's timing rule)."""
    import numpy as np
    import torch
    import souffle_hip as sh
    import synth
    out = {}
    oracle = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle
    thr = _threads()
    timed = lambda launch: sh.bench_us(launch, warmup=10, rounds=3, repeat=max(10, min(50, args.steps)))

    # configs[1]: stacked LSTM
    import lstm_binding
    w_ih, w_hh, x = synth.lstm_tensors(1)
    d = lambda a, t: torch.from_numpy(a).to("cuda:0", dtype=t).contiguous()
    dx, dwi, dwh = d(x, torch.float32).view(1, 100, 256), d(w_ih, torch.float16), d(w_hh, torch.float16)
    y = lstm_binding.fused_lstm(dx, dwi, dwh)[0].cpu().numpy()
    par = _parity("lstm", y, oracle.lstm(x, w_ih, w_hh)) if oracle else None
    mn, med = timed(lambda: lstm_binding.fused_lstm(dx, dwi, dwh))
    out["lstm"] = {"workload": "stacked LSTM 10x256, T=100, batch 1 (BASELINE configs[1])", "us": mn, "median_us": med, "parity": par,
                   "us_per_wavefront_step": mn / 109, "note": "109 dependent steps; timed through the binding (it allocates the output)"}

    # configs[3]: Swin block pair
    import swin_transformer_binding as sb
    ws = [synth.swin_block_weights(3, b) for b in range(2)]
    xs = synth.swin_input(3)
    dw = [{k: torch.from_numpy(v).cuda() for k, v in w.items()} for w in ws]
    dxs = torch.from_numpy(xs).cuda()
    ys = torch.empty_like(dxs)
    launch = sb.block_pair_launcher(dxs, dw[0], dw[1], ys)
    launch()
    par = _parity("swin", ys.float().cpu().numpy(), oracle.swin_block_pair(xs, ws, threads=thr)) if oracle else None
    mn, med = timed(launch)
    flops = 2 * (2.0 * 3136 * 196608 + 4.0 * 64 * 4 * 49 * 49 * 32)
    out["swin_pair"] = {"workload": "Swin-Base stage-1 block pair 56x56, C=128, window 7, shift 3 (BASELINE configs[3])", "us": mn, "median_us": med,
                        "parity": par, "mfma_frac": flops / (mn * 1e-6) / 1e12 / MFMA_F16_PEAK_TFLOPS}

    # the reference's SE module, its ten shapes (fp32; tolerance 1e-4 relative to the largest value)
    import efficientnet_se_module_binding as eb
    shapes = [(32, 112, 8), (96, 56, 4), (144, 56, 6), (144, 28, 6), (240, 28, 10), (240, 14, 10), (480, 14, 20),
              (672, 14, 28), (672, 7, 28), (1152, 7, 48)]
    a100 = [23.33, 14.14, 15.65, 12.48, 12.86, 12.03, 12.86, 13.86, 13.28, 15.36]   # cpp/efficientnet/scripts/efficientnet-se_module_v2-max-block.xlsx, "Duration [usecond]", A100
    rows, worst = [], 0.0
    g = torch.Generator(device="cpu").manual_seed(5)
    for (Cc, Hh, R), ref_us in zip(shapes, a100):
        xn = torch.rand((1, Cc, Hh, Hh), generator=g).numpy()
        wr, we = (torch.randn((R, Cc), generator=g) * 0.3).numpy(), (torch.randn((Cc, R), generator=g) * 0.3).numpy()
        xd, wrd, wed = torch.from_numpy(xn).cuda(), torch.from_numpy(wr).cuda(), torch.from_numpy(we).cuda()
        yd, pd = torch.empty_like(xd), torch.empty((1, Cc), device="cuda:0")
        launch = eb.se_launcher(xd, wrd, wed, yd, pd, combine="add")
        launch()
        if oracle:
            ref = oracle.se_module(xn.reshape(Cc, Hh * Hh), wr, we, combine="add")
            ref_y = ref[0] if isinstance(ref, (tuple, list)) else ref
            err = float(np.abs(yd.cpu().numpy().reshape(-1) - np.asarray(ref_y, np.float32).reshape(-1)).max() / max(1.0, float(np.abs(ref_y).max())))
            if not err <= 1e-4:
                print("PARITY FAILURE (se C=%d H=%d): relative error %.3g" % (Cc, Hh, err), file=sys.stderr)
                sys.exit(1)
            worst = max(worst, err)
        mn, _ = timed(launch)
        rows.append({"C": Cc, "H": Hh, "R": R, "us": mn, "reference_a100_us": ref_us, "vs_reference_a100": ref_us / mn})
    out["se"] = {"workload": "EfficientNet-B0 SE module, the reference's 10 shapes, fp32, combine = add as in the reference", "us": sum(r["us"] for r in rows),
                 "parity": {"max_rel": worst} if oracle else None, "reference_a100_sum_us": sum(a100), "per_shape": rows}

    # configs[4]: MBConv stack
    import efficientnet_binding as efb
    blocks = synth.mbconv_stack_weights()
    xm = synth.mbconv_input()
    up = lambda v: torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v
    stack = efb.MBConvStack([{k: up(v) for k, v in b.items()} for b in blocks])
    dxm = torch.from_numpy(xm).cuda()
    ym = stack(dxm).float().cpu().numpy()
    par = _parity("mbconv", ym, oracle.mbconv_stack(xm, blocks, threads=thr)) if oracle else None
    mn, med = timed(lambda: stack(dxm))
    stages = sum(4 if b["expand_w"] is not None else 3 for b in blocks)
    out["mbconv"] = {"workload": "EfficientNet-B0 MBConv stack (16 blocks), 112x112x32 -> 7x7x320, fp16 (BASELINE configs[4], behind the stem)", "us": mn,
                     "median_us": med, "parity": par, "stages": stages, "us_per_stage": mn / stages}
    return out


def run(args):
    if args.workload == "swin_merge":
        return bench_swin_merge(args)
    if args.workload == "mbconv":
        return bench_mbconv(args)
    if args.workload == "lstm":
        return bench_lstm(args)
    if args.workload == "swin":
        return bench_swin(args)
    if args.workload == "se":
        return bench_se(args)
    print("unknown workload %r" % args.workload, file=sys.stderr)
    sys.exit(2)
