#!/usr/bin/env python3
"""Headline benchmark: requests/s of the serving hot path on one MI355X.

A "step" is one request served end to end: client library -> shared-memory request ring -> server poll loop
-> full3 block-level scheduler -> one HIP kernel per stage with workgroup start/end notifications -> copy out
-> completion.  Workload at N=1: ResNet-18 (batch 1, fp32, 1x3x224x224, seeded weights, synthetic input),
the configuration the metric is quoted on.  W warm-up requests are served untimed, then exactly K requests
are timed from first submission to last completion with the arrival process at saturation (closed by
--concurrency outstanding requests, the reference's `--iat 0` mode); `value` = K / elapsed.

Next to it, in the same run: the comparison arms (job-by-job `fifo` on a stream pool = plain multi-stream
serving, `fifo` on one stream, and a direct single-stream forward loop without any server), an open-loop
Poisson sweep with p50/p99, the roofline of the dominant kernel (MFMA implicit-GEMM conv, per-launch HIP
events on its stream), the GPU->host notification latency probes and the CPU oracle timed on the host cores.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "requests/sec at p99 latency SLO (mixed-model Poisson load, 1 GPU); notify latency µs"
FP32_MFMA_PEAK_TFLOPS = 157.3


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# HBM-side bytes per conv launch (mean over the conv launches of one forward pass), from the FETCH_SIZE / WRITE_SIZE
# counter passes of `bench.py --roofline-only` scaled by the copy-kernel calibration (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0);
# counters cannot be collected from inside this process, so the figure is carried here and is null for other models.
CONV_TRAFFIC_BYTES_PER_LAUNCH = {"resnet18": 7.10e6}  # 17 launches: 20 convs, 3 of them sharing a launch with another


def serve_arm(serve, sched, streams, jobs, concurrency, steps, warmup, iat_us=0.0, seed=1, mem_marker=True, extra_kernels=2, unfair=1e6,
              dist="exp", ln_sigma=2.0):
    name = "bench%d_%s_%d" % (os.getpid(), sched, int(time.time() * 1000) % 100000)
    with serve.Server(name, sched, num_streams=streams, mem_marker=mem_marker, cpu=4, extra_kernels=extra_kernels, unfair=unfair) as srv:
        r = serve.client_run(srv.name, jobs, iat_us, concurrency, steps, warmup_jobs=warmup, seed=seed, dist=dist, ln_sigma=ln_sigma,
                             pin_threads=True)
    return r


def conv_roofline(models, hip, model, reps):
    """Per-launch durations of every stage of one forward pass, measured with HIP events on the launch stream."""
    ex = models.Exec(model, seed=1)
    stream = ctypes.c_void_p()
    hip.llis_hip_stream_create(ctypes.byref(stream))
    n = ex.num_stages
    ops = models._abi.ops()
    ev = []
    for _ in range(2):
        e = ctypes.c_void_p()
        hip.llis_hip_event_create(ctypes.byref(e))
        ev.append(e)
    work = [ex.stage_work(i) for i in range(n)]
    for _ in range(3):
        ex.forward(stream)
    hip.llis_hip_stream_synchronize(stream)
    # Each launch stamps the event pair with the kernel's own begin/end time on the device (what a kernel trace
    # reports); one launch at a time on an otherwise idle GPU, in forward-pass order so caches see the real sequence.
    total = [0.0] * n
    ops.paella_ops_time_launches(ev[0], ev[1])
    for _ in range(reps):
        for i in range(n):
            ex.launch_stage(i, stream)
            hip.llis_hip_stream_synchronize(stream)
            ms = ctypes.c_float()
            hip.llis_hip_event_elapsed_ms(ev[0], ev[1], ctypes.byref(ms))
            total[i] += ms.value
    ops.paella_ops_time_launches(None, None)
    per_stage = [t / reps * 1e3 for t in total]  # us
    # back-to-back forward without events: single-stream direct serving rate
    t0 = time.perf_counter()
    direct_n = 200
    for _ in range(direct_n):
        ex.forward(stream)
    hip.llis_hip_stream_synchronize(stream)
    direct_rps = direct_n / (time.perf_counter() - t0)
    for e in ev:
        hip.llis_hip_event_destroy(e)
    hip.llis_hip_stream_destroy(stream)
    ex.close()
    conv_flops = sum(w[1] for w in work if w[0] == "conv")
    conv_us = sum(t for t, w in zip(per_stage, work) if w[0] == "conv")
    conv_launches = sum(1 for w in work if w[0] == "conv")
    by_op = {}
    for t, w in zip(per_stage, work):
        d = by_op.setdefault(w[0], {"launches": 0, "us": 0.0, "flops": 0.0, "bytes": 0.0})
        d["launches"] += 1
        d["us"] += t
        d["flops"] += w[1]
        d["bytes"] += w[2]
    return {"per_stage_us": per_stage, "work": work, "conv_flops": conv_flops, "conv_us": conv_us, "conv_launches": conv_launches,
            "by_op": by_op, "direct_rps": direct_rps, "forward_us": sum(per_stage)}


def multi_queue_rate(models, model, nq=4, reps=200):
    """Forward passes per second with nq requests in flight and no scheduler in between: nq executors, each on its own
    ordered direct-dispatch queue, kernels without hooks.  The GPU-side ceiling of the served path.  Four queues is
    the best this device does: 1/2/3/4/5/6 queues gave 6.2/10.2/13.0/14.5/7.4/8.7 thousand ResNet-18 passes per second."""
    from paella_amd import ops
    execs = [models.Exec(model, seed=1) for _ in range(nq)]
    queues = [ops.DirectQueue(ordered=True) for _ in range(nq)]
    try:
        for e, q in zip(execs, queues):
            e.forward(q.handle)
        for q in queues:
            q.wait()
        t0 = time.perf_counter()
        for _ in range(reps):
            for e, q in zip(execs, queues):
                e.forward(q.handle)
        for q in queues:
            q.wait()
        return nq * reps / (time.perf_counter() - t0)
    finally:
        for q in queues:
            q.close()
        for e in execs:
            e.close()


def cpu_baseline(model, budget_s):
    from oracle import models as om
    from oracle import ops as orc
    from paella_amd import models
    desc = models.describe(model)
    x = om.make_input(desc, 1)
    om.run(desc, x, seed=1, fast=True)  # touch everything once
    n, t0 = 0, time.perf_counter()
    while True:
        om.run(desc, x, seed=1, fast=True)
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or n >= 64:
            break
    return {"value": n / dt, "unit": "requests/s", "cores": orc.num_threads(), "kind": "port",
            "sample": "%d %s forward passes (batch 1, fp32, same graph and seeded weights) with the float-accumulate CPU oracle, %.1f s" % (n, model, dt)}


def torch_cpu_baseline(model, budget_s):
    """The same graph and seeded weights through torch's CPU operators (oneDNN), all host threads: the stronger CPU
    figure, standing in for the reference's TVM-llvm target, which cannot exist offline."""
    import numpy as np
    import torch
    import torch.nn.functional as F
    from oracle import models as om
    from paella_amd import models
    d = models.describe(model)
    desc = om.Desc(d)
    W = {i: torch.from_numpy(desc.weight(i, 1)) for i in range(len(d["weights"]))}
    bufs = [torch.zeros(b["C"] * b["H"] * b["W"]) for b in d["buffers"]]

    def get(v):
        return None if v["buf"] < 0 else bufs[v["buf"]][v["off"]:v["off"] + v["C"] * v["H"] * v["W"]].view(1, v["C"], v["H"], v["W"])

    def act(y, n):
        a = n["act"]
        if a == 1:
            return F.relu(y)
        if a == 2:
            return torch.clamp(y, 0.0, 6.0)
        if a == 3:
            return F.prelu(y, W[n["slope"]])
        if a == 4:
            return torch.clamp(y, n["lo"], n["hi"])
        return y

    def forward(x):
        get(d["input"]).copy_(x)
        for n in d["nodes"]:
            xin, x2, op = get(n["x"]), get(n["x2"]), n["op"]
            if op == "conv":
                y = F.conv2d(xin, W[n["w"]], W[n["bias"]] if n["bias"] >= 0 else None, tuple(n["stride"]), tuple(n["pad"]), tuple(n["dil"]), n["groups"])
                y = act(y + x2 if x2 is not None else y, n)
            elif op == "dense":
                y = act(F.linear(xin.reshape(1, -1), W[n["w"]], W[n["bias"]]), n)
            elif op == "pool":
                if n["avg"]:
                    y = F.avg_pool2d(xin, tuple(n["k"]), tuple(n["stride"]), tuple(n["pad"]), bool(n["ceil"]), bool(n["count_include_pad"]))
                else:
                    y = F.max_pool2d(xin, tuple(n["k"]), tuple(n["stride"]), tuple(n["pad"]), 1, bool(n["ceil"]))
            elif op == "gap":
                y = xin.mean((2, 3), keepdim=True)
            elif op == "eltwise":
                y = xin
                if n["scale"] >= 0:
                    y = y * W[n["scale"]].view(1, -1, 1, 1)
                if n["shift"] >= 0:
                    y = y + W[n["shift"]].view(1, -1, 1, 1)
                y = act(y + x2 if x2 is not None else y, n)
            elif op == "softmax":
                y = F.softmax(xin.reshape(n["rows"], n["cols"]), 1)
            elif op == "lrn":
                y = F.local_response_norm(xin, n["size"], n["alpha"], n["beta"], n["k"])
            else:
                raise ValueError(op)
            get(n["y"]).copy_(y.reshape(get(n["y"]).shape))
        return get(d["output"]).reshape(-1).clone()

    x = torch.from_numpy(om.make_input(d, 1))
    with torch.no_grad():
        out = forward(x)
        ref = om.run(desc, x.numpy(), seed=1, fast=True)
        if not np.allclose(out.numpy(), ref, rtol=1e-2, atol=1e-3):
            return None  # not the same computation: do not report a time for it
        n, t0 = 0, time.perf_counter()
        while True:
            forward(x)
            n += 1
            dt = time.perf_counter() - t0
            if dt >= budget_s or n >= 2000:
                break
    return {"value": n / dt, "unit": "requests/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d %s forward passes (batch 1, fp32, same graph and seeded weights) through torch's CPU operators, %.1f s" % (n, model, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=400)
    ap.add_argument("--model", default="resnet18")
    ap.add_argument("--concurrency", type=int, default=32)
    ap.add_argument("--num-streams", type=int, default=64)
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--extra-kernels", type=int, default=16, help="full3: kernels admitted beyond the occupancy budget")
    ap.add_argument("--no-arms", action="store_true", help="skip the comparison arms and the Poisson sweep")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-mix", action="store_true", help="skip the small-CNN + Inception-v3 two-tenant arm")
    ap.add_argument("--mem-notify", choices=["marker", "hostfunc"], default="marker",
                    help="how the end of a copy stage reaches the scheduler in the timed arms: ring-marker kernel or host callback")
    ap.add_argument("--fairness-sweep", action="store_true",
                    help="also sweep full3's deficit threshold over a ResNet-18 : Inception-v3 = 0.952 : 0.048 mix and report Jain's index")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the plain copy kernel over a 64 MiB buffer five times (reference point for memory-traffic counters)")
    ap.add_argument("--zoo-ops", nargs="?", const="all", default=None, metavar="MODELS",
                    help="only this: per operator family of every zoo model (or of the comma-separated ones), launches, time and rates "
                         "of one forward pass, one launch at a time")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the isolated per-launch timing of one forward pass (the leg roofline.achieved comes from); value is null")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build serves from ONE GPU (one server process per GPU, no cross-GPU exchange); run with --gpus 1")
        sys.exit(2)

    from paella_amd import _abi, models, serve
    hip = _abi.hip()
    _abi.ops()
    serve.lib()
    if args.copy_calibration:
        import torch
        n = 16 << 20  # floats: 64 MiB read + 64 MiB written per launch
        x = torch.ones(n, dtype=torch.float32, device="cuda:0")
        y = torch.empty_like(x)
        torch.cuda.synchronize()
        for _ in range(5):
            _abi.check(_abi.ops().paella_copy_launch(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(y.data_ptr()), n, None, 0, None), "copy")
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"launches": 5, "kib_read_per_launch": n * 4 / 1024, "kib_written_per_launch": n * 4 / 1024}}), flush=True)
        return
    if args.zoo_ops:
        # Isolated launches, so every figure contains the 4 us an empty kernel shows by these time stamps: operators
        # that read 4.0 us are at that floor, whatever their kernels do.
        wanted = models.names() if args.zoo_ops == "all" else args.zoo_ops.split(",")
        table = {}
        for m in wanted:
            r = conv_roofline(models, hip, m, 20)
            log("[bench] %-17s %3d launches, forward pass %7.1f us, back to back %6.0f passes/s" % (m, len(r["per_stage_us"]), r["forward_us"], r["direct_rps"]))
            table[m] = {"launches": len(r["per_stage_us"]), "forward_us": r["forward_us"], "back_to_back_passes_per_s": r["direct_rps"], "by_op": {}}
            for op, d in sorted(r["by_op"].items(), key=lambda kv: -kv[1]["us"]):
                row = {"launches": d["launches"], "us": d["us"], "us_per_launch": d["us"] / d["launches"], "tflops": d["flops"] / d["us"] / 1e6,
                       "gbytes_per_s": d["bytes"] / d["us"] / 1e3, "frac_of_fp32_mfma_peak": d["flops"] / d["us"] / 1e6 / FP32_MFMA_PEAK_TFLOPS,
                       "frac_of_hbm_peak": d["bytes"] / d["us"] / 1e3 / 8000.0}
                table[m]["by_op"][op] = row
                log("[bench]     %-8s %3d launches %8.1f us (%5.2f each)  %6.2f TFLOP/s (%4.1f%% of fp32 MFMA)  %7.1f GB/s (%4.1f%% of HBM)" %
                    (op, row["launches"], row["us"], row["us_per_launch"], row["tflops"], 100 * row["frac_of_fp32_mfma_peak"],
                     row["gbytes_per_s"], 100 * row["frac_of_hbm_peak"]))
        print(json.dumps({"zoo_ops": table}), flush=True)
        return
    os.environ.setdefault("LLIS_MODEL_SEED", "1")
    job = serve.job_path("tvm_" + {"mobilenetv2": "mobilenet"}.get(args.model, args.model))
    jobs = [(job, 1.0, args.concurrency)]
    tot = models.totals(args.model)
    in_bytes = models.io_bytes(args.model)[0]
    in_shape = {602112: "1x3x224x224", 3136: "1x1x28x28", 1072812: "1x3x299x299", 921600: "1x3x240x320", 150528: "1x3x112x112"}.get(in_bytes, "%d input bytes" % in_bytes)

    # The isolated per-launch timing goes first: after a minute of serving arms the same launches measure about 4 %
    # longer (the part has been under sustained load by then).
    rl = conv_roofline(models, hip, args.model, reps=50)

    log("[bench] timed arm: full3, %d streams, concurrency %d, %d warm-up + %d timed requests" % (args.num_streams, args.concurrency, args.warmup, args.steps))
    # The timed arm and its comparison arms serve requests whose input already sits in device memory (the job
    # adapters skip their host-to-device stage); the same arm with the 602 KB copy per request is reported beside it.
    os.environ["PAELLA_INPUT_RESIDENT"] = "1"
    pcie_inclusive = None
    if args.roofline_only:
        args.no_arms = args.no_cpu = True
        main_run, value = None, None
    else:
        main_run = serve_arm(serve, "full3", args.num_streams, jobs, args.concurrency, args.steps, args.warmup, extra_kernels=args.extra_kernels,
                             mem_marker=args.mem_notify == "marker")
        value = main_run["throughput_rps"]
        log("[bench]   %.1f req/s" % value)
        os.environ["PAELLA_INPUT_RESIDENT"] = "0"
        r = serve_arm(serve, "full3", args.num_streams, jobs, args.concurrency, max(500, args.steps // 2), args.warmup // 2, extra_kernels=args.extra_kernels,
                      mem_marker=args.mem_notify == "marker")
        pcie_inclusive = r["throughput_rps"]
        log("[bench]   %.1f req/s with the host-to-device copy of every request's input" % pcie_inclusive)
        os.environ["PAELLA_INPUT_RESIDENT"] = "1"

    arms, sweep, lognormal_point = {}, [], None
    if not args.no_arms:
        n_arm = max(500, args.steps // 2)
        for label, sched, streams in [("fifo_multi_stream", "fifo", args.concurrency), ("fifo2_kernel_by_kernel", "fifo2", args.num_streams),
                                      ("fifo_single_stream", "fifo", 1)]:
            r = serve_arm(serve, sched, streams, jobs, args.concurrency, n_arm, args.warmup // 2)
            arms[label] = {"requests_per_s": r["throughput_rps"], "p50_us": r["all"]["p50"], "p99_us": r["all"]["p99"], "streams": streams}
            log("[bench]   arm %-24s %.1f req/s, p99 %.0f us" % (label, r["throughput_rps"], r["all"]["p99"]))
        single = serve_arm(serve, "full3", args.num_streams, [(job, 1.0, 1)], 1, 300, 50, extra_kernels=args.extra_kernels)
        arms["full3_one_outstanding"] = {"requests_per_s": single["throughput_rps"], "p50_us": single["all"]["p50"], "p99_us": single["all"]["p99"]}
        # open-loop Poisson arrivals at fractions of the saturation rate, full3 vs multi-stream fifo
        for frac in (0.5, 0.8, 0.95):
            rate = frac * min(value, arms["fifo_multi_stream"]["requests_per_s"])
            point = {"offered_rps": rate}
            for label, sched, streams in [("full3", "full3", args.num_streams), ("fifo_multi_stream", "fifo", args.concurrency)]:
                r = serve_arm(serve, sched, streams, jobs, args.concurrency, n_arm, args.warmup // 2, iat_us=1e6 / rate, extra_kernels=args.extra_kernels)
                point[label] = {"achieved_rps": r["throughput_rps"], "p50_us": r["all"]["p50"], "p99_us": r["all"]["p99"]}
            sweep.append(point)
            log("[bench]   poisson %.0f req/s: full3 p99 %.0f us, fifo p99 %.0f us" % (rate, point["full3"]["p99_us"], point["fifo_multi_stream"]["p99_us"]))
        # The reference client's default arrival process is log-normal (reference app/client.cpp:133-134, sigma 1.5 or 2): one
        # point of it at half the saturation rate -- the same mean rate as the first Poisson point, in bursts.
        rate = 0.5 * min(value, arms["fifo_multi_stream"]["requests_per_s"])
        point = {"offered_rps": rate, "arrivals": "log-normal, sigma 1.5"}
        for label, sched, streams in [("full3", "full3", args.num_streams), ("fifo_multi_stream", "fifo", args.concurrency)]:
            r = serve_arm(serve, sched, streams, jobs, args.concurrency, n_arm, args.warmup // 2, iat_us=1e6 / rate, extra_kernels=args.extra_kernels,
                          dist="ln", ln_sigma=1.5)
            point[label] = {"achieved_rps": r["throughput_rps"], "p50_us": r["all"]["p50"], "p99_us": r["all"]["p99"]}
        lognormal_point = point
        log("[bench]   log-normal arrivals, %.0f req/s: full3 p50 / p99 %.0f / %.0f us, fifo %.0f / %.0f us" %
            (rate, point["full3"]["p50_us"], point["full3"]["p99_us"], point["fifo_multi_stream"]["p50_us"], point["fifo_multi_stream"]["p99_us"]))

    # The two-tenant mix of the target statement: small CNN : Inception-v3 (299x299) = 9 : 1, full3 against plain
    # multi-stream serving (fifo), first at saturation, then open-loop Poisson at fractions of the lower of the two.
    def mix_arm(workload, tenants, fracs, n_mix=3000):
        """tenants: (label, job adapter, share).  Saturation, then open-loop Poisson at fractions of the lower saturation rate."""
        mix_jobs = [(serve.job_path(adapter), share, args.concurrency) for _, adapter, share in tenants]
        arms2 = [("full3", "full3", args.num_streams), ("fifo_multi_stream", "fifo", args.concurrency)]
        sat = {}
        for label, sched, streams in arms2:
            r = serve_arm(serve, sched, streams, mix_jobs, args.concurrency, n_mix, 300, extra_kernels=args.extra_kernels)
            sat[label] = r["throughput_rps"]
        res = {"workload": workload, "saturation_rps": sat, "poisson": []}
        log("[bench]   %s, saturation: full3 %.0f req/s, fifo %.0f req/s" % (workload, sat["full3"], sat["fifo_multi_stream"]))
        for frac in fracs:
            rate = frac * min(sat.values())
            point = {"offered_rps": rate}
            for label, sched, streams in arms2:
                r = serve_arm(serve, sched, streams, mix_jobs, args.concurrency, n_mix, 300, iat_us=1e6 / rate, extra_kernels=args.extra_kernels)
                point[label] = {"achieved_rps": r["throughput_rps"], "p50_us": r["all"]["p50"], "p99_us": r["all"]["p99"]}
                for k, (tenant, _, _) in enumerate(tenants):
                    point[label][tenant + "_p99_us"] = r["per_type"][k]["p99"]
            res["poisson"].append(point)
            log("[bench]   %s, poisson %.0f req/s: p99 full3 %.0f us, fifo %.0f us; per tenant full3 %s | fifo %s" %
                (workload, rate, point["full3"]["p99_us"], point["fifo_multi_stream"]["p99_us"],
                 " ".join("%.0f" % point["full3"][t + "_p99_us"] for t, _, _ in tenants),
                 " ".join("%.0f" % point["fifo_multi_stream"][t + "_p99_us"] for t, _, _ in tenants)))
        return res

    # The two-tenant mix of the target statement: small CNN : Inception-v3 (299x299) = 9 : 1, full3 against plain
    # multi-stream serving (fifo), first at saturation, then open-loop Poisson at fractions of the lower of the two.
    # Then the other two mixes of the benchmark configurations, the same way at one load point.
    mix, other_mixes = None, []
    if not args.no_arms and not args.no_mix:
        mix = mix_arm("small CNN : Inception-v3 = 9 : 1, inputs resident",
                      [("small_cnn", "tvm_mnist", 0.9), ("inception_v3", "tvm_inception_v3", 0.1)], (0.5, 0.8))
        other_mixes.append(mix_arm("MobileNetV2 : ResNet-50 = 1 : 1, inputs resident",
                                   [("mobilenetv2", "tvm_mobilenet", 0.5), ("resnet50", "tvm_resnet50", 0.5)], (0.8,)))
        eight = ["densenet121", "googlenet", "squeezenet1_1", "resnet34", "ultraface320", "arcfaceresnet100", "mobilenet", "mnist"]
        other_mixes.append(mix_arm("eight models, uniform choice, inputs resident",
                                   [(m, "tvm_" + m, 0.125) for m in eight], (0.8,), n_mix=2000))

    # One client, one request at a time, small CNN, 10 000 requests, input and output crossing PCIe: the latency
    # floor of the full path (its 5 kernels are small enough to be issued as one scheduler stage).
    closed_loop = None
    if not args.no_arms:
        import numpy as np
        os.environ["PAELLA_INPUT_RESIDENT"] = "0"
        name = "bench%d_closed_%d" % (os.getpid(), int(time.time() * 1000) % 100000)
        x = np.random.default_rng(1).random((1, 1, 28, 28), dtype=np.float32)
        with serve.Server(name, "full3", num_streams=args.num_streams, cpu=4, extra_kernels=args.extra_kernels) as srv:
            serve.client_single(srv.name, serve.job_path("tvm_mnist"), x, 10, n=500)
            _, lat = serve.client_single(srv.name, serve.job_path("tvm_mnist"), x, 10, n=10000)
        os.environ["PAELLA_INPUT_RESIDENT"] = "1"
        lat = np.sort(lat)
        probe = models.Exec("mnist", seed=1)
        kernels = probe.num_stages
        one_piece = all(probe.stage_dims(i).grid * probe.stage_dims(i).block <= 65536 for i in range(kernels))
        probe.close()
        stages = 1 if one_piece else kernels
        closed_loop = {"workload": "small CNN 1x1x28x28, one client, one request outstanding, 10000 requests, input and output crossing PCIe "
                                   "inside the first and last kernel (tensors under 64 KiB have no copy stage)",
                       "kernels_per_request": kernels, "stages_per_request": stages,
                       "mean_us": float(lat.mean()), "p50_us": float(lat[len(lat) // 2]), "p99_us": float(lat[int(len(lat) * 0.99)])}
        log("[bench]   small CNN closed loop: mean %.1f us, p50 %.1f us, p99 %.1f us per request (%d kernels in %d scheduler stage%s)" %
            (closed_loop["mean_us"], closed_loop["p50_us"], closed_loop["p99_us"], kernels, stages, "" if stages == 1 else "s"))

    # Deficit-threshold sweep over a two-model mix at saturation: latency of each model in the mix over its
    # latency when served alone, and Jain's index over those slowdowns.
    fairness_sweep = None
    if args.fairness_sweep:
        from paella_amd import fairness
        fjobs = [(serve.job_path("tvm_resnet18"), 0.952, 119), (serve.job_path("tvm_inception_v3"), 0.048, 6)]
        alone = []
        for path, prop, cap in fjobs:
            r = serve_arm(serve, "full3", args.num_streams, [(path, 1.0, cap)], cap, int(3000 * prop) + 1, 200, extra_kernels=args.extra_kernels)
            alone.append(r["all"]["mean"])
        fairness_sweep = {"workload": "ResNet-18 : Inception-v3 = 0.952 : 0.048, 119 + 6 outstanding, 3000 requests at saturation",
                          "alone_mean_latency_us": alone, "points": []}
        for f in (0.01, 1.0, 10.0, 50.0, 100.0, 500.0, 1000.0, 100000.0):
            r = serve_arm(serve, "full3", args.num_streams, fjobs, 125, 3000, 300, extra_kernels=args.extra_kernels, unfair=f)
            slow = [r["per_type"][i]["mean"] / alone[i] for i in range(2)]
            fairness_sweep["points"].append({"unfair": f, "requests_per_s": r["throughput_rps"], "slowdown": slow, "jain_index": float(fairness.jain_index(slow))})
            log("[bench]   unfair %-9g %.0f req/s, slowdown ResNet-18 %.2f, Inception-v3 %.2f, Jain index %.3f" %
                (f, r["throughput_rps"], slow[0], slow[1], fairness_sweep["points"][-1]["jain_index"]))

    log("[bench] per-launch timing of the forward pass (kernel begin/end timestamps through HIP events), taken before the serving arms")
    achieved = rl["conv_flops"] / (rl["conv_us"] * 1e-6) / 1e12
    roofline = {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
                "traffic": CONV_TRAFFIC_BYTES_PER_LAUNCH.get(args.model), "kernel": "conv_mfma_kernel and conv_mfma_group_kernel (all %d conv launches of one %s forward pass)" % (rl["conv_launches"], args.model),
                "flops_per_launch_avg": rl["conv_flops"] / rl["conv_launches"], "us_per_launch_avg": rl["conv_us"] / rl["conv_launches"]}
    log("[bench]   conv: %.2f TFLOP/s (%.1f%% of fp32 MFMA peak), forward %.0f us, direct loop %.0f req/s" %
        (achieved, 100 * roofline["frac"], rl["forward_us"], rl["direct_rps"]))
    for op, v in rl["by_op"].items():
        log("[bench]     %-8s %3d launches %8.1f us  %7.3f GFLOP %8.2f MB  -> %6.2f TFLOP/s %7.1f GB/s" %
            (op, v["launches"], v["us"], v["flops"] / 1e9, v["bytes"] / 1e6, v["flops"] / (v["us"] * 1e-6) / 1e12, v["bytes"] / (v["us"] * 1e-6) / 1e9))

    try:
        # Not under --roofline-only: that leg is the one run under the profiler's counter collection, which
        # intercepts queues it created itself and does not survive packets on queues owned by this library.
        if args.roofline_only:
            raise RuntimeError("skipped with --roofline-only")
        mq = multi_queue_rate(models, args.model)
        roofline["under_load"] = {"forward_passes_per_s": mq, "conv_tflops": mq * rl["conv_flops"] / 1e12,
                                  "frac": mq * rl["conv_flops"] / 1e12 / FP32_MFMA_PEAK_TFLOPS,
                                  "how": "4 forward passes in flight on 4 ordered direct-dispatch queues, no hooks, no scheduler"}
        log("[bench]   4 forward passes in flight (direct queues, no scheduler): %.0f passes/s = %.1f TFLOP/s of conv work (%.1f%% of peak)" %
            (mq, mq * rl["conv_flops"] / 1e12, 100 * mq * rl["conv_flops"] / 1e12 / FP32_MFMA_PEAK_TFLOPS))
    except RuntimeError as ex:
        log("[bench]   direct-dispatch queues unavailable: %s" % ex)
    lib = _abi.ops()
    peak = ctypes.c_double()
    if lib.paella_mfma_peak_probe(ctypes.byref(peak)) == 0:
        roofline["peak_measured"] = peak.value  # register-resident fp32 MFMA loop on this box; `peak` stays the published figure
        log("[bench]   fp32 MFMA rate measured with a register-resident loop: %.1f TFLOP/s" % peak.value)
    floor = ctypes.c_double()
    if lib.paella_empty_kernel_probe(200, ctypes.byref(floor)) == 0 and floor.value > 0:
        # what the same time stamps report for a kernel that does nothing (the profiler's kernel trace gives 1.4 us for
        # it): every per-launch figure taken this way contains it, so measured like this the 20 conv launches of a pass
        # cannot show more than flops / (20 x floor) however fast the kernels are
        bound = rl["conv_flops"] / (rl["conv_launches"] * floor.value * 1e-6) / 1e12
        roofline["empty_kernel_us"] = floor.value
        roofline["launch_bound_tflops"] = bound
        roofline["frac_of_launch_bound"] = achieved / bound
        log("[bench]   an empty kernel is %.2f us long by the same time stamps: ceiling of this measurement %.1f TFLOP/s, conv at %.0f%% of it" %
            (floor.value, bound, 100 * achieved / bound))
    ring = ctypes.c_void_p()
    notify = {}
    if not args.roofline_only and lib.paella_ring_create(1024000, 1, ctypes.byref(ring)) == 0:
        us = ctypes.c_double()
        if lib.paella_ring_bench_drain(ring, 64, 6400, 50, 500, ctypes.byref(us)) == 0:
            notify["ring_drain_64_blocks_us_per_kernel"] = us.value
        flag, sync = ctypes.c_double(), ctypes.c_double()
        if lib.paella_ring_bench_pingpong(100, 2000, ctypes.byref(flag), ctypes.byref(sync), None) == 0:
            notify["launch_plus_flag_store_us"] = flag.value
            notify["launch_plus_stream_sync_us"] = sync.value
        # resident lane answering host pings through the ring: no launch in the way
        import numpy as np
        n_echo = 5000
        rtt, one_way = np.zeros(n_echo), np.zeros(n_echo)
        if lib.paella_ring_bench_echo(ring, 500, n_echo, rtt.ctypes.data, one_way.ctypes.data) == 0:
            rtt.sort()
            notify["echo_round_trip_us"] = {"p50": float(rtt[n_echo // 2]), "p99": float(rtt[int(n_echo * 0.99)]),
                                            "what": "host flag store -> resident lane sees it -> ring message readable on the host"}
            ow = np.sort(one_way[one_way > -1e29])
            if len(ow):
                # The translation interpolates between clock pairs the runtime samples itself and is good to a
                # microsecond or two: a figure outside (0, round trip) says so.  The round trip is the hard bound.
                notify["device_to_host_us_clock_translated"] = {
                    "p50": float(ow[len(ow) // 2]), "p99": float(ow[int(len(ow) * 0.99)]),
                    "inside_round_trip": bool(0.0 < ow[len(ow) // 2] < rtt[n_echo // 2]),
                    "what": "host clock when the message became readable minus the lane's realtime counter just before the ring write, "
                            "translated to the host clock by the runtime"}
            log("[bench]   notification: echo round trip p50 %.2f / p99 %.2f us%s" % (rtt[n_echo // 2], rtt[int(n_echo * 0.99)],
                "" if not len(ow) else (", device->host p50 %.2f / p99 %.2f us" % (ow[len(ow) // 2], ow[int(len(ow) * 0.99)])) +
                ("" if 0.0 < ow[len(ow) // 2] < rtt[n_echo // 2] else " (outside the round trip: the runtime's clock translation is off by more than that here)")))
        lib.paella_ring_destroy(ring)

    cpu = None if args.no_cpu else cpu_baseline(args.model, args.cpu_seconds)
    cpu_torch = None
    if not args.no_cpu:
        try:
            cpu_torch = torch_cpu_baseline(args.model, min(args.cpu_seconds, 8.0))
        except Exception as ex:  # torch missing or an operator it lacks: the oracle figure stands alone
            log("[bench]   torch CPU baseline unavailable: %s" % ex)
        if cpu and cpu_torch:
            log("[bench]   CPU: oracle %.2f req/s on %d threads, torch CPU operators %.1f req/s on %d threads" %
                (cpu["value"], cpu["cores"], cpu_torch["value"], cpu_torch["cores"]))

    out = {
        "metric": METRIC,
        "value": value,
        "unit": "requests/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_run["elapsed_us"] / 1e3 / args.steps if main_run else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s batch 1 fp32 %s, seeded weights, inputs resident in device memory, full3 scheduler, %d streams, "
                               "saturation with %d outstanding requests" % (args.model, in_shape, args.num_streams, args.concurrency),
                   # kernels only: the input is resident and an output of at most 64 KiB is written to host memory by the last kernel
                   "gmac_per_request": tot["macs"] / 1e9, "operators_per_request": tot["stages"],
                   "stages_per_request": (len(rl["per_stage_us"]) if rl else tot["stages"]) + (0 if models.io_bytes(args.model)[1] <= 65536 else 1)},
        "pcie_inclusive_requests_per_s": pcie_inclusive,
        # open-loop latency at 80 % of the saturation rate; at saturation every request is submitted at t = 0 and
        # its latency is its position in the queue, so no latency is quoted for the timed arm itself
        "latency_us": ({"offered_rps": sweep[1]["offered_rps"], "p50": sweep[1]["full3"]["p50_us"], "p99": sweep[1]["full3"]["p99_us"]}
                       if len(sweep) > 1 else None),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_baseline_torch": cpu_torch,
        "arms": arms,
        "poisson_sweep": sweep,
        "lognormal_point": lognormal_point,
        "two_tenant_mix": mix,
        "other_mixes": other_mixes,
        "small_cnn_closed_loop": closed_loop,
        "fairness_sweep": fairness_sweep,
        "direct_single_stream_rps": rl["direct_rps"],
        # per operator family, one forward pass, isolated launches: time, algorithmic work, and the rates they imply
        "per_op_us": {k: {"launches": v["launches"], "us": v["us"], "gflop": v["flops"] / 1e9, "mbytes": v["bytes"] / 1e6,
                          "tflops": v["flops"] / (v["us"] * 1e-6) / 1e12 if v["us"] else None,
                          "gbytes_per_s": v["bytes"] / (v["us"] * 1e-6) / 1e9 if v["us"] else None} for k, v in rl["by_op"].items()},
        "notify_us": notify,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
