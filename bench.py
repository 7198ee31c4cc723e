#!/usr/bin/env python3
"""Benchmark of the MI355X backend on the reference's headline workloads.

Default workload (N=1): the standalone fp32 matmul through the array API, M=N=K=8192, with the fused
per-element epilogue bias + leaky_relu(0.01); one step = one run of that graph with A, B and bias already
resident in HBM.  Prints ONE JSON line; `--all` adds the other matmul shapes and the ConvNet (batch 1000)
train-step rate under "extra".

No torch: device memory, the stream and event timing all go through libdescent_hip.so.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
# HBM bytes one launch of the headline kernel moves, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same
# command, each counter scaled by what it reads for the streaming kernel of known size (--copy-calibration); the
# summary is profiles/matmul_mfma_8192.txt.  Only the 8192^3 workload has been counted.
MEASURED_TRAFFIC_BYTES = {8192: 3.705e9}


def time_graph(env, graph, steps: int, warmup: int, seed0: int = 1, profile: bool = True):
    """W untimed runs, then K timed runs bracketed by stream syncs; returns the wall seconds of the K runs.
    With `profile` every launch of the timed region is bracketed by HIP events on the context's stream (per-kernel
    durations for dsc_prof_query / the report).  The events cost a few microseconds per launch, so schedules
    made of many small kernels are timed with profile=False and profiled in a second, untimed pass."""
    be = env.backend
    for i in range(warmup):
        env.run(graph, seed0 + i)
    be.sync()
    be.profile_reset()
    be.profile(profile)
    t0 = time.perf_counter()
    for i in range(steps):
        env.run(graph, seed0 + warmup + i)
    be.sync()
    wall = time.perf_counter() - t0
    be.profile(False)
    return wall


EVENT_PASS = True  # --no-events: skip the second, per-launch-event pass (for runs under an external profiler)


def time_then_profile(env, graph, steps: int, warmup: int):
    wall = time_graph(env, graph, steps, warmup, profile=False)
    if EVENT_PASS:
        time_graph(env, graph, steps, 0, seed0=1000, profile=True)
    return wall


def verify_matmul_rows(env, w, count=64):
    """`count` sampled rows of the product the timed launches left in C, against a float64 product of the operands
    read back from the device: relative L2 error over those rows (the tolerance of the benchmark definition is 1e-4)."""
    be = env.backend
    rows = np.sort(np.random.default_rng(0).choice(w.m, min(count, w.m), replace=False))
    b = np.frombuffer(be.read(w.b.buffer, 0, 4 * w.k * w.n), np.float32).reshape(w.k, w.n).astype(np.float64)
    bias = np.frombuffer(be.read(w.bias.buffer, 0, 4 * w.n), np.float32).astype(np.float64)
    a = np.stack([np.frombuffer(be.read(w.a.buffer, 4 * w.k * int(r), 4 * w.k), np.float32) for r in rows]).astype(np.float64)
    got = np.stack([np.frombuffer(be.read(w.c.buffer, 4 * w.n * int(r), 4 * w.n), np.float32) for r in rows]).astype(np.float64)
    z = a @ b + bias
    want = np.where(z > 0, z, 0.01 * z)
    return float(np.linalg.norm(got - want) / np.linalg.norm(want))


def bench_matmul(env, m, n, k, steps, warmup, verify=False):
    from descent_amd import workloads

    w = workloads.matmul_epilogue(env, m, n, k, seed=2)
    wall = time_graph(env, w.graph, steps, warmup)
    avg_us, launches = env.backend.timing_query("MatMul")
    all_us, _, _, all_n = env.backend.timing_work("")  # every launch of the step (a re-split product has two)
    report = env.backend.timing_report(0)
    env.backend.profile_reset()
    rel_err = verify_matmul_rows(env, w) if verify else None
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    for p in (w.a, w.b, w.bias, w.c):
        if p.buffer is not None:
            env.backend.free(p.buffer)
            p.buffer = None
    return {
        "shape": [m, n, k],
        "flops": w.flops,
        "wall_s": wall,
        "ms_per_step": 1e3 * wall / steps,
        "tflops_wall": w.flops * steps / wall / 1e12,
        "kernel_avg_us": avg_us,
        "kernel_us_per_step": all_us / steps if all_n else None,
        "kernel_launches": launches,
        "tflops_kernel": (w.flops / (avg_us * 1e-6) / 1e12) if avg_us else None,
        "launches_per_step": sched.launch_count()[0],
        "report": report,
        "rel_l2_error_sampled_rows": rel_err,
    }


KERNEL_CLASSES = ("MatMul", "ConvDataGrad", "ConvBackward", "ConvForward", "PerElement", "Reduce", "RowFused", "WindowsToImage", "Unpad", "ScatterAdd",
                  "Multi (4 kernels: ScatterAdd", "Multi", "Fill")


def class_rooflines(be, steps):
    """Per kernel class (label prefix) of the launches profiled since the last reset: time per step, and the
    algorithmic bytes / flops those launches stand for as GB/s against the HBM peak and TFLOP/s against the fp32
    MFMA peak.  A "Multi" launch is several small kernels sharing one launch."""
    out = {}
    for prefix in KERNEL_CLASSES:
        us, nbytes, flops, n = be.timing_work(prefix)
        if not n:
            continue
        row = {"us_per_step": us / steps, "launches_per_step": n / steps, "gbs": nbytes / (us * 1e-6) / 1e9,
               "frac_hbm": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        if flops:
            row["tflops"] = flops / (us * 1e-6) / 1e12
            row["frac_mfma"] = row["tflops"] / MFMA_FP32_PEAK_TFLOPS
        out[prefix] = row
    return out


def bench_convnet(env, steps, warmup, batch=1000, repeats=5, blur_pool=False, min_warmup=1000):
    """ConvNet train steps per second: `repeats` timed regions of `steps` steps each (no per-launch events), the
    median reported with the spread beside it; then one more pass with events for the per-kernel table."""
    import re

    from descent_amd import workloads

    w = workloads.convnet(env, batch=batch, seed=3, blur_pool=blur_pool)
    # (the warm-up is long enough for the device to reach the clock it holds under this load: the first region of a run
    # that starts from idle reads 1.5 % low)
    walls = [time_graph(env, w.graph, steps, max(warmup, min_warmup) if r == 0 else 0, seed0=1 + r * steps, profile=False) for r in range(repeats)]
    wall = sorted(walls)[len(walls) // 2]
    if EVENT_PASS:
        time_graph(env, w.graph, min(steps, 50), 0, seed0=100000, profile=True)
    report = env.backend.timing_report(int(os.environ.get("DSC_BENCH_TOPN", "12")))
    classes = class_rooflines(env.backend, min(steps, 50)) if EVENT_PASS else {}
    env.backend.profile_reset()
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    listing = sched.describe()
    work = listing.strip().splitlines()[-1]
    m = re.search(r"([0-9.]+) MB moved, ([0-9.]+) GFLOP", work)
    nbytes, flops = (float(m.group(1)) * 1e6, float(m.group(2)) * 1e9) if m else (None, None)
    out = {
        "steps_per_s": steps / wall,
        "ms_per_step": 1e3 * wall / steps,
        "steps_per_s_min_max": [steps / max(walls), steps / min(walls)],
        "timed": "%d regions of %d steps, median" % (repeats, steps),
        "launches_per_step": sched.launch_count()[0],
        "clusters": sched.launch_count()[1],
        "algorithmic_work_per_step": work.lstrip("# "),
        "kernel_classes": classes,
        "report": report,
    }
    if nbytes:
        # the whole step against both roofs: its algorithmic bytes at 8 TB/s, its MatMul flops at the fp32 MFMA peak
        out["roofline"] = {
            "bound": "hbm", "achieved": nbytes / (wall / steps) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": nbytes / (wall / steps) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes_per_step": nbytes,
            "matmul_tflops": flops / (wall / steps) / 1e12, "frac_mfma": flops / (wall / steps) / 1e12 / MFMA_FP32_PEAK_TFLOPS,
        }
    return out


def bench_convnet_minibatch_uploads(env, steps=300, batch=1000):
    """ConvNet train steps with a new mini-batch (x: batch x 28 x 28 floats, y: batch labels) uploaded before every
    step, as a training loop does: through the compute stream (the reference's writer contract), and through the
    copy stream from alternating pinned arrays, where the upload of step n+1 runs beside step n."""
    from descent_amd import workloads

    be = env.backend
    w = workloads.convnet(env, batch=batch, seed=3)
    x, y = w.inputs["x"], w.inputs["y"]
    px = [env.host_array(x) for _ in range(2)]
    py = [env.host_array(y) for _ in range(2)]
    rng = np.random.default_rng(0)
    for a in px:
        a[...] = rng.random(a.shape, dtype=np.float32)
    for a in py:
        a[...] = rng.integers(0, 10, a.shape).astype(np.float32)

    def loop(n, mode):
        for i in range(n):
            s = i & 1
            if mode == "serial":
                env.write_parameter(x, px[s])
                env.write_parameter(y, py[s])
            elif mode == "overlapped":
                env.write_parameter_async(x, px[s])
                env.write_parameter_async(y, py[s])
            env.run(w.graph, i)
        be.sync()

    out = {"upload_bytes_per_step": int(px[0].nbytes + py[0].nbytes)}
    for mode in ("resident", "serial", "overlapped"):
        loop(20, mode)
        t0 = time.perf_counter()
        loop(steps, mode)
        out[mode + "_steps_per_s"] = steps / (time.perf_counter() - t0)
    for a in px + py:
        be.host_release(a)
    return out


def bench_elementwise(env, n, steps, warmup):
    """c = a * 2 + b over n elements: 2 reads + 1 write of 4n bytes each (a plain streaming kernel of known
    size, also used to calibrate the FETCH_SIZE / WRITE_SIZE counters)."""
    rng = np.random.Generator(np.random.PCG64(9))
    a = env.static_parameter([n], "a")
    b = env.static_parameter([n], "b")
    c = env.static_parameter([n], "c")
    env.write_parameter(a, rng.random(n, dtype=np.float32))
    env.write_parameter(b, rng.random(n, dtype=np.float32))
    graph = env.build_graph(lambda s: s.write_parameter_value(c, s.parameter_value(a) * 2.0 + s.parameter_value(b)))
    wall = time_graph(env, graph, steps, warmup)
    avg_us, launches = env.backend.timing_query("PerElement")
    env.backend.profile_reset()
    for p in (a, b, c):
        env.backend.free(p.buffer)
        p.buffer = None
    nbytes = 12.0 * n
    return {"elements": n, "bytes": nbytes, "kernel_avg_us": avg_us, "gbs_kernel": nbytes / (avg_us * 1e-6) / 1e9,
            "gbs_wall": nbytes * steps / wall / 1e9, "frac_hbm": nbytes / (avg_us * 1e-6) / 1e9 / HBM_PEAK_GBS}


def bench_workload(env, build, steps, warmup, topn=8, read_loss=False):
    """Step rate of one of the image-fit configurations, with the per-kernel table."""
    w = build(env)
    wall = time_then_profile(env, w.graph, steps, warmup)
    be = env.backend
    out = {"steps_per_s": steps / wall, "ms_per_step": 1e3 * wall / steps}
    if read_loss:
        out["loss_finite"] = bool(all(np.all(np.isfinite(env.read_parameter(p))) for p in w.scalars.values()))
    out["kernel_classes"] = class_rooflines(be, steps) if EVENT_PASS else {}
    report = be.timing_report(topn)
    be.profile_reset()
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    out["launches_per_step"], out["clusters"] = sched.launch_count()
    for p in list(w.inputs.values()) + w.trainable + w.state + list(w.scalars.values()):
        if p.buffer is not None:
            be.free(p.buffer)
            p.buffer = None
    return out, report


def bench_reduce(env, rows, cols, axis, steps, warmup):
    """Sum of a [rows, cols] array along one axis: 4*(rows*cols + outputs) bytes."""
    rng = np.random.Generator(np.random.PCG64(10))
    a = env.static_parameter([rows, cols], "a")
    out_shape = [rows, 1] if axis == 1 else [1, cols]
    o = env.static_parameter(out_shape, "o")
    env.write_parameter(a, rng.random(rows * cols, dtype=np.float32))
    graph = env.build_graph(lambda s: s.write_parameter_value(o, s.parameter_value(a).reduce_sum(axis, True)))
    wall = time_graph(env, graph, steps, warmup)
    avg_us, launches = env.backend.timing_query("Reduce")
    per_step_us = avg_us * launches / steps
    env.backend.profile_reset()
    for p in (a, o):
        env.backend.free(p.buffer)
        p.buffer = None
    nbytes = 4.0 * (rows * cols + (rows if axis == 1 else cols))
    return {"shape": [rows, cols], "axis": axis, "kernels_us_per_step": per_step_us, "launches_per_step": launches / steps,
            "gbs": nbytes / (per_step_us * 1e-6) / 1e9, "frac_hbm": nbytes / (per_step_us * 1e-6) / 1e9 / HBM_PEAK_GBS}


def bench_upload(env, n):
    """Host -> device through the library's pinned staging ring (dsc_buf_write), and the headline product with the
    upload of A and B inside the timed region (the rate a caller sees when its operands start in host memory)."""
    from descent_amd import workloads

    be = env.backend
    w = workloads.matmul_epilogue(env, n, n, n, seed=2)
    env.run(w.graph, 0)
    be.sync()
    rng = np.random.Generator(np.random.PCG64(4))
    a = rng.standard_normal(n * n, dtype=np.float32)
    b = rng.standard_normal(n * n, dtype=np.float32)
    reps = 3
    t0 = time.perf_counter()
    for i in range(reps):
        be.write(w.a.buffer, 0, a)
        be.write(w.b.buffer, 0, b)
        env.run(w.graph, i)
    be.sync()
    dt = (time.perf_counter() - t0) / reps
    t0 = time.perf_counter()
    be.write(w.a.buffer, 0, a)
    be.sync()
    up = time.perf_counter() - t0
    for p in (w.a, w.b, w.bias, w.c):
        if p.buffer is not None:
            be.free(p.buffer)
            p.buffer = None
    return {"upload_gbs": a.nbytes / up / 1e9, "matmul_with_upload_tflops": w.flops / dt / 1e12, "ms_per_step_with_upload": dt * 1e3}


# the cfg2 shapes beside the headline, each with the warm-up and the number of timed launches that put about a quarter of
# a second of the same work before and inside the timed region
CFG2_OTHER_SHAPES = (((1024, 1024, 1024), 4000, 6000), ((4096, 4096, 4096), 150, 250), ((1000, 128, 784), 4000, 6000), ((262144, 256, 256), 600, 900))


def _compact_classes(classes):
    """Kernel classes of a step, compact: microseconds per step, launches, and the fraction of the roof each class's
    algorithmic work reaches (HBM always; fp32 MFMA where the class multiplies matrices)."""
    out = {}
    for name, row in classes.items():
        c = {"us": round(row["us_per_step"], 1), "launches": round(row["launches_per_step"], 2), "frac_hbm": round(row["frac_hbm"], 3)}
        if "frac_mfma" in row:
            c["frac_mfma"] = round(row["frac_mfma"], 3)
        out[name.split(" (")[0] if name.startswith("Multi (") else name] = c
    return out


def bench_configs(env):
    """The configurations the headline does not cover, compact enough for the one JSON line: the other four
    standalone matmul shapes (each verified on sampled rows against float64 after its timed region), the linear
    classifier, the ConvBlurNet, both coordinate MLPs and the hash-grid fit (step rate, launches, per-class roofline fractions,
    and the summed loss of the timed steps, which must be finite).

    Every timed region follows a warm-up of the same launches that lasts a quarter of a second or so, and lasts about
    as long itself: the device raises its clock over the first milliseconds of a burst of work, and a launch of tens or
    hundreds of microseconds timed twenty times from idle is measured on the ramp (262144x256x256: 345 us per launch
    over 20 launches from idle, 288 over 200, 275 over 3000; 4096^3 1099 us over 10, 977 over 300; the 8192^3 headline
    takes 7.6 ms per launch and reads the same over 5 launches and over 100)."""
    from descent_amd import workloads as _w

    out = {"matmul": {}}
    for (m, n, k), warmup, steps in CFG2_OTHER_SHAPES:
        r = bench_matmul(env, m, n, k, steps, warmup, verify=True)
        ok = r["rel_l2_error_sampled_rows"] <= 1e-4
        # a product of one launch: rate of that launch; of several (k re-split + the sum of its partials): of all of them
        us = r["kernel_us_per_step"]
        out["matmul"]["%dx%dx%d" % (m, n, k)] = {
            "tflops_kernels": round(r["flops"] / (us * 1e-6) / 1e12, 2), "frac_mfma": round(r["flops"] / (us * 1e-6) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 3),
            "kernels_us": round(us, 2), "tflops_wall": round(r["tflops_wall"], 2), "launches": r["launches_per_step"], "steps": steps, "warmup": warmup,
            "rel_l2_error_sampled_rows": r["rel_l2_error_sampled_rows"], "verified": bool(ok)}
    # (the ConvBlurNet is the reference example's other convolutional network -- strided depthwise blurs behind stride-1
    # max pools, examples/fashion_mnist/main.rs:187-199 -- and not one of the five configurations)
    builds = (("cfg1_linear_classifier_bs1000", lambda e: _w.linear_classifier(e), 2000, 5000),
              ("conv_blur_net_bs1000", lambda e: _w.convnet(e, blur_pool=True), 300, 600),
              ("cfg4_coordinate_mlp_relu_pe_512", lambda e: _w.coordinate_mlp(e), 40, 80),
              ("cfg4_coordinate_mlp_siren_512", lambda e: _w.coordinate_mlp(e, variant="siren"), 40, 80),
              ("cfg5_hash_grid_2p18", lambda e: _w.hash_grid_fit(e), 200, 400))
    for name, build, warmup, steps in builds:
        r, _ = bench_workload(env, build, steps, warmup, read_loss=True)
        out[name] = {"steps_per_s": round(r["steps_per_s"], 1), "ms_per_step": round(r["ms_per_step"], 4), "launches": r["launches_per_step"],
                     "clusters": r["clusters"], "steps": steps, "warmup": warmup, "loss_sum_finite": r["loss_finite"],
                     "kernel_classes": _compact_classes(r["kernel_classes"])}
    return out


def cpu_baseline_matmul(n: int, rows: int):
    """The CPU oracle (restatement of the reference's algorithm; the reference itself needs Rust + Vulkan) on
    a slab of `rows` rows of the same n^3 product, epilogue included, and on a few ConvNet train steps, all host
    cores through OpenMP."""
    from descent_amd import Environment, workloads
    from oracle.cpu_backend import CpuBackend

    env = Environment(CpuBackend())
    w = workloads.matmul_epilogue(env, rows, n, n, seed=2)
    env.run(w.graph, 1)  # warm
    t0 = time.perf_counter()
    env.run(w.graph, 1)
    dt = time.perf_counter() - t0
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    # the other half of the headline metric on the same cores: ConvNet (batch 1000) train steps
    cw = workloads.convnet(env, batch=1000, seed=3)
    env.run(cw.graph, 1)  # warm
    conv_steps = 24
    t0 = time.perf_counter()
    for i in range(conv_steps):
        env.run(cw.graph, 2 + i)
    conv_dt = time.perf_counter() - t0
    return {
        "value": 2.0 * rows * n * n / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": min(cores, threads),
        "kind": "port",
        "sample": f"{rows} of {n} rows of the {n}^3 product (A slab {rows}x{n}, full B), bias+leaky_relu included, {dt:.2f} s; "
                  f"plus {conv_steps} ConvNet bs1000 train steps, {conv_dt:.2f} s",
        "convnet_bs1000_steps_per_s": conv_steps / conv_dt,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the headline matmul")
    ap.add_argument("--shape", default=None, help="M,N,K: with --workload matmul, time this matmul + bias + leaky_relu "
                                                  "alone and print its line (e.g. under rocprofv3 --pmc)")
    ap.add_argument("--all", action="store_true", help="also time the other matmul shapes and the ConvNet step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="leave the other configurations out of the headline line")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only the streaming c=a*2+b kernel over 2^26 elements (counter calibration)")
    ap.add_argument("--cpu-rows", type=int, default=8192,
                    help="rows of the headline product the CPU baseline computes (a bounded sample of the same workload)")
    ap.add_argument("--workload", default="headline",
                    choices=["headline", "matmul", "convnet", "conv-blur-net", "convnet-uploads", "linear", "relu-pe", "siren", "hash-grid"],
                    help="headline: the 8192^3 matmul line with the ConvNet step rate beside it (default); matmul: "
                         "that line without the ConvNet; the others run one workload alone, e.g. under rocprofv3")
    ap.add_argument("--no-events", action="store_true", help="no per-launch HIP events (wall time only)")
    ap.add_argument("--min-warmup", type=int, default=1000,
                    help="convnet / conv-blur-net: warm-up steps at least (1000 bring the device to its sustained clock; a counter "
                         "run, which serialises every dispatch, wants a handful)")
    ap.add_argument("--markers", action="store_true",
                    help="wrap every launch in a ROCTx range named by the kernel's label (rocprofv3 --marker-trace)")
    args = ap.parse_args()
    global EVENT_PASS
    EVENT_PASS = not args.no_events
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; run with --gpus 1 (nothing here uses a second device)", file=sys.stderr)
        sys.exit(2)

    from descent_amd import Environment
    from descent_amd.hip_backend import HipBackend

    env = Environment(HipBackend())
    if args.markers:
        env.backend.markers(True)
    if args.copy_calibration:
        print(json.dumps(bench_elementwise(env, 1 << 26, args.steps, args.warmup)))
        return
    if args.workload not in ("headline", "matmul"):
        from descent_amd import workloads as _w

        if args.workload in ("convnet", "conv-blur-net"):
            out = bench_convnet(env, args.steps, args.warmup, blur_pool=args.workload == "conv-blur-net", min_warmup=args.min_warmup)
            sys.stderr.write(out.pop("report"))
        elif args.workload == "convnet-uploads":
            out = bench_convnet_minibatch_uploads(env, steps=max(args.steps, 20))
        else:
            build = {"linear": lambda e: _w.linear_classifier(e), "relu-pe": lambda e: _w.coordinate_mlp(e), "siren": lambda e: _w.coordinate_mlp(e, variant="siren"),
                     "hash-grid": lambda e: _w.hash_grid_fit(e)}[args.workload]
            out, rep = bench_workload(env, build, args.steps, args.warmup, topn=int(os.environ.get("DSC_BENCH_TOPN", "12")))
            sys.stderr.write(rep)
        out["workload"] = args.workload
        print(json.dumps(out))
        return
    n = args.size
    if args.shape:
        m_, n_, k_ = (int(v) for v in args.shape.split(","))
        r = bench_matmul(env, m_, n_, k_, args.steps, args.warmup)
        sys.stderr.write(r.pop("report"))
        print(json.dumps(r))
        return
    head = bench_matmul(env, n, n, n, args.steps, args.warmup, verify=True)
    sys.stderr.write(head["report"])
    if not head["rel_l2_error_sampled_rows"] <= 1e-4:
        print("bench.py: the timed product is wrong: relative L2 error %r on 64 sampled rows against float64"
              % head["rel_l2_error_sampled_rows"], file=sys.stderr)
        sys.exit(1)

    extra = {}
    conv = None
    if args.all:
        extra["matmul"] = []
        for (m, nn, k), shape_warmup, shape_steps in CFG2_OTHER_SHAPES:
            r = bench_matmul(env, m, nn, k, shape_steps, shape_warmup)
            r.pop("report")
            extra["matmul"].append(r)
        extra["elementwise_axpb_64M"] = bench_elementwise(env, 1 << 26, 1500, 1000)
        extra["host_operands"] = bench_upload(env, n)
        extra["convnet_bs1000_minibatch_uploads"] = bench_convnet_minibatch_uploads(env)
        extra["reduce"] = [bench_reduce(env, 8192, 8192, 1, 3000, 2000), bench_reduce(env, 8192, 8192, 0, 3000, 2000),
                           bench_reduce(env, 262144, 256, 0, 3000, 2000)]
        from descent_amd import workloads as _w

        mlp, rep = bench_workload(env, lambda e: _w.coordinate_mlp(e), 80, 40)
        sys.stderr.write("cfg4 coordinate MLP (relu-pe):\n" + rep)
        extra["coordinate_mlp_relu_pe_512"] = mlp
        siren, rep = bench_workload(env, lambda e: _w.coordinate_mlp(e, variant="siren"), 80, 40)
        extra["coordinate_mlp_siren_512"] = siren
        lin, rep = bench_workload(env, lambda e: _w.linear_classifier(e), 5000, 2000)
        sys.stderr.write("cfg1 linear classifier:\n" + rep)
        extra["linear_classifier_bs1000"] = lin
        hg, rep = bench_workload(env, lambda e: _w.hash_grid_fit(e), 400, 200)
        sys.stderr.write("cfg5 hash grid:\n" + rep)
        sc = hg["kernel_classes"].get("Multi (4 kernels: ScatterAdd") or hg["kernel_classes"].get("ScatterAdd")
        hg["scatter_atomics_per_s"] = 16 * 4 * 2 * (1 << 18) / (sc["us_per_step"] * 1e-6) if sc else None
        extra["hash_grid_2p18"] = hg
    if args.workload == "headline":
        # the other half of the headline metric: ConvNet (batch 1000) train steps per second
        conv = bench_convnet(env, max(args.steps, 200), args.warmup)
        sys.stderr.write(conv.pop("report"))
    configs = bench_configs(env) if args.workload == "headline" and not args.no_configs else None

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_matmul(n, args.cpu_rows)

    achieved = head["tflops_kernel"] or head["tflops_wall"]
    line = {
        "metric": "fp32 matmul TFLOP/s (M=N=K=%d through the array API, fused bias + leaky_relu epilogue)" % n,
        "value": head["tflops_wall"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg2 standalone fp32 matmul %dx%dx%d + bias + leaky_relu(0.01), N(0,1) entries" % (n, n, n),
                   "launches_per_step": head["launches_per_step"]},
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": MFMA_FP32_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / MFMA_FP32_PEAK_TFLOPS,
            "traffic": MEASURED_TRAFFIC_BYTES.get(n),
            "kernel_avg_us": head["kernel_avg_us"],
            "algorithmic_flops_per_launch": head["flops"],
        },
        "cpu_baseline": cpu,
        # 64 sampled rows of the C the timed launches wrote, against a float64 product of the operands read back
        "verified": bool(head["rel_l2_error_sampled_rows"] <= 1e-4),
        "rel_l2_error_sampled_rows": head["rel_l2_error_sampled_rows"],
    }
    if conv is not None:
        # the first half of the headline metric: ConvNet (batch 1000) train steps per second, with the step's own roofline
        line["convnet_bs1000"] = conv
    if configs is not None:
        # the remaining configurations, timed in this same run (matmul shapes verified on sampled rows)
        line["configs"] = configs
    if extra:
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
