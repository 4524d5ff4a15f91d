#!/usr/bin/env python3
"""Benchmark of the tuned hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only-headline]
                    [--workload NAME]

One step = one run of the tuned kernel plan of the headline workload, the
largest single-GPU configuration of the benchmark set (int8 x int8 -> int32
GEMM, M = N = K = 4096, B stored K-major), over seeded synthetic inputs that
are resident in HBM before the timed region. The device is first kept busy
for about 150 ms (idle clocks need that long to settle), then W untimed
steps, then exactly K steps between two device synchronisations.
Prints ONE JSON line with the whole-job throughput (`value`, TFLOP/s), the
roofline position of the dominant kernel measured with HIP events on the
launch stream, the same figures for the other benchmark configurations
(`per_config`) and the CPU baseline (the multi-threaded CPU port of the
reference's llvm path, oracle/cpu_baseline.c) timed on this host.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published MI355X peaks (dense)
PEAK_F32_TFLOPS = 157.3
PEAK_I8_TOPS = 5000.0
PEAK_HBM_GBS = 8000.0

WORKLOADS = [
    # name, task key, op count (FLOP or OP), compulsory bytes, bound, dtype
    ("gemm_f32_1024", "gemm_gemm_(1024, 1024, 1024)_rocm(0)", 2 * 1024 ** 3, 12582912, "mfma", "f32"),
    ("conv2d_1x64x56x56_k64_3x3", "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)",
     231211008, 1753088, "mfma", "f32"),
    ("conv2d_8x256x14x14_k512_3x3", "conv2d_baseline1_(8, 256, 14, 14, 512, 3, 1, 1, 1, 1)_rocm(0)",
     3699376128, 9535488, "mfma", "f32"),
    ("conv2d_8x512x7x7_k2048_1x1", "conv2d_baseline2_(8, 512, 7, 7, 2048, 1, 1, 0, 1, 1)_rocm(0)",
     822083584, 8208384, "mfma", "f32"),
    ("depthwise_8x512x28x28_3x3", "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)",
     57802752, 25708544, "hbm", "f32"),
    ("gemm_i8_4096", "gemm_gemm_int8_(4096, 4096, 4096)_rocm(0)", 2 * 4096 ** 3, 100663296, "mfma", "i8"),
]
# The metric is quoted per operator, on no single configuration, so the headline is the largest
# configuration that fits one GPU: configs[4] of the benchmark set (137 GOP per step).
HEADLINE = 5
HEADLINE_NOTE = " (largest single-GPU configuration, BASELINE.json configs[4])"


def config_hash(plan):
    """Identifies the kernels a plan launches (templates' constants and geometry)."""
    import hashlib
    h = hashlib.sha256()
    for spec in plan.specs:
        h.update(("%s|%s|%s|%s;" % (spec.kernel, sorted(spec.defines.items()), spec.grid, spec.block)).encode())
    return h.hexdigest()[:16]


def measured_traffic(name, plan):
    """(HBM bytes per launch of the plan's kernels, provenance) from rocprofv3
    FETCH_SIZE / WRITE_SIZE runs scaled by a plain copy of known size
    (flextensor_amd/tuned/hbm_traffic.json). The record carries the hash of
    the kernels it was taken on: when the shipped config has changed since,
    the figure is withheld (None) instead of being reported for other kernels."""
    path = os.path.join(ROOT, "flextensor_amd", "tuned", "hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)[name]
    except (OSError, KeyError, ValueError):
        return None, None
    prov = {"measured": rec.get("measured"), "config_hash": rec.get("config_hash"),
            "current_config_hash": config_hash(plan)}
    if rec.get("config_hash") != prov["current_config_hash"]:
        prov["stale"] = True
        return None, prov
    return rec["hbm_bytes_per_launch"], prov


NOMINAL_GHZ = 2.4       # the shader clock the published MFMA peaks assume


def roofline(name, bound, dtype, ops, nbytes, ms, plan, clock=None):
    """``clock``: what Measurer.shader_clock read inside the instrumented build of the same kernel
    in the same process: the sustained shader clock (the published MFMA peaks assume 2.4 GHz; under
    load the power limit sets the real one, which differs from box to box) and the median life of a
    workgroup, which a kernel trace's duration and the per-launch event time both have to exceed."""
    traffic, prov = measured_traffic(name, plan)
    if bound == "hbm":
        achieved = nbytes / (ms * 1e-3) / 1e9
        out = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
               "frac": achieved / PEAK_HBM_GBS, "traffic": traffic, "traffic_provenance": prov}
    else:
        peak = PEAK_I8_TOPS if dtype == "i8" else PEAK_F32_TFLOPS
        achieved = ops / (ms * 1e-3) / 1e12
        out = {"bound": "mfma", "achieved": achieved, "peak": peak,
               "unit": "TOP/s" if dtype == "i8" else "TFLOP/s", "frac": achieved / peak,
               "traffic": traffic, "traffic_provenance": prov}
    if clock:
        out["shader_clock_ghz"] = clock["ghz"]
        out["shader_clock_ghz_p5_p95"] = [clock["ghz_min"], clock["ghz_max"]]
        out["workgroup_life_ms"] = clock["workgroup_us"] * 1e-3
        if "time_axis_us" in clock:
            # microseconds after a launch's first workgroup began: last begin, first and last end of a
            # workgroup (its first wavefront's stores completed); gap = last end -> first begin of the
            # next launch; period = begin to begin
            out["time_axis_us"] = clock["time_axis_us"]
        if bound == "mfma":
            # the same fraction against the peak at the clock the part sustains under this load
            out["frac_at_sustained_clock"] = out["frac"] * NOMINAL_GHZ / clock["ghz"]
    return out


def shader_clock(m, plan):
    """The sustained clock and, on one time axis of the device's 100 MHz counter, where a launch's
    time goes when launches follow one another (Measurer.time_axis): both read inside instrumented
    builds of the same kernel, after the timing."""
    try:
        clock = m.shader_clock(plan, ms=TIMED_WINDOW_MS, warm_ms=WARM_MS)
        if clock is not None:
            axis = m.time_axis(plan, launches=max(int(TIMED_WINDOW_MS / max(clock["workgroup_us"] * 1e-3, 2e-3)), 200),
                               warm_ms=WARM_MS)
            clock["time_axis_us"] = {k: axis[k] for k in ("period", "start_skew", "first_end", "last_end", "gap")}
        return clock
    except Exception as e:  # noqa: BLE001 - the clock is an annotation, the timing stands without it
        print("shader clock probe failed: %s" % e, file=sys.stderr)
        return None


def gpu_workload(key, seed=0):
    """(built plan, buffer sets, plan) for a task, using its shipped tuned config."""
    from flextensor_amd.measure import get_measurer
    from flextensor_amd.scheduler import schedule_with_config
    from flextensor_amd.tuned import lookup
    from flextensor_amd.utils import Config
    cfg = lookup(key) or Config([], None)
    s, _ = schedule_with_config(key, cfg)
    m = get_measurer(key, seed)
    built = s.build()
    return built, m, s


TIMED_WINDOW_MS = 25.0  # every workload is timed over about this much device time
WARM_MS = 150.0         # untimed device work first: idle clocks need ~100 ms to reach steady state


def kernel_ms(built, m, iters=None, warmup=20):
    """Mean duration of one plan run, HIP events on the launch stream. The
    number of timed launches is chosen so that every workload is measured
    over the same wall window (a 6 us kernel and a 70 us kernel then see the
    same clock/power conditions)."""
    import torch
    first = m.sets[0]
    built(*first)
    torch.cuda.synchronize()
    ok, metric = m.check(first[-1])
    if not ok:
        raise RuntimeError("tuned plan fails the correctness gate (metric %g)" % metric)
    if iters is None:
        probe = built.time(m.sets, warmup=warmup, iters=10)
        iters = int(min(max(TIMED_WINDOW_MS / max(probe, 1e-4), 20), 10000))
    return built.time(m.sets, warmup=warmup, iters=iters, warm_ms=WARM_MS), metric


def launch_floor_ms():
    """Mean time per launch of an empty kernel, back to back on the launch
    stream: what any kernel measured per launch pays before it does work."""
    from flextensor_amd import runtime as rt
    from flextensor_amd.plan import current_stream
    mod = rt.Module.from_source('extern "C" __global__ void ft_empty(int* p) { if (p == nullptr) return; }', "ft_empty")
    import torch
    x = torch.zeros(1, dtype=torch.int32, device="cuda")
    ms = mod.time((256,), (256,), [rt.ptr(x)], warmup=20000, iters=4000, stream=current_stream())
    mod.close()
    return ms


def copy_yardstick(mib, iters):
    """Time copy_f32 over `mib` MiB (read) + `mib` MiB (write)."""
    import ctypes as ct
    import torch
    from flextensor_amd import runtime as rt
    from flextensor_amd.plan import current_stream
    from flextensor_amd.templates import gfx950
    n = mib * (1 << 20) // 4
    src = torch.ones(n, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    mod = rt.Module(rt.compile_to_code(gfx950.template_source("elementwise.hip"), []), "copy_f32")
    ms = mod.time((8192,), (256,), [rt.ptr(src), rt.ptr(dst), ct.c_longlong(n)], warmup=3,
                  iters=iters, stream=current_stream())
    assert torch.equal(src[:1024], dst[:1024])
    return {"workload": "copy_%dMiB" % mib, "ms": ms, "read_bytes": n * 4, "write_bytes": n * 4,
            "GBps_read_plus_write": 2 * n * 4 / ms / 1e6}


def cpu_baseline_for(name, key, ops, budget_s):
    """Time the multi-threaded CPU port on the same seeded workload.
    GEMM and convolution first run a small sweep over the port's register
    tiles (and the GEMM's K tile), one pass each, and the best one is timed.
    Returns (ms per pass, threads, sample description)."""
    import numpy as np
    from flextensor_amd.measure import seeded_inputs
    from flextensor_amd.task import TASK_TABLE
    from oracle import oracle as o  # CPU baseline leg: the only use of the oracle here
    task = TASK_TABLE[key]
    _, bufs = task.func(*task.args)
    host = seeded_inputs(bufs, 0)
    threads = o.baseline_threads()
    frac = 1.0
    swept = ""

    def once(f):
        f()
        t = time.perf_counter()
        f()
        return time.perf_counter() - t

    if name.startswith("gemm_f32"):
        out = np.empty(bufs[-1].shape, np.float32)
        cands = [(v, tk) for v in range(len(o.baseline_gemm_f32_tiles())) for tk in (128, 256, 512)]
        best = min(cands, key=lambda c: once(lambda: o.baseline_gemm_f32_v(host[0], host[1], out, c[1], c[0])))
        swept = "; best of %d tilings: register tile %dx%d, K tile %d" % (
            (len(cands),) + o.baseline_gemm_f32_tiles()[best[0]] + (best[1],))
        fn = lambda: o.baseline_gemm_f32_v(host[0], host[1], out, best[1], best[0])  # noqa: E731
    elif name.startswith("gemm_i8"):
        out = np.zeros(bufs[-1].shape, np.int32)
        rows = 256
        frac = rows / bufs[-1].shape[0]
        fn = lambda: o.baseline_gemm_i8(host[0], host[1], out, 0, rows)  # noqa: E731
    elif name.startswith("conv2d"):
        a = task.args
        out = np.empty(bufs[-1].shape, np.float32)
        scratch = np.empty((a[0], a[1], a[2] + 2 * a[7], a[3] + 2 * a[7]), np.float32)
        cands = list(range(len(o.baseline_conv2d_tiles())))
        best = min(cands, key=lambda v: once(lambda: o.baseline_conv2d_v(host[0], host[1], out, scratch,
                                                                         a[6], a[7], a[8], v)))
        swept = "; best of %d register tiles: %d output channels x %d columns" % (
            (len(cands),) + o.baseline_conv2d_tiles()[best])
        fn = lambda: o.baseline_conv2d_v(host[0], host[1], out, scratch, a[6], a[7], a[8], best)  # noqa: E731
    else:
        a = task.args
        out = np.empty(bufs[-1].shape, np.float32)
        scratch = np.empty((a[0], a[1], a[2] + 2 * a[7], a[3] + 2 * a[7]), np.float32)
        fn = lambda: o.baseline_depthwise(host[0], host[1], out, scratch, a[6], a[7], a[8])  # noqa: E731
    fn()  # warm-up
    t0 = time.perf_counter()
    n = 0
    while True:
        fn()
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s or n >= 2000:
            break
    ms = el / n * 1e3 / frac
    sample = "%d passes of the full workload" % n if frac == 1.0 else \
        "%d passes over the first %d output rows, scaled to the full matrix" % (n, rows)
    return ms, threads, sample + swept


def cpu_baseline_dict(name, key, ops, dtype, budget_s):
    """The cpu_baseline object of one workload."""
    ms, threads, sample = cpu_baseline_for(name, key, ops, budget_s)
    naive_ms, naive_sample = cpu_naive_for(name, key)
    return {"value": ops / (ms * 1e-3) / 1e12, "unit": "TOP/s" if dtype == "i8" else "TFLOP/s", "cores": threads,
            "kind": "port", "ms": ms, "sample": sample + " (oracle/cpu_baseline.c, the "
            "reference's llvm template structure in C/OpenMP; TVM itself is unavailable)",
            "naive_1thread_ms": naive_ms, "naive_sample": naive_sample + " (oracle/oracle.c, the "
            "default-schedule loop nest on one thread)"}


def cpu_naive_for(name, key):
    """One pass of the default-schedule loop nest (what `create_schedule` + an
    llvm build gives before any tuning) on ONE host thread: the oracle's plain C
    restatement. The int8 GEMM is timed on 32 output rows and scaled.
    Returns (ms per full pass, sample description)."""
    import numpy as np
    from flextensor_amd.measure import seeded_inputs
    from flextensor_amd.task import TASK_TABLE
    from oracle import oracle as o  # CPU baseline leg only
    task = TASK_TABLE[key]
    _, bufs = task.func(*task.args)
    host = seeded_inputs(bufs, 0)
    a = task.args
    frac, sample = 1.0, "one pass of the full workload"
    t0 = time.perf_counter()
    if name.startswith("gemm_f32"):
        o.gemm_f32_c(host[0], host[1])
    elif name.startswith("gemm_i8"):
        rows = 32
        frac, sample = rows / bufs[-1].shape[0], "the first %d output rows, scaled to the full matrix" % rows
        o.gemm_i8_c(host[0], host[1], 0, rows)
    elif name.startswith("conv2d"):
        o.conv2d_nchw_c(host[0], host[1], a[6], a[7], a[8], a[9])
    else:
        o.depthwise_nchw_c(host[0], host[1], a[6], a[7], a[8])
    return (time.perf_counter() - t0) * 1e3 / frac, sample


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps K (default: about %g ms of device time)" % TIMED_WINDOW_MS)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps W (default: about %g ms of device time, which is what "
                         "idle clocks need to reach their steady state)" % WARM_MS)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--only-headline", action="store_true", help="skip the per_config table")
    ap.add_argument("--no-clock", action="store_true",
                    help="skip the in-kernel probes of the shader clock and of the launches' time axis "
                         "(instrumented builds of the same kernel, run after the timing; under a profiler "
                         "they would show up as extra dispatches)")
    ap.add_argument("--copy-mib", type=int, default=0,
                    help="instead of a workload, run a plain device copy of this many MiB "
                         "(bandwidth yardstick; calibrates FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--workload", default=None, choices=[w[0] for w in WORKLOADS],
                    help="time this configuration as the headline instead of the largest one "
                         "(used to profile one kernel at a time)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the tuned kernels are single-device and nothing "
              "here shards across GPUs; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from flextensor_amd import runtime as rt
    from flextensor_amd.plan import current_stream
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    props = rt.device_props(0)

    if args.copy_mib:
        print(json.dumps(copy_yardstick(args.copy_mib, max(args.steps or 100, 1))))
        return
    headline = HEADLINE if args.workload is None else [w[0] for w in WORKLOADS].index(args.workload)
    name, key, ops, nbytes, bound, dtype = WORKLOADS[headline]
    built, m, plan = gpu_workload(key)
    # ---- headline: W untimed steps, exactly K timed steps -----------------
    # one list of launches per buffer set; steps walk through the sets in turn (the depthwise
    # workload rotates enough sets that its traffic is HBM traffic, not cache hits)
    per_set = [built.launches(ts) for ts in m.sets]
    def steps_seq(n):
        return [d for i in range(n) for d in per_set[i % len(per_set)]]
    stream = current_stream()
    if args.steps is None or args.warmup is None:
        probe = built.time(m.sets, warmup=5, iters=20)
        if args.steps is None:
            args.steps = int(min(max(TIMED_WINDOW_MS / probe, 100), 100000))
        if args.warmup is None:
            args.warmup = int(min(max(WARM_MS / probe, 100), 100000))
    # clocks first: ~150 ms of untimed runs whatever W is, so that the timed steps (and the event
    # timing below) see the steady state and agree with each other
    built.time(m.sets, warmup=1, iters=2, warm_ms=WARM_MS)
    if args.warmup > 0:
        wseq = steps_seq(args.warmup)
        rt._check(rt.lib().ftr_launch_seq(rt._desc_array(wseq), len(wseq), ctypes.c_void_p(stream)),
                  "ftr_launch_seq")
    torch.cuda.synchronize()
    seq = steps_seq(args.steps)          # one C call enqueues all K steps
    arr = rt._desc_array(seq)
    t0 = time.perf_counter()
    rt._check(rt.lib().ftr_launch_seq(arr, len(seq), ctypes.c_void_p(stream)), "ftr_launch_seq")
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = ops / (ms_per_step * 1e-3) / 1e12
    ok, metric = m.check(m.sets[0][-1])
    if not ok:
        raise RuntimeError("headline plan fails the correctness gate (metric %g)" % metric)
    k_ms, _ = kernel_ms(built, m)
    roof = roofline(name, bound, dtype, ops, nbytes, k_ms, plan, None if args.no_clock else shader_clock(m, plan))
    roof["kernel"] = plan.specs[-1].kernel
    roof["kernel_ms"] = k_ms
    # 24 000 launches of an empty kernel: left out of the short runs that a profiler wraps
    # (--only-headline), where every dispatch is intercepted
    roof["launch_floor_ms"] = None if args.only_headline else launch_floor_ms()
    built.close()

    per_config = []
    if not args.only_headline:
        for (wname, wkey, wops, wbytes, wbound, wdtype) in WORKLOADS:
            b, mm, pl = gpu_workload(wkey)
            ms, met = kernel_ms(b, mm)
            r = roofline(wname, wbound, wdtype, wops, wbytes, ms, pl, None if args.no_clock else shader_clock(mm, pl))
            entry = {"workload": wname, "ms": ms, "dtype": wdtype,
                     "throughput": wops / (ms * 1e-3) / 1e12,
                     "throughput_unit": "TOP/s" if wdtype == "i8" else "TFLOP/s",
                     "roofline": r, "check": met,
                     "kernels": [s.kernel for s in pl.specs],
                     "config": json.loads(json.dumps(pl.configs))}
            b.close()
            per_config.append(entry)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_dict(name, key, ops, dtype, args.cpu_seconds)
        for entry, (wname, wkey, wops, _, _, wdtype) in zip(per_config, WORKLOADS):
            # every configuration carries its own baseline object; the headline's is the long sample
            entry["cpu_baseline"] = cpu if wname == name else cpu_baseline_dict(wname, wkey, wops, wdtype, 1.0)

    line = {
        "metric": "best-config TFLOPS + % of MI355X roofline per op vs CPU llvm baseline",
        "value": value, "unit": "TOP/s" if dtype == "i8" else "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": name + (HEADLINE_NOTE if headline == HEADLINE else ""), "task_key": key,
                   "tuned_config": json.loads(json.dumps(plan.configs)),
                   "device": props["name"], "arch": props["arch"]},
        "roofline": roof, "cpu_baseline": cpu, "per_config": per_config,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
