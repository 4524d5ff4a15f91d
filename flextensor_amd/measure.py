"""Build, check and time one candidate on the local GPU.

Counterpart of the reference's flextensor/measure.py: ``build_and_eval``
(:77-115) is tvm.build -> export_library -> load_module -> time_evaluator;
here it is hiprtc -> hipModule -> hipEvent timing through libftrocm.so, with
one step the reference lacks: before a timing is admitted the candidate's
output is compared *on the device* with the output of the plain
one-lane-per-output kernel of the same operator (templates/naive.hip), which
plays the role of the reference's default-schedule build
(flextensor/optimize/common.py:63-82). fp32 must satisfy
max|out-ref| / max|ref| <= 1e-5; int32 must be identical.

Candidates are evaluated in this process: forking a child per candidate, as
the reference does (:55-74), is not safe once the HIP runtime is initialised.
A failing candidate never propagates: callers map any exception to ``inf``.
"""
import ctypes
import struct

import numpy as np

from . import runtime as rt
from .plan import KernelPlan, current_stream
from .templates import gfx950
from .utils import to_tuple, ceil_div

FP32_TOL = 1e-5
WARM_MS = 60.0             # untimed device work before a candidate is timed
# buffers of a memory-bound operator are rotated so that consecutive timed
# launches do not find their data in the 256 MB last-level cache
LLC_BYTES = 256 << 20
MAX_SETS = 24


class WrongResult(RuntimeError):
    """A candidate kernel ran but its output failed the correctness gate."""


def seeded_inputs(bufs, seed=0):
    """Host arrays for the input buffers: fp32 uniform[-1,1), int8 uniform
    over [-128,127], from numpy's default_rng(seed)."""
    rng = np.random.default_rng(seed)
    arrays = []
    for b in bufs[:-1]:
        shape = to_tuple(b.shape)
        if b.dtype == "float32":
            arrays.append(rng.uniform(-1.0, 1.0, size=shape).astype(np.float32))
        elif b.dtype == "int8":
            arrays.append(rng.integers(-128, 128, size=shape, dtype=np.int8))
        else:
            raise ValueError("no input generator for dtype %s" % b.dtype)
    return arrays


_naive_modules = {}


def _naive(kernel):
    if kernel not in _naive_modules:
        src = gfx950.template_source("naive.hip")
        _naive_modules[kernel] = rt.Module(rt.compile_to_code(src, []), kernel)
    return _naive_modules[kernel]


def _grid1d(n, cap=None):
    g = ceil_div(int(n), 256)
    if cap:
        g = min(g, cap)
    return (max(g, 1), 1, 1)


def run_default_schedule(ops, tensors, stream=0):
    """Run the task with the plain per-output kernels (the 'default schedule').

    ``ops`` is the task's output op list; ``tensors`` are device tensors in
    ``bufs`` order and the last one receives the result. Intermediate
    operators (padding) are folded into the consumer's index predicate, which
    is what the operator definitions compute.
    """
    op = ops[0]
    i32 = ctypes.c_int
    out = tensors[-1]
    if op.kind == "bias_add_nchw":
        # the stage before it first (into a temporary), then one lane per output adds the bias
        import torch
        from .templates import gfx950
        tmp = torch.empty_like(out)
        run_default_schedule([op.input_tensors[0].op], list(tensors[:-2]) + [tmp], stream=stream)
        b, c, h, w = [a.extent for a in op.axis]
        n = b * c * h * w
        mod = rt.Module(rt.compile_to_code(gfx950.template_source("elementwise.hip"), []), "bias_add_nchw_f32")
        mod.launch(_grid1d(n), (256, 1, 1), [rt.ptr(tmp), rt.ptr(tensors[-2]), rt.ptr(out), i32(n), i32(h * w), i32(c)],
                   stream=stream)
        torch.cuda.synchronize()
        mod.close()
        return
    if op.kind == "col2img_nchw":
        # im2col, GEMM, (bias,) col2img define the same function as the direct
        # convolution: one lane per output runs the convolution's own sum
        import torch
        from .templates import gfx950
        stage = op.input_tensors[0].op
        has_bias = stage.kind == "bias_add_ghw"
        if has_bias:
            stage = stage.input_tensors[0].op
        a = stage.attrs
        b, ko, p, q = [x.extent for x in op.axis]
        _, c, h, w = a["in_shape"]
        r, s = a["kernel"]
        dst = torch.empty_like(out) if has_bias else out
        args = [rt.ptr(tensors[0]), rt.ptr(tensors[1]), rt.ptr(dst)] + [i32(v) for v in (
            b, c, h, w, ko, r, s, a["stride"][0], a["stride"][1], a["padding"][0], a["padding"][1],
            a["dilation"][0], a["dilation"][1], a["groups"], p, q)]
        _naive("conv2d_nchw_naive").launch(_grid1d(b * ko * p * q), (256, 1, 1), args, stream=stream)
        if has_bias:
            n = b * ko * p * q
            mod = rt.Module(rt.compile_to_code(gfx950.template_source("elementwise.hip"), []), "bias_add_nchw_f32")
            mod.launch(_grid1d(n), (256, 1, 1), [rt.ptr(dst), rt.ptr(tensors[2]), rt.ptr(out), i32(n), i32(p * q), i32(ko)],
                       stream=stream)
            torch.cuda.synchronize()
            mod.close()
        return
    if op.kind == "batch_gemm":
        nb, M, N = [a.extent for a in op.axis]
        K = op.reduce_axis[0].extent
        for b in range(nb):
            args = [rt.ptr(tensors[0][b]), rt.ptr(tensors[1][b]), rt.ptr(out[b]), i32(M), i32(N), i32(K),
                    i32(1 if op.attrs.get("transposeB") else 0), i32(1 if op.attrs.get("transposeA") else 0)]
            _naive("gemm_f32_naive").launch(_grid1d(M * N), (256, 1, 1), args, stream=stream)
        return
    if op.kind == "gemm":
        M, N = [a.extent for a in op.axis]
        K = op.reduce_axis[0].extent
        args = [rt.ptr(tensors[0]), rt.ptr(tensors[1]), rt.ptr(out), i32(M), i32(N), i32(K),
                i32(1 if op.attrs.get("transposeB") else 0), i32(1 if op.attrs.get("transposeA") else 0)]
        _naive("gemm_f32_naive").launch(_grid1d(M * N), (256, 1, 1), args, stream=stream)
    elif op.kind == "gemm_int8":
        M, N = [a.extent for a in op.axis]
        K = op.reduce_axis[0].extent
        args = [rt.ptr(tensors[0]), rt.ptr(tensors[1]), rt.ptr(out), i32(M), i32(N), i32(K)]
        _naive("gemm_i8_naive").launch(_grid1d(M * N), (256, 1, 1), args, stream=stream)
    elif op.kind == "conv2d_nchw":
        a = op.attrs
        b, ko, p, q = [x.extent for x in op.axis]
        _, c, h, w = a["in_shape"]
        s, r = op.reduce_axis[1].extent, op.reduce_axis[2].extent
        args = [rt.ptr(tensors[0]), rt.ptr(tensors[1]), rt.ptr(out)] + [i32(v) for v in (
            b, c, h, w, ko, r, s, a["stride"][0], a["stride"][1], a["padding"][0], a["padding"][1],
            a["dilation"][0], a["dilation"][1], a["groups"], p, q)]
        _naive("conv2d_nchw_naive").launch(_grid1d(b * ko * p * q), (256, 1, 1), args, stream=stream)
    elif op.kind == "depthwise_conv2d_nchw":
        a = op.attrs
        b, co, p, q = [x.extent for x in op.axis]
        _, c, h, w = a["in_shape"]
        s, r = op.reduce_axis[0].extent, op.reduce_axis[1].extent
        args = [rt.ptr(tensors[0]), rt.ptr(tensors[1]), rt.ptr(out)] + [i32(v) for v in (
            b, c, h, w, a["factor"], r, s, a["stride"][0], a["stride"][1], a["padding"][0],
            a["padding"][1], a["dilation"][0], a["dilation"][1], p, q)]
        _naive("depthwise_nchw_naive").launch(_grid1d(b * co * p * q), (256, 1, 1), args, stream=stream)
    elif op.kind == "zero_pad2d":
        b, c, ph, pw = [x.extent for x in op.axis]
        pt, pb, pl, pr = op.attrs["padding"]
        args = [rt.ptr(tensors[0]), rt.ptr(out)] + [i32(v) for v in (
            b * c, ph - pt - pb, pw - pl - pr, pt, pb, pl, pr)]
        _naive("zero_pad2d_naive").launch(_grid1d(b * c * ph * pw), (256, 1, 1), args, stream=stream)
    else:
        raise NotImplementedError("no default-schedule kernel for %s" % op.kind)


def compare_on_device(out, ref, stream=0):
    """(passed, metric) with metric = max|out-ref|/max|ref| for fp32 tensors and
    the number of differing entries for int32 tensors."""
    import torch
    n = out.numel()
    res = torch.zeros(2, dtype=torch.int32, device=out.device)
    args = [rt.ptr(out), rt.ptr(ref), ctypes.c_longlong(n), rt.ptr(res)]
    if out.dtype == torch.float32:
        _naive("check_f32").launch(_grid1d(n, 2048), (256, 1, 1), args, stream=stream)
        bits = res.cpu().numpy().astype(np.uint32)
        md, mr = struct.unpack("ff", bits.tobytes())
        if not np.isfinite(md):
            return False, float("inf")
        rel = md / mr if mr > 0 else md
        return rel <= FP32_TOL, rel
    if out.dtype == torch.int32:
        _naive("check_i32").launch(_grid1d(n, 2048), (256, 1, 1), args, stream=stream)
        bad = int(res.cpu().numpy().astype(np.uint32)[0])
        return bad == 0, float(bad)
    raise ValueError("no comparison for dtype %s" % out.dtype)


class Measurer(object):
    """Device-resident inputs and the default-schedule result of one task."""

    def __init__(self, task_key, seed=0):
        import torch
        from .task import TASK_TABLE
        if not torch.cuda.is_available():
            raise rt.RuntimeError_("no GPU visible: candidates can only be measured on a device")
        self.task_key = task_key
        task = TASK_TABLE[task_key]
        self.ops, self.bufs = task.func(*task.args)
        torch.cuda.set_device(task.dev_id if task.dev_id < torch.cuda.device_count() else 0)
        host = seeded_inputs(self.bufs, seed)
        out_b = self.bufs[-1]
        tdt = {"float32": torch.float32, "int32": torch.int32}[out_b.dtype]
        bytes_per_set = sum(a.nbytes for a in host) + int(np.prod(out_b.shape)) * 4
        kind = self.ops[0].kind
        if kind == "depthwise_conv2d_nchw":
            nsets = int(min(MAX_SETS, max(1, ceil_div(2 * LLC_BYTES, bytes_per_set))))
        else:
            nsets = 1
        self.sets = []
        for i in range(nsets):
            ins = [torch.from_numpy(a).cuda() for a in host]
            self.sets.append(ins + [torch.empty(to_tuple(out_b.shape), dtype=tdt, device="cuda")])
        self.ref = torch.empty(to_tuple(out_b.shape), dtype=tdt, device="cuda")
        run_default_schedule(self.ops, self.sets[0][:-1] + [self.ref], stream=current_stream())
        torch.cuda.synchronize()

    def check(self, out):
        import torch
        ok, metric = compare_on_device(out, self.ref, stream=current_stream())
        torch.cuda.synchronize()
        return ok, metric

    def shader_clock(self, plan, ms=25.0, warm_ms=150.0):
        """The shader clock ``plan``'s main kernel sustains, read inside the kernel: the
        instrumented build of its template (KernelPlan.with_clock_probe) runs back to back for
        ``warm_ms`` + ``ms`` milliseconds like a timed measurement, and every workgroup of the last
        launch reports the shader clocks (s_memtime) and the ticks of the constant 100 MHz counter
        (s_memrealtime) of its life. Returns {"ghz": median ratio, "ghz_min", "ghz_max" (5th and
        95th percentile over the workgroups), "workgroup_us": median life of a workgroup,
        "workgroups": how many reported}. The result of the instrumented run is checked too."""
        import torch
        probe = plan.with_clock_probe()
        built = probe.build()
        try:
            first = self.sets[0]
            built(*first)
            torch.cuda.synchronize()
            ok, metric = self.check(first[-1])
            if not ok:
                raise WrongResult("instrumented build differs from the default schedule (metric %g)" % metric)
            one = built.time(self.sets, warmup=2, iters=5)
            built.time(self.sets, warmup=1, iters=max(int(ms / max(one, 1e-4)), 5), warm_ms=warm_ms)
            torch.cuda.synchronize()
            clk = built.scratch["clk_probe"].cpu().numpy().astype(np.float64)
        finally:
            built.close()
        clk = clk[clk[:, 1] >= 20]          # workgroups that found no work live a few ticks
        if len(clk) == 0:
            return None
        ghz = clk[:, 0] / clk[:, 1] * 0.1   # clocks per 10 ns
        return {"ghz": float(np.median(ghz)), "ghz_min": float(np.percentile(ghz, 5)),
                "ghz_max": float(np.percentile(ghz, 95)), "workgroup_us": float(np.median(clk[:, 1]) / 100.0),
                "workgroups": int(len(clk))}

    def time_axis(self, plan, launches=3000, warm_ms=150.0):
        """Where the time of a launch goes when launches follow one another on one stream, read
        inside the kernels: two instrumented builds of ``plan`` (KernelPlan.with_clock_probe with
        ``absolute=True``) are launched in turn, so the stamps of the last two launches survive,
        and every workgroup reports the device's 100 MHz counter at its begin and at the
        completion of its first wavefront's stores. Returns microseconds: ``period`` (first begin
        of one launch to first begin of the next), ``start_skew`` (first to last begin of a launch),
        ``first_end`` / ``last_end`` (after the launch's first begin) and ``gap`` (last end of one
        launch to first begin of the next: the other wavefronts' last stores, the write-back of
        what the launch left in the caches, and the dispatch of the next launch). 10 ns steps."""
        import torch
        builds = [plan.with_clock_probe(absolute=True).build() for _ in range(2)]
        try:
            sets = self.sets
            for b in builds:
                b(*sets[0])
            torch.cuda.synchronize()
            for b in builds:
                ok, metric = self.check(sets[0][-1])
                if not ok:
                    raise WrongResult("instrumented build differs from the default schedule (metric %g)" % metric)
            builds[0].time(sets, warmup=1, iters=5, warm_ms=warm_ms)
            # one call enqueues the whole alternating sequence, so the launches follow one another
            # as closely as the device lets them (launched one by one the host would set the pace)
            per = [[x.launches(ts) for ts in sets] for x in builds]
            pairs = max(int(launches) // 2, 1)      # an even number: the second build launches last
            seq = [d for i in range(2 * pairs) for d in per[i % 2][i % len(sets)]]
            rt._check(rt.lib().ftr_launch_seq(rt._desc_array(seq), len(seq), ctypes.c_void_p(current_stream())),
                      "ftr_launch_seq")
            torch.cuda.synchronize()
            a, b = [x.scratch["clk_probe"].cpu().numpy().astype(np.int64) for x in builds]
        finally:
            for x in builds:
                x.close()
        a, b = a[a[:, 1] - a[:, 0] >= 20], b[b[:, 1] - b[:, 0] >= 20]     # workgroups that found work
        t0 = a[:, 0].min()
        us = lambda ticks: float(ticks) / 100.0
        return {"period": us(b[:, 0].min() - t0), "start_skew": us(a[:, 0].max() - t0),
                "first_end": us(a[:, 1].min() - t0), "last_end": us(a[:, 1].max() - t0),
                "gap": us(b[:, 0].min() - a[:, 1].max()), "workgroups": int(len(a))}

    def evaluate(self, plan, number=10, warmup=2, warm_ms=WARM_MS, timeout=0.0):
        """ms per run of ``plan``; raises on build failure or wrong output.
        Candidates are compiled between measurements, so each one meets an
        idle device: ``warm_ms`` of untimed runs bring the clocks up first.

        ``timeout`` > 0 is the candidate's time limit in seconds
        (flextensor/measure.py:63-74 gives a child process that long): every
        wait on the device has that deadline and raises
        ``runtime.DeviceTimeout`` when it passes. The work already enqueued
        cannot be taken back, so the next candidate first waits (with its own
        deadline) for the stream to run empty; while it has not, candidates
        keep failing instead of being timed behind foreign work."""
        import torch
        timeout = float(timeout or 0.0)
        stream = current_stream()
        if timeout > 0:
            rt.stream_idle(stream, timeout)
            for m in _abandoned:          # the stream is empty: what an overrun left loaded can go
                m.close()
            del _abandoned[:]
        built = plan.build()
        try:
            first = self.sets[0]
            first[-1].zero_()
            built(*first)
            if timeout > 0:
                rt.stream_idle(stream, timeout)
            torch.cuda.synchronize()
            ok, metric = self.check(first[-1])
            if not ok:
                raise WrongResult("output differs from the default schedule (metric %g)" % metric)
            return built.time(self.sets, warmup=warmup, iters=max(int(number), 1), warm_ms=warm_ms,
                              timeout=timeout)
        finally:
            if timeout > 0:
                # unloading a module waits for its kernels: give up after the limit and leave the
                # modules to the garbage collector rather than block on a candidate that overran
                try:
                    rt.stream_idle(stream, timeout)
                except rt.DeviceTimeout:
                    _abandoned.extend(built.modules)
                    built.modules = []
            built.close()


_measurers = {}
_abandoned = []       # modules of candidates that overran their time limit, kept loaded until the stream is idle


def get_measurer(task_key, seed=0):
    key = (task_key, seed)
    if key not in _measurers:
        _measurers.clear()  # one task at a time keeps device memory bounded
        _measurers[key] = Measurer(task_key, seed)
    return _measurers[key]


def build_and_eval(lib, s, bufs, target, dev_id, rpc_info=None, number=1, timeout=0.0):
    """Build plan ``s``, verify it, time ``number`` launches; returns mean ms.

    ``lib`` (a path the reference writes the exported library to) receives the
    code object of the plan's last kernel when it is not None.
    """
    if not isinstance(s, KernelPlan):
        raise TypeError("build_and_eval expects a KernelPlan")
    if rpc_info is not None and getattr(rpc_info, "use_rpc", None):
        raise RuntimeError("remote measurement is not supported by the gfx950 backend")
    if lib:
        codes = s.compile()
        with open(lib, "wb") as f:
            f.write(codes[-1])
    return get_measurer(s.task_key).evaluate(s, number=number, timeout=timeout)


def _evaluate(s, bufs, target, dev_id, number=1, q=None, timeout=0.0):
    """In-process build + time (flextensor/measure.py:29-52)."""
    time_cost = build_and_eval(None, s, bufs, target, dev_id, None, number, timeout=timeout)
    if q:
        q.put(time_cost)
    return time_cost


def servant_routine(func, que, *args, **kwargs):
    try:
        ret = func(*args, **kwargs)
    except Exception as e:  # noqa: BLE001 - every failure becomes a value
        ret = e
    que.put(ret)


def master_routine(timeout, func, *args, **kwargs):
    """Run ``func`` and return its result, or the exception it raised
    (a ``runtime.DeviceTimeout`` when the time limit passed).

    The reference runs ``func`` in a forked child and waits ``timeout`` seconds
    (flextensor/measure.py:63-74). A process that has initialised the GPU must
    not fork, so the call is made in-process and the limit is enforced where
    the time goes: ``timeout`` is handed to ``func`` as its ``timeout``
    keyword (``_evaluate`` / ``build_and_eval`` pass it to the device waits,
    which poll with a deadline). Kernels built from the templates have
    compile-time loop bounds and always terminate; a candidate that overruns
    is abandoned, not killed.
    """
    try:
        if timeout:
            import inspect
            params = inspect.signature(func).parameters
            if "timeout" in params or any(p.kind == p.VAR_KEYWORD for p in params.values()):
                kwargs.setdefault("timeout", timeout)
        return func(*args, **kwargs)
    except Exception as e:  # noqa: BLE001
        return e
