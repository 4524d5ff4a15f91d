"""Kernel plans: what ``schedule_with_config`` returns in place of a TVM schedule.

A ``KernelPlan`` is the host-side description of how one task runs on the
device: an ordered list of ``KernelSpec`` (template + constants + geometry)
and the intermediate buffers between them. ``build`` compiles and loads the
kernels and yields a callable over device tensors in ``bufs`` order — the
counterpart of ``tvm.build(s, bufs, target)`` followed by ``func(*arrays)``
in the reference (README.md:151-158, flextensor/optimize/common.py:34-48).
"""
import ctypes

from . import runtime as rt


class KernelPlan(object):
    def __init__(self, task_key, bufs, specs, intermediates, configs):
        self.task_key = task_key
        self.bufs = list(bufs)
        self.specs = list(specs)
        # name -> (shape, dtype) of buffers the plan owns (e.g. a padded image)
        self.intermediates = dict(intermediates)
        # name -> (shape, dtype) of zero-initialised workspaces the kernels declare
        self.workspaces = {}
        for spec in self.specs:
            self.workspaces.update(getattr(spec, "workspace", {}))
        self.configs = configs
        # argument names of the caller's buffers, inputs..., output
        self.buf_names = ["in%d" % i for i in range(len(bufs) - 1)] + ["out"]

    def describe(self):
        return [(s.kernel, dict(s.defines), s.grid, s.block) for s in self.specs]

    def compile(self, arch=rt.DEFAULT_ARCH):
        """Compile every kernel to a code object (no device needed)."""
        return [rt.compile_to_code(s.source(), s.options(), arch) for s in self.specs]

    def build(self, static_workspace=False):
        return BuiltPlan(self, static_workspace=static_workspace)

    def verify(self, static=True):
        """Run the plan once on the task's seeded inputs and compare the result with the
        default-schedule kernels on the device (the gate every candidate of a search passes):
        fp32 max|out - ref| / max|ref| <= 1e-5, int32 bit-exact. With ``static`` and hipcc
        installed the generated assembly goes through the static checks as well. Returns the
        metric; raises measure.WrongResult otherwise. For plans that did not come out of a
        search: a config replayed from a log, or written by hand."""
        import os
        from . import isa_check
        from .measure import WrongResult, get_measurer
        m = get_measurer(self.task_key)
        built = self.build()
        try:
            built(*m.sets[0])
            ok, metric = m.check(m.sets[0][-1])
        finally:
            built.close()
        if not ok:
            raise WrongResult("%s: result differs from the default schedule's (metric %g)" % (self.task_key, metric))
        if static and os.path.exists(isa_check.HIPCC):
            found = isa_check.check_plan(self)
            if found:
                raise WrongResult("%s: static check of the assembly: %s" % (self.task_key, found[:2]))
        return metric

    def with_clock_probe(self, absolute=False):
        """A copy of the plan whose main kernel is the instrumented build of its template
        (FT_CLKPROBE): every workgroup writes the shader clocks and the ticks of the 100 MHz
        counter it lived into the workspace ``clk_probe`` ([workgroups][2] int64). Same work,
        same launch geometry; used to read the clock the kernel sustains, never timed.
        ``absolute``: the two numbers are the 100 MHz counter's own readings at the workgroup's
        begin and end instead (one counter for the whole device), which puts the workgroups of
        several launches on one time axis."""
        import copy
        idx = [i for i, s in enumerate(self.specs) if s.template in PROBE_TEMPLATES]
        if not idx:
            raise ValueError("no kernel of this plan can carry the clock probe")
        specs = list(self.specs)
        spec = copy.copy(specs[idx[-1]])
        spec.defines = dict(spec.defines, CLKPROBE=2 if absolute else 1)
        spec.args = list(spec.args) + [("buf", "clk_probe")]
        nwg = spec.grid[0] * spec.grid[1] * spec.grid[2]
        spec.workspace = dict(spec.workspace, clk_probe=((nwg, 2), "int64"))
        specs[idx[-1]] = spec
        return KernelPlan(self.task_key, self.bufs, specs, self.intermediates, self.configs)

    def __repr__(self):
        return "KernelPlan(%s: %s)" % (self.task_key, ", ".join(s.kernel for s in self.specs))


# templates that take the FT_CLKPROBE instrumentation
PROBE_TEMPLATES = ("igemm_f32.hip", "gemm_i8.hip", "depthwise_f32.hip")


_TORCH_DTYPES = None


def _torch_dtype(name):
    global _TORCH_DTYPES
    import torch
    if _TORCH_DTYPES is None:
        _TORCH_DTYPES = {"float32": torch.float32, "int8": torch.int8, "int32": torch.int32,
                         "int64": torch.int64}
    return _TORCH_DTYPES[name]


def current_stream():
    """Handle of the stream device work is enqueued on (torch's current one)."""
    import torch
    return int(torch.cuda.current_stream().cuda_stream)


class BuiltPlan(object):
    """Loaded kernels of a plan; call it with device tensors in ``bufs`` order."""

    def __init__(self, plan, static_workspace=False):
        """``static_workspace=True`` keeps the plan's workspaces (K-streaming
        slots and counters) in the runtime library's fixed device array instead
        of allocating them, and calls go through ftr_launch_seq_static_ws."""
        import torch
        if not torch.cuda.is_available():
            raise rt.RuntimeError_("no GPU visible: a kernel plan can only be built on a device")
        self.plan = plan
        self.modules = []
        for spec, code in zip(plan.specs, plan.compile()):
            self.modules.append(rt.Module(code, spec.kernel))
        self.scratch = {}
        for name, (shape, dtype) in plan.intermediates.items():
            self.scratch[name] = torch.empty(shape, dtype=_torch_dtype(dtype), device="cuda")
        self.static_layout = None
        if static_workspace:
            # name -> (offset, bytes, zero): consecutive 256-byte aligned ranges; the
            # arrival counters must start at zero, the slots are written before they are read
            self.static_layout, offset = {}, 0
            for name, (shape, dtype) in sorted(plan.workspaces.items()):
                n = 1
                for d in shape:
                    n *= int(d)
                nbytes = (n * {"float32": 4, "int32": 4, "int8": 1, "int64": 8}[dtype] + 15) // 16 * 16
                self.static_layout[name] = (offset, nbytes, 0 if name.endswith("_parts") else 1)
                offset = (offset + nbytes + 255) // 256 * 256
            if offset > rt.STATIC_WS_BYTES:
                raise rt.RuntimeError_("the plan's workspaces need %d bytes, the static workspace holds %d"
                                       % (offset, rt.STATIC_WS_BYTES))
        else:
            for name, (shape, dtype) in plan.workspaces.items():
                self.scratch[name] = torch.zeros(shape, dtype=_torch_dtype(dtype), device="cuda")

    def attrs(self):
        return [m.attrs() for m in self.modules]

    def _check(self, tensors):
        plan = self.plan
        if len(tensors) != len(plan.bufs):
            raise ValueError("expected %d tensors (inputs..., output), got %d"
                             % (len(plan.bufs), len(tensors)))
        for t, b in zip(tensors, plan.bufs):
            if tuple(t.shape) != tuple(b.shape):
                raise ValueError("tensor shape %s does not match %s" % (tuple(t.shape), b))
            if t.dtype != _torch_dtype(b.dtype):
                raise ValueError("tensor dtype %s does not match %s" % (t.dtype, b))
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError("tensors must be contiguous device tensors")

    def launches(self, tensors):
        """Launch descriptors of one run over ``tensors`` (validated)."""
        self._check(tensors)
        named = dict(zip(self.plan.buf_names, tensors))
        named.update(self.scratch)
        out = []
        self._binds = []
        for li, (spec, mod) in enumerate(zip(self.plan.specs, self.modules)):
            vals = []
            for ai, (kind, v) in enumerate(spec.args):
                if kind == "buf" and self.static_layout is not None and v in self.static_layout:
                    vals.append(ctypes.c_void_p(0))      # the library writes the address here
                    self._binds.append((li, ai) + self.static_layout[v])
                elif kind == "buf":
                    vals.append(rt.ptr(named[v]))
                elif kind == "i32":
                    vals.append(ctypes.c_int(int(v)))
                elif kind == "u32":
                    vals.append(ctypes.c_uint(int(v)))
                elif kind == "i64":
                    vals.append(ctypes.c_longlong(int(v)))
                else:
                    raise ValueError("unknown argument kind %s" % kind)
            out.append(rt.Launch(mod, spec.grid, spec.block, vals, spec.lds_bytes))
        return out

    def __call__(self, *tensors):
        launches = self.launches(tensors)
        if self.static_layout is not None:
            rt.launch_seq_static_ws(launches, self._binds, stream=current_stream())
        else:
            rt.launch_seq(launches, stream=current_stream())

    def time(self, tensor_sets, warmup=2, iters=10, warm_ms=0.0, timeout=0.0):
        """Mean ms per run, rotating through ``tensor_sets``. ``timeout`` > 0
        is a deadline in seconds for each wait on the device
        (runtime.DeviceTimeout when it passes).

        ``warm_ms`` > 0 keeps the device busy with untimed runs for about that
        long first: after an idle period the clocks take on the order of
        100 ms of continuous work to reach their steady state, and a kernel
        timed before that reads 15-25 % slow."""
        if self.static_layout is not None:
            raise rt.RuntimeError_("timing runs over caller-owned workspaces: build without static_workspace")
        sets = [self.launches(ts) for ts in tensor_sets]
        stream = current_stream()
        if warm_ms > 0:
            probe = rt.time_seq(sets, warmup=1, iters=3, stream=stream, timeout=timeout)
            warmup = max(warmup, int(min(warm_ms / max(probe, 1e-4), 1e6)))
        return rt.time_seq(sets, warmup=warmup, iters=iters, stream=stream, timeout=timeout)

    def close(self):
        for m in self.modules:
            m.close()
        self.modules = []


def build(s, bufs=None, target=None):
    """``build(s, bufs, target)``: the call a user of the reference makes with
    ``tvm.build`` on the result of ``schedule`` / ``schedule_with_config``."""
    if not isinstance(s, KernelPlan):
        raise TypeError("expected the plan returned by schedule()/schedule_with_config()")
    return s.build()
