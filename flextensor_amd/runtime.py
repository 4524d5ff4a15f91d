"""ctypes binding of libftrocm.so (see include/ftrocm.h) plus an on-disk
code-object cache.

This is the only module that touches the device runtime. It stands where the
reference calls into TVM's runtime: ``tvm.build`` / ``export_library`` /
``load_module`` / ``time_evaluator`` (flextensor/measure.py:77-115).

There is no CPU fallback: if the shared library cannot be loaded, or a device
call fails, an exception is raised.
"""
import atexit
import ctypes
import hashlib
import json
import os
import subprocess
import sys
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libftrocm.so")
CACHE_DIR = os.environ.get("FLEXTENSOR_AMD_KCACHE", os.path.join(_HERE, "_kcache"))
DEFAULT_ARCH = "gfx950"
ABI_VERSION = 2
FTR_TIMEOUT = 2

EXPORTS = (
    "ftr_abi_version", "ftr_last_error", "ftr_compile_to_code", "ftr_code_free",
    "ftr_module_load", "ftr_compile", "ftr_module_free", "ftr_module_attrs",
    "ftr_launch", "ftr_launch_seq", "ftr_launch_seq_static_ws", "ftr_time", "ftr_time_seq",
    "ftr_time_seq_deadline", "ftr_stream_idle",
    "ftr_device_props", "ftr_device_count",
)


class RuntimeError_(RuntimeError):
    """A failing call into libftrocm.so."""


class DeviceTimeout(RuntimeError_):
    """A call with a deadline gave up waiting; the device work is still enqueued."""


class _Props(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 256),
        ("arch", ctypes.c_char * 64),
        ("compute_units", ctypes.c_int),
        ("wave_size", ctypes.c_int),
        ("lds_bytes_per_block", ctypes.c_int),
        ("max_threads_per_block", ctypes.c_int),
        ("regs_per_block", ctypes.c_int),
        ("clock_khz", ctypes.c_int),
        ("mem_clock_khz", ctypes.c_int),
        ("mem_bus_bits", ctypes.c_int),
        ("l2_bytes", ctypes.c_int),
        ("hbm_bytes", ctypes.c_size_t),
    ]


class _LaunchDesc(ctypes.Structure):
    _fields_ = [
        ("mod", ctypes.c_void_p),
        ("grid", ctypes.c_uint * 3),
        ("block", ctypes.c_uint * 3),
        ("lds_bytes", ctypes.c_uint),
        ("args", ctypes.POINTER(ctypes.c_void_p)),
    ]


class _WsBind(ctypes.Structure):
    _fields_ = [
        ("launch", ctypes.c_int),
        ("arg", ctypes.c_int),
        ("offset", ctypes.c_size_t),
        ("bytes", ctypes.c_size_t),
        ("zero", ctypes.c_int),
    ]


STATIC_WS_BYTES = 64 << 20      # FTR_STATIC_WS_BYTES of include/ftrocm.h

_lib = None
_lib_lock = threading.Lock()


def lib():
    """Load libftrocm.so once; raise if it is missing or has the wrong ABI."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError_(
                "libftrocm.so is not built (%s); run `make -C flextensor_amd/csrc` "
                "or __graft_entry__.build()" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.ftr_abi_version.restype = ctypes.c_int
        L.ftr_last_error.restype = ctypes.c_char_p
        L.ftr_compile_to_code.argtypes = [
            ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p),
            ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
            ctypes.POINTER(ctypes.c_size_t)]
        L.ftr_code_free.argtypes = [ctypes.c_void_p]
        L.ftr_code_free.restype = None
        L.ftr_module_load.argtypes = [
            ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p,
            ctypes.POINTER(ctypes.c_void_p)]
        L.ftr_compile.argtypes = [
            ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p),
            ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
        L.ftr_module_free.argtypes = [ctypes.c_void_p]
        L.ftr_module_free.restype = None
        L.ftr_module_attrs.argtypes = [ctypes.c_void_p] + [ctypes.POINTER(ctypes.c_int)] * 4
        L.ftr_launch.argtypes = [
            ctypes.c_void_p, ctypes.c_uint * 3, ctypes.c_uint * 3, ctypes.c_uint,
            ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
        L.ftr_launch_seq.argtypes = [ctypes.POINTER(_LaunchDesc), ctypes.c_int, ctypes.c_void_p]
        L.ftr_launch_seq_static_ws.argtypes = [ctypes.POINTER(_LaunchDesc), ctypes.c_int,
                                               ctypes.POINTER(_WsBind), ctypes.c_int, ctypes.c_void_p]
        L.ftr_time.argtypes = [
            ctypes.c_void_p, ctypes.c_uint * 3, ctypes.c_uint * 3, ctypes.c_uint,
            ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int,
            ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
        L.ftr_time_seq.argtypes = [
            ctypes.POINTER(_LaunchDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
            ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
        L.ftr_time_seq_deadline.argtypes = [
            ctypes.POINTER(_LaunchDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
            ctypes.c_int, ctypes.c_void_p, ctypes.c_double, ctypes.POINTER(ctypes.c_float)]
        L.ftr_stream_idle.argtypes = [ctypes.c_void_p, ctypes.c_double]
        L.ftr_device_props.argtypes = [ctypes.c_int, ctypes.POINTER(_Props)]
        L.ftr_device_count.restype = ctypes.c_int
        if L.ftr_abi_version() != ABI_VERSION:
            raise RuntimeError_("libftrocm.so ABI %d, binding expects %d"
                                % (L.ftr_abi_version(), ABI_VERSION))
        _lib = L
    return _lib


def _check(rc, what):
    if rc != 0:
        msg = lib().ftr_last_error()
        text = "%s: %s" % (what, msg.decode("utf-8", "replace") if msg else "?")
        raise DeviceTimeout(text) if rc == FTR_TIMEOUT else RuntimeError_(text)


def device_count():
    return lib().ftr_device_count()


def device_props(dev=0):
    p = _Props()
    _check(lib().ftr_device_props(dev, ctypes.byref(p)), "ftr_device_props")
    out = {}
    for name, _ in _Props._fields_:
        v = getattr(p, name)
        out[name] = v.decode() if isinstance(v, bytes) else v
    return out


# --------------------------------------------------------------------------
# compile (+ cache)
# --------------------------------------------------------------------------

def _opt_array(opts):
    arr = (ctypes.c_char_p * max(len(opts), 1))()
    for i, o in enumerate(opts):
        arr[i] = o.encode()
    return arr


def code_key(src, opts, arch=DEFAULT_ARCH):
    h = hashlib.sha256()
    h.update(arch.encode())
    h.update(b"\0")
    for o in opts:
        h.update(o.encode())
        h.update(b"\0")
    h.update(src.encode())
    return h.hexdigest()[:32]


_worker = None
_worker_lock = threading.Lock()
WORKER_REPLY_MARK = "FTR-REPLY "


def _stop_worker():
    global _worker
    if _worker is not None:
        try:
            _worker.stdin.close()
            _worker.wait(timeout=5)
        except Exception:  # noqa: BLE001
            _worker.kill()
        _worker = None


def _compile_out_of_process(src, opts, arch):
    """Compile through the compile server (see compile_worker.py)."""
    global _worker
    with _worker_lock:
        if _worker is None or _worker.poll() is not None:
            env = dict(os.environ)
            env["PYTHONPATH"] = os.path.dirname(_HERE) + os.pathsep + env.get("PYTHONPATH", "")
            env["FLEXTENSOR_AMD_KCACHE"] = CACHE_DIR
            _worker = subprocess.Popen([sys.executable, "-m", "flextensor_amd.compile_worker"],
                                       stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                                       universal_newlines=True, env=env)
            atexit.register(_stop_worker)
        _worker.stdin.write(json.dumps({"src": src, "opts": list(opts), "arch": arch,
                                        "cache_dir": CACHE_DIR}) + "\n")
        _worker.stdin.flush()
        while True:
            line = _worker.stdout.readline()
            if not line:
                raise RuntimeError_("compile server died")
            if line.startswith(WORKER_REPLY_MARK):      # anything else is a library's chatter
                break
    rep = json.loads(line[len(WORKER_REPLY_MARK):])
    if not rep.get("ok"):
        raise RuntimeError_("ftr_compile_to_code: %s" % rep.get("error"))
    if "b64" in rep:
        import base64
        return base64.b64decode(rep["b64"])
    with open(rep["path"], "rb") as f:
        return f.read()


def compile_to_code(src, opts=(), arch=DEFAULT_ARCH, use_cache=True, _in_process=False):
    """HIP source -> code object bytes (hiprtc, no device needed).

    Results are cached on disk under CACHE_DIR, keyed by a hash of the source,
    the options and the architecture. When PyTorch is loaded in this process
    the compile runs in the compile server process instead (compile_worker.py)
    so that the ROCm installation's compiler is used, not PyTorch's copy.
    """
    opts = list(opts)
    path = None
    if use_cache:
        path = os.path.join(CACHE_DIR, code_key(src, opts, arch) + ".hsaco")
        if os.path.exists(path):
            with open(path, "rb") as f:
                data = f.read()
            if data:
                return data
    if "torch" in sys.modules and not _in_process:
        return _compile_out_of_process(src, opts, arch)
    code = ctypes.c_void_p()
    size = ctypes.c_size_t()
    rc = lib().ftr_compile_to_code(src.encode(), arch.encode(), _opt_array(opts),
                                   len(opts), ctypes.byref(code), ctypes.byref(size))
    _check(rc, "ftr_compile_to_code")
    try:
        data = ctypes.string_at(code.value, size.value)
    finally:
        lib().ftr_code_free(code)
    if path is not None:
        try:
            os.makedirs(CACHE_DIR, exist_ok=True)
            tmp = path + ".%d.tmp" % os.getpid()
            with open(tmp, "wb") as f:
                f.write(data)
            os.replace(tmp, path)
        except OSError:
            pass
    return data


# --------------------------------------------------------------------------
# kernel arguments
# --------------------------------------------------------------------------

def ptr(x):
    """Device pointer argument from a torch tensor or an int address."""
    if hasattr(x, "data_ptr"):
        return ctypes.c_void_p(x.data_ptr())
    return ctypes.c_void_p(int(x))


def i32(v):
    return ctypes.c_int(int(v))


def f32(v):
    return ctypes.c_float(float(v))


class ArgPack(object):
    """Owns the ctypes values of one launch and the void*[] that points at them."""

    def __init__(self, values):
        self.values = list(values)
        self.array = (ctypes.c_void_p * max(len(self.values), 1))()
        for i, v in enumerate(self.values):
            self.array[i] = ctypes.cast(ctypes.pointer(v), ctypes.c_void_p)

    def as_param(self):
        return ctypes.cast(self.array, ctypes.POINTER(ctypes.c_void_p))


def _u3(v):
    v = tuple(v) + (1,) * (3 - len(v))
    return (ctypes.c_uint * 3)(*[int(x) for x in v])


class Module(object):
    """A loaded code object with one resolved kernel."""

    def __init__(self, code, kernel_name):
        self.kernel_name = kernel_name
        self._h = ctypes.c_void_p()
        self._code = code  # keep the blob alive as long as the module
        rc = lib().ftr_module_load(code, len(code), kernel_name.encode(), ctypes.byref(self._h))
        _check(rc, "ftr_module_load(%s)" % kernel_name)

    @classmethod
    def from_source(cls, src, kernel_name, opts=(), arch=DEFAULT_ARCH):
        return cls(compile_to_code(src, opts, arch), kernel_name)

    @property
    def handle(self):
        return self._h

    def attrs(self):
        v = [ctypes.c_int() for _ in range(4)]
        _check(lib().ftr_module_attrs(self._h, *[ctypes.byref(x) for x in v]), "ftr_module_attrs")
        return {"num_regs": v[0].value, "static_lds_bytes": v[1].value,
                "private_bytes": v[2].value, "max_threads": v[3].value}

    def launch(self, grid, block, args, lds_bytes=0, stream=0):
        pack = args if isinstance(args, ArgPack) else ArgPack(args)
        rc = lib().ftr_launch(self._h, _u3(grid), _u3(block), int(lds_bytes),
                              pack.as_param(), ctypes.c_void_p(stream))
        _check(rc, "ftr_launch(%s)" % self.kernel_name)

    def time(self, grid, block, args, lds_bytes=0, warmup=3, iters=20, stream=0):
        pack = args if isinstance(args, ArgPack) else ArgPack(args)
        ms = ctypes.c_float()
        rc = lib().ftr_time(self._h, _u3(grid), _u3(block), int(lds_bytes), pack.as_param(),
                            int(warmup), int(iters), ctypes.c_void_p(stream), ctypes.byref(ms))
        _check(rc, "ftr_time(%s)" % self.kernel_name)
        return ms.value

    def close(self):
        if self._h:
            lib().ftr_module_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Launch(object):
    """One kernel launch of a plan: module, geometry, packed arguments."""

    def __init__(self, module, grid, block, args, lds_bytes=0):
        self.module = module
        self.grid = tuple(int(x) for x in grid)
        self.block = tuple(int(x) for x in block)
        self.lds_bytes = int(lds_bytes)
        self.pack = args if isinstance(args, ArgPack) else ArgPack(args)

    def fill(self, d):
        d.mod = self.module.handle
        d.grid = _u3(self.grid)
        d.block = _u3(self.block)
        d.lds_bytes = self.lds_bytes
        d.args = self.pack.as_param()


def _desc_array(launches):
    arr = (_LaunchDesc * len(launches))()
    for d, l in zip(arr, launches):
        l.fill(d)
    return arr


def launch_seq(launches, stream=0):
    arr = _desc_array(launches)
    _check(lib().ftr_launch_seq(arr, len(launches), ctypes.c_void_p(stream)), "ftr_launch_seq")


def launch_seq_static_ws(launches, binds, stream=0):
    """``launch_seq`` with the workspace arguments bound to the library's
    static device array instead of caller-owned buffers; allocates nothing.
    ``binds`` = [(launch index, argument index, offset, bytes, zero)]."""
    arr = _desc_array(launches)
    b = (_WsBind * max(len(binds), 1))()
    for dst, (launch, arg, offset, nbytes, zero) in zip(b, binds):
        dst.launch, dst.arg, dst.offset, dst.bytes, dst.zero = int(launch), int(arg), int(offset), int(nbytes), int(zero)
    _check(lib().ftr_launch_seq_static_ws(arr, len(launches), b, len(binds), ctypes.c_void_p(stream)),
           "ftr_launch_seq_static_ws")


def stream_idle(stream=0, timeout=0.0):
    """Wait up to ``timeout`` seconds for the stream to run empty; raises DeviceTimeout if it does not."""
    _check(lib().ftr_stream_idle(ctypes.c_void_p(stream), float(timeout)), "ftr_stream_idle")


def time_seq(sets, warmup=3, iters=20, stream=0, timeout=0.0):
    """Mean ms per iteration; ``sets`` is a list of equally long launch lists
    (one per buffer set) that the timed loop rotates through. ``timeout`` > 0
    is a deadline in seconds for the whole call (DeviceTimeout when it passes)."""
    n_per = len(sets[0])
    flat = []
    for s in sets:
        if len(s) != n_per:
            raise ValueError("all launch sets must have the same length")
        flat.extend(s)
    arr = _desc_array(flat)
    ms = ctypes.c_float()
    rc = lib().ftr_time_seq_deadline(arr, n_per, len(sets), int(warmup), int(iters),
                                     ctypes.c_void_p(stream), float(timeout or 0.0), ctypes.byref(ms))
    _check(rc, "ftr_time_seq")
    return ms.value
