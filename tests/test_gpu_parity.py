"""Device parity: tuned-kernel plans, called through the C-ABI (libftrocm.so),
against the CPU oracle on the same seeded inputs.

Acceptance: fp32  max|out - ref| / max|ref| <= 1e-5 ; int32 bit-exact.
Sizes are chosen so that the oracle finishes in seconds; the five benchmark
configurations are also covered at full size.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available() and os.environ.get("FT_TESTS_COMPILE_ONLY") != "1":
    pytest.skip("no GPU visible", allow_module_level=True)

from flextensor_amd import runtime as rt  # noqa: E402
from flextensor_amd.measure import (Measurer, WrongResult, compare_on_device,  # noqa: E402
                                    run_default_schedule, seeded_inputs)
from flextensor_amd.plan import build, current_stream  # noqa: E402
from flextensor_amd.scheduler import schedule, schedule_with_config  # noqa: E402
from flextensor_amd.task import (TASK_TABLE, Task, register, gemm, gemm_int8, conv2d,  # noqa: E402
                                 depthwise_conv2d)
from flextensor_amd.nn import gemm as op_gemm  # noqa: E402
from flextensor_amd.te import placeholder  # noqa: E402
from flextensor_amd.templates.gfx950 import InvalidConfig, special_knobs  # noqa: E402
from flextensor_amd.utils import Config, ceil_div  # noqa: E402

TOL = 1e-5
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_cases.npz"))
KEYS = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]


def rel(a, b):
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(np.asarray(a, np.float64) - b)) / np.max(np.abs(b)))


def key_of(category, name, args):
    return Task(category, name, None, args, "rocm", 0).key


def gcfg(M, N, K, wm, rm, wn, rn, mf, bk, sk=1, st=2, gm=4, xcd=1, wk=0, ks=0, ls=1):
    """st = pipeline depth; wk=1: the sk K-partitions are wavefront groups of one workgroup;
    ks > 0: balanced K streaming with ks workgroups per compute unit; ls: k blocks over which
    depth 8 spreads the loads of the next tile."""
    c = {k: [] for k in KEYS}
    c["spatial"] = [[ceil_div(M, wm * rm * mf), wm, rm, mf], [ceil_div(N, wn * rn * mf), wn, rn, mf]]
    c["reduce"] = [[sk, K // (sk * bk), bk]]
    c["unroll"], c["fuse"], c["reorder"] = [[st, ls]], [[gm]], [[xcd, wk, ks] if ks else [xcd, wk]]
    return c


def dcfg(b, c, p, q, th, tw, waves):
    cfg = {k: [] for k in KEYS}
    cfg["spatial"] = [[b, 1, 1, 1], [c, 1, 1, 1], [ceil_div(p, th), 1, 1, th], [ceil_div(q, tw), 1, 1, tw]]
    cfg["fuse"] = [[waves]]
    return cfg


def run_plan(key, configs, host_inputs):
    """Lower, build through the C-ABI, run once; returns the output as numpy."""
    s, bufs = schedule_with_config(key, configs)
    func = build(s, bufs, "rocm")
    tdt = {"float32": torch.float32, "int32": torch.int32}[bufs[-1].dtype]
    ins = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in host_inputs]
    out = torch.full(bufs[-1].shape, -77, dtype=tdt, device="cuda")
    func(*ins, out)
    torch.cuda.synchronize()
    func.close()
    return out.cpu().numpy()


def conv_cfgs(op_cfg, inline=None, special=None):
    g = None
    if inline is not None or special is not None:
        g = {k: [] for k in KEYS}
        g["inline"] = [inline if inline is not None else [1, 0]]
        if special is not None:
            g["special"] = special
    return Config([{k: [] for k in KEYS}, op_cfg], g)


# ---------------------------------------------------------------- runtime --

def test_device_is_gfx950_and_library_in_tree():
    p = rt.device_props(0)
    assert p["arch"].startswith("gfx950") and p["wave_size"] == 64
    assert p["lds_bytes_per_block"] == 160 * 1024
    assert os.path.dirname(rt.LIB_PATH).endswith("flextensor_amd")


def test_raw_cabi_launch_and_timing():
    src = ('extern "C" __global__ void axpy(float* y, const float* x, float a, int n)'
           '{ int i = blockIdx.x * 256 + threadIdx.x; if (i < n) y[i] += a * x[i]; }')
    mod = rt.Module.from_source(src, "axpy")
    n = 100003
    x = torch.arange(n, dtype=torch.float32, device="cuda")
    y = torch.ones(n, dtype=torch.float32, device="cuda")
    args = [rt.ptr(y), rt.ptr(x), rt.f32(2.0), rt.i32(n)]
    mod.launch((ceil_div(n, 256),), (256,), args, stream=current_stream())
    torch.cuda.synchronize()
    assert torch.equal(y, 1 + 2 * x)
    ms = mod.time((ceil_div(n, 256),), (256,), args, warmup=1, iters=3, stream=current_stream())
    assert 0 < ms < 10
    assert torch.equal(y, 1 + 2 * 5 * x)  # 1 + 1 + 3 launches in total
    a = mod.attrs()
    assert a["private_bytes"] == 0 and a["num_regs"] > 0
    with pytest.raises(rt.RuntimeError_):
        rt.Module(b"\x7fELFgarbage" + b"\0" * 64, "axpy")
    with pytest.raises(rt.RuntimeError_):
        mod.launch((0,), (256,), args)


def test_shader_clock_is_read_inside_the_kernels():
    """The instrumented build of each template (FT_CLKPROBE) computes the same result and reports
    a plausible sustained clock and workgroup life; the probed plan is a copy, the plan itself is
    left as it was."""
    cases = [("gemm", gemm, (256, 256, 256)), ("gemm", gemm_int8, (256, 256, 256)),
             ("conv2d", depthwise_conv2d, (2, 16, 28, 28, 1, 3, 1, 1, 1)),
             ("conv2d", conv2d, (2, 16, 14, 14, 32, 3, 1, 1, 1, 1))]
    for category, func, args in cases:
        name = {gemm: "gemm", gemm_int8: "gemm_int8", depthwise_conv2d: "depthwise", conv2d: "t"}[func]
        register(func, category, name, args, "rocm", 0)
        key = key_of(category, name, args)
        s, _ = schedule_with_config(key, Config([], None))
        before = [(k.kernel, dict(k.defines), list(k.args)) for k in s.specs]
        probe = s.with_clock_probe()
        assert [(k.kernel, dict(k.defines), list(k.args)) for k in s.specs] == before
        assert probe.specs[-1].defines["CLKPROBE"] == 1 and probe.specs[-1].args[-1] == ("buf", "clk_probe")
        assert "clk_probe" in probe.workspaces and "clk_probe" not in s.workspaces
        m = Measurer(key, seed=4)
        clk = m.shader_clock(s, ms=3.0, warm_ms=30.0)
        assert clk is not None and 0.5 < clk["ghz"] < 2.6 and clk["ghz_min"] <= clk["ghz"] <= clk["ghz_max"]
        assert 0.2 < clk["workgroup_us"] < 1000 and clk["workgroups"] >= 1
        # the same with the counter's own readings: two launches on one time axis
        assert s.with_clock_probe(absolute=True).specs[-1].defines["CLKPROBE"] == 2
        axis = m.time_axis(s, launches=201, warm_ms=30.0)        # odd: rounded down to whole pairs
        # (a grid larger than what the device holds at once may begin its last workgroup after its first has ended)
        assert 0 <= axis["start_skew"] <= axis["last_end"] and 0 < axis["first_end"] <= axis["last_end"] < axis["period"] < 1000
        assert abs(axis["gap"] - (axis["period"] - axis["last_end"])) < 1e-6 and axis["gap"] > 0
        per_launch = m.evaluate(s, number=200, warm_ms=30.0) * 1e3
        assert 0.5 * per_launch < axis["period"] < 2.0 * per_launch + 2.0


def test_time_limit_abandons_an_overrunning_measurement_and_recovers():
    """The per-candidate time limit (flextensor/measure.py:63-74): a measurement that cannot
    finish inside it comes back as DeviceTimeout (-> inf for the search) without anything being
    killed; once the stream has drained the same plan measures normally and is still right."""
    import time
    register(gemm, "gemm", "gemm", (512, 512, 512), "rocm", 0)
    key = key_of("gemm", "gemm", (512, 512, 512))
    s, bufs = schedule_with_config(key, Config([], None))
    m = Measurer(key, seed=2)
    t0 = time.time()
    with pytest.raises(rt.DeviceTimeout):
        # ten million timed launches of a kernel of a few microseconds cannot fit into 0.2 s
        m.evaluate(s, number=10 ** 7, warmup=0, warm_ms=0.0, timeout=0.2)
    assert time.time() - t0 < 20
    rt.stream_idle(current_stream(), 120.0)           # every enqueued kernel finishes by itself
    ms = m.evaluate(s, number=20, timeout=30.0)
    assert 0 < ms < 5
    from flextensor_amd.measure import master_routine, _evaluate
    slow = master_routine(0.2, m.evaluate, s, number=10 ** 7, warmup=0, warm_ms=0.0)
    assert isinstance(slow, rt.DeviceTimeout)
    rt.stream_idle(current_stream(), 120.0)
    fine = master_routine(30.0, _evaluate, s, bufs, "rocm", 0, number=5)
    assert isinstance(fine, float) and 0 < fine < 5


# ------------------------------------------------------- golden fixtures --

def test_golden_gemm_small_ragged():
    a, b = GOLD["gemm_a"], GOLD["gemm_b"]       # 37x64 @ 64x29: ragged M and N
    register(gemm, "gemm", "gemm", (37, 64, 29), "rocm", 0)
    key = key_of("gemm", "gemm", (37, 64, 29))
    for cfg in (None, gcfg(37, 29, 64, 1, 1, 1, 1, 16, 16), gcfg(37, 29, 64, 2, 1, 1, 1, 32, 32),
                gcfg(37, 29, 64, 1, 2, 2, 1, 16, 16, sk=2), gcfg(37, 29, 64, 1, 1, 1, 1, 32, 8, st=1)):
        out = run_plan(key, Config([cfg] if cfg else [], None), [a, b])
        assert rel(out, GOLD["gemm_c"]) <= TOL, cfg


def test_golden_gemm_int8_small_ragged():
    a, b = GOLD["i8_a"], GOLD["i8_b"]           # 19x48 · (23x48)^T, K tail, extreme products
    register(gemm_int8, "gemm", "gemm_int8", (19, 48, 23), "rocm", 0)
    key = key_of("gemm", "gemm_int8", (19, 48, 23))
    for cfg in (None, gcfg(19, 23, 64, 1, 1, 1, 1, 16, 64), gcfg(19, 23, 64, 1, 1, 2, 1, 32, 64),
                gcfg(19, 23, 64, 2, 1, 1, 1, 16, 64, st=1)):
        out = run_plan(key, Config([cfg] if cfg else [], None), [a, b])
        assert np.array_equal(out, GOLD["i8_c"]), cfg
        assert out[0, 0] == 48 * 128 * 128


def test_golden_conv_small():
    x = GOLD["conv_a_x"]                         # [2,5,9,6]; K = 45 -> padded K tail
    for wname, yname, ks, pad in (("conv_a_w", "conv_a_y", 3, 1), ("conv_b_w", "conv_b_y", 1, 0)):
        w = GOLD[wname]
        args = (2, 5, 9, 6, w.shape[0], ks, 1, pad, 1, 1)
        register(conv2d, "conv2d", "t", args, "rocm", 0)
        key = key_of("conv2d", "t", args)
        for inline in (None, [1, 0], [0, 0]):
            if pad == 0 and inline == [0, 0]:
                pass  # a zero-width pad kernel is still a valid copy
            out = run_plan(key, conv_cfgs({}, inline), [x, w])
            assert rel(out, GOLD[yname]) <= TOL, (wname, inline)


def test_golden_conv_grouped_reference_case():
    """The reference's own conv2d test case (flextensor/test/test_ops.py:85-115):
    x [4,6,7,7], w [9,2,3,3], stride 2, padding 1, dilation 2, groups 3."""
    x, w = GOLD["conv_g3_x"], GOLD["conv_g3_w"]
    args = (4, 6, 7, 7, 9, 3, 2, 1, 2, 3)
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    key = key_of("conv2d", "t", args)
    # per group: M = 3, N = 4*3*3 = 36, K = 2*9 = 18 -> 32
    for cfg in ({}, gcfg(3, 36, 32, 1, 1, 1, 1, 16, 16), gcfg(3, 36, 32, 1, 1, 2, 1, 16, 16, sk=2, wk=1),
                gcfg(3, 36, 32, 1, 1, 1, 1, 32, 8, sk=2, st=3)):
        for inline in ([1, 0], [0, 0]):
            out = run_plan(key, conv_cfgs(cfg, inline), [x, w])
            assert out.shape == (4, 9, 3, 3)
            assert rel(out, GOLD["conv_g3_y"]) <= TOL, (cfg, inline)


def test_golden_depthwise_reference_case():
    # the reference's own case: x [4,6,7,7], w [6,3,3,3], stride 2, pad 1, dilation 2
    x, w = GOLD["dw_x"], GOLD["dw_w"]
    args = (4, 6, 7, 7, 3, 3, 2, 1, 2)
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    for cfg in ({}, dcfg(4, 18, 3, 3, 1, 1, 1), dcfg(4, 18, 3, 3, 2, 2, 2), dcfg(4, 18, 3, 3, 3, 1, 4)):
        out = run_plan(key, conv_cfgs(cfg), [x, w])
        assert rel(out, GOLD["dw_y"]) <= TOL, cfg
    x, w = GOLD["dw1_x"], GOLD["dw1_w"]          # [2,5,8,12], 3x3 s1 p1: vector path
    args = (2, 5, 8, 12, 1, 3, 1, 1, 1)
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    for cfg in ({}, dcfg(2, 5, 8, 12, 4, 4, 1), dcfg(2, 5, 8, 12, 7, 4, 2), dcfg(2, 5, 8, 12, 2, 2, 1)):
        for inline in (None, [0, 0]):
            out = run_plan(key, conv_cfgs(cfg, inline), [x, w])
            assert rel(out, GOLD["dw1_y"]) <= TOL, (cfg, inline)


# ------------------------------------------------ seeded inputs vs oracle --

GEMM_CASES = [
    # M, K, N, config knobs
    (256, 256, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=16)),
    (256, 256, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=16, bk=32, sk=2)),
    (256, 256, 256, dict(wm=1, rm=4, wn=4, rn=1, mf=16, bk=64, st=1, gm=1, xcd=0)),
    (200, 136, 328, dict(wm=2, rm=1, wn=1, rn=3, mf=32, bk=8)),      # ragged M, N; N % 4 == 0
    (96, 80, 67, dict(wm=1, rm=1, wn=2, rn=1, mf=16, bk=16)),        # N % 4 != 0 -> scalar loads
    (512, 1024, 128, dict(wm=4, rm=1, wn=1, rn=2, mf=32, bk=32, sk=8, gm=2)),
    (256, 256, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, st=3)),                 # prefetch 2 tiles
    (256, 512, 256, dict(wm=2, rm=2, wn=2, rn=1, mf=16, bk=16, st=4)),                 # prefetch 3 tiles
    (200, 96, 328, dict(wm=1, rm=1, wn=1, rn=2, mf=32, bk=16, st=4)),                  # KT < prefetch + ragged
    (256, 512, 256, dict(wm=1, rm=2, wn=2, rn=1, mf=16, bk=32, sk=4, wk=1, st=3)),     # in-workgroup split-K
    (96, 256, 67, dict(wm=1, rm=1, wn=1, rn=1, mf=32, bk=16, sk=8, wk=1)),             # 8 k-groups, ragged
    (128, 1024, 128, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=32, sk=2, wk=1, st=4)),    # big reduce buffer
    (256, 512, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, ks=1)),                 # K streaming: 16 sharers per tile
    (200, 136, 328, dict(wm=2, rm=1, wn=1, rn=3, mf=32, bk=8, ks=1, st=3)),            # K streaming, ragged
    (512, 1024, 128, dict(wm=2, rm=2, wn=1, rn=2, mf=16, bk=64, ks=2, st=4, gm=2)),    # two workgroups per CU
    (1024, 4096, 1024, dict(wm=4, rm=1, wn=4, rn=1, mf=16, bk=64, ks=1, st=3)),        # whole tiles and shared tiles mixed
]


@pytest.mark.parametrize("M,K,N,kn", GEMM_CASES)
def test_gemm_f32_vs_oracle(oracle, M, K, N, kn):
    register(gemm, "gemm", "gemm", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm", (M, K, N))
    ops, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=M + N)
    kp = ceil_div(K, 16) * 16
    out = run_plan(key, Config([gcfg(M, N, kp, **kn)], None), [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL
    assert rel(out, oracle.gemm_f32_c(a, b)) <= TOL


def test_k_streaming_plan_is_reusable_and_deterministic(oracle):
    """The arrival counters return to zero inside the kernel, so one built plan
    serves any number of launches; the slots are summed in a fixed order, so
    equal inputs give bit-equal outputs."""
    M, K, N = 320, 768, 192
    register(gemm, "gemm", "gemm", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm", (M, K, N))
    ops, bufs = TASK_TABLE[key].func(M, K, N)
    cfg = Config([gcfg(M, N, K, wm=2, rm=1, wn=2, rn=1, mf=16, bk=32, ks=1, st=3)], None)
    s, bufs = schedule_with_config(key, cfg)
    assert s.workspaces and s.specs[-1].defines["SK_PER"] >= 1
    func = build(s, bufs, "rocm")
    outs = []
    for seed in (1, 2, 1, 1):
        a, b = seeded_inputs(bufs, seed=seed)
        out = torch.full((M, N), -77.0, device="cuda")
        func(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), out)
        torch.cuda.synchronize()
        assert rel(out.cpu().numpy(), oracle.gemm_np(a, b)) <= TOL, seed
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[2]) and np.array_equal(outs[0], outs[3])
    assert int(func.scratch["out_count"].abs().sum().item()) == 0
    func.close()
    # the hand-off as a device-scope release / acquire on the counter (a task opts in): the same
    # sums in the same order, so the same bits
    TASK_TABLE[key].set_specific_space("sk_fenced", "enum", [[1]])
    try:
        g = {k: [] for k in KEYS}
        g["special"] = [[-1, -1], [1]]
        assert list(TASK_TABLE[key].special_space)[-1] == "sk_fenced"
        fenced = Config(cfg.op_config_lst, g)
        s2, _ = schedule_with_config(key, fenced)
        assert s2.specs[-1].defines["SK_FENCED"] == 1 and "SK_FENCED" not in s.specs[-1].defines
        a, b = seeded_inputs(bufs, seed=1)
        assert np.array_equal(run_plan(key, fenced, [a, b]), outs[0])
    finally:
        TASK_TABLE[key].special_space.pop("sk_fenced", None)


def test_grid_level_split_k_repeats_within_a_few_ulp(oracle):
    """K parts that meet in C through float atomics (after a zero fill) add in the order the
    workgroups happen to arrive, so the last bits move from run to run. The bound: every run within
    1e-5 of the oracle like any other plan, and any two runs within 2e-6 of max|ref| of each other
    (16 partial sums of magnitude <= max|ref| each, a few ulp of reordering); K streaming and the
    in-workgroup split, which add in a fixed order, repeat exactly."""
    M, K, N = 256, 4096, 192
    register(gemm, "gemm", "gemm", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm", (M, K, N))
    _, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=12)
    ref = oracle.gemm_np(a, b)
    scale = float(np.max(np.abs(ref)))
    for kn, exact in ((dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, sk=16), False),
                      (dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=32, sk=4, wk=1), True),
                      (dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, ks=1, st=3), True)):
        s, _ = schedule_with_config(key, Config([gcfg(M, N, K, **kn)], None))
        assert (s.specs[0].kernel == "fill_zero_f32") == (not exact)
        outs = [run_plan(key, Config([gcfg(M, N, K, **kn)], None), [a, b]) for _ in range(6)]
        for o in outs:
            assert rel(o, ref) <= TOL
        spread = max(float(np.max(np.abs(o.astype(np.float64) - outs[0]))) for o in outs[1:]) / scale
        if exact:
            assert spread == 0.0, kn
        else:
            assert spread <= 2e-6, spread


@pytest.mark.parametrize("M,K,N,kn,pad", [
    (256, 256, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, st=5), [-1, -1]),            # swizzled A rows
    (256, 512, 256, dict(wm=4, rm=1, wn=4, rn=1, mf=16, bk=64, st=5), [-1, 4]),
    (200, 136, 328, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=8, st=5), [0, 8]),               # ragged M, N; padded K
    (320, 768, 192, dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=32, st=5, ks=1), [-1, -1]),      # with K streaming
    (96, 144, 128, dict(wm=1, rm=1, wn=1, rn=2, mf=32, bk=72, st=5), [0, 0]),               # partial last round of chunks
    (200, 136, 328, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=8, st=5), [0, 0]),               # B in swizzled 16-byte chunks, ragged
    (256, 256, 512, dict(wm=2, rm=2, wn=2, rn=4, mf=16, bk=32, st=5), [-1, -1]),            # same, 128-wide tile
    (96, 144, 128, dict(wm=1, rm=1, wn=1, rn=2, mf=32, bk=72, st=5), [-1, 0]),              # 18 chunks a row: XOR of the low chunk bit
    (128, 288, 128, dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=48, st=5), [-1, -1]),            # 12 chunks a row: XOR of two bits
    (128, 288, 64, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=144, st=5), [-1, 0]),             # 36 chunks a row
    (128, 240, 64, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=40, st=5), [-1, 0]),              # 10 chunks a row
    # three and four buffers: two and three tiles requested ahead
    (256, 512, 256, dict(wm=4, rm=1, wn=4, rn=1, mf=16, bk=64, st=6), [-1, -1]),
    (256, 512, 256, dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=32, st=7), [-1, -1]),
    (256, 64, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, st=7), [-1, -1]),             # fewer tiles than buffers
    (200, 136, 328, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=16, st=6), [0, 0]),               # ragged, padded K, odd tile count
    (320, 768, 192, dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=32, st=6, ks=1), [-1, -1]),      # with K streaming: segments of any length
    (320, 768, 192, dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=32, st=7, ks=2), [-1, -1]),
    # depth 8: two buffers, the next tile's first operands read behind the barrier, ahead of the last MFMAs
    (256, 256, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, st=8), [-1, -1]),
    (200, 136, 328, dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=8, st=8), [0, 8]),               # one k block per tile, ragged, padded K
    (256, 64, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=16, bk=64, st=8), [-1, -1]),             # a single tile
    (128, 288, 128, dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=48, st=8), [-1, -1]),            # three k blocks per tile
    (320, 768, 192, dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=32, st=8, ks=1), [-1, -1]),      # K streaming: segments of any length
    (256, 512, 256, dict(wm=1, rm=2, wn=2, rn=1, mf=16, bk=32, sk=4, wk=1, st=8), [-1, -1]),  # four k-groups in the workgroup
    (128, 288, 128, dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=48, st=8, ls=2), [-1, -1]),      # the next tile's loads in two parts
    (200, 512, 136, dict(wm=2, rm=1, wn=1, rn=2, mf=32, bk=64, st=8, ls=7), [-1, 0]),        # in seven parts, more parts than loads, ragged
])
def test_gemm_f32_direct_to_lds(oracle, M, K, N, kn, pad):
    """Pipeline depths 5 to 7: tiles travel global -> LDS without staging registers."""
    register(gemm, "gemm", "gemm", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm", (M, K, N))
    ops, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=M + N)
    kp = K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[0]], [pad]
    s, _ = schedule_with_config(key, Config([gcfg(M, N, kp, **kn)], g))
    assert s.specs[-1].defines["DTL"] == 1
    out = run_plan(key, Config([gcfg(M, N, kp, **kn)], g), [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL


@pytest.mark.parametrize("M,K,N,kn", [
    (128, 288, 128, dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=48, st=3)),     # 12 chunks a row
    (200, 216, 136, dict(wm=2, rm=1, wn=1, rn=2, mf=32, bk=72, st=2)),     # 18 chunks, ragged M and N
    (128, 240, 64, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=40, st=4)),      # 10 chunks
])
def test_gemm_f32_swizzled_rows_of_any_even_length(oracle, M, K, N, kn):
    """lds_pad -1 on the register-staged pipelines: unpadded A rows whose chunk
    index is XOR-ed by the row, also when the row is not a power of two long."""
    register(gemm, "gemm", "gemm", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm", (M, K, N))
    ops, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=M + N)
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[0]], [[-1, -1]]
    s, _ = schedule_with_config(key, Config([gcfg(M, N, K, **kn)], g))
    assert s.specs[-1].defines["APAD"] == -1
    out = run_plan(key, Config([gcfg(M, N, K, **kn)], g), [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL


def test_gemm_transpose_b_direct_to_lds(oracle):
    def wrap(M, K, N):
        A = placeholder((M, K), name="A")
        B = placeholder((N, K), name="B")
        C = op_gemm(A, B, transposeB=True)
        return [C.op], [A, B, C]
    register(wrap, "gemm", "gemm_nt", (160, 96, 224), "rocm", 0)
    key = key_of("gemm", "gemm_nt", (160, 96, 224))
    TASK_TABLE[key].set_specific_space("lds_pad", "enum", [[-1, -1]])
    _, bufs = wrap(160, 96, 224)
    a, b = seeded_inputs(bufs, seed=9)
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[0]], [[-1, -1]]
    out = run_plan(key, Config([gcfg(160, 224, 96, 2, 1, 2, 1, 32, 32, st=5)], g), [a, b])
    assert rel(out, oracle.gemm_f32_c(a, b, transB=True)) <= TOL


@pytest.mark.parametrize("args,kn,pad", [
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=16, st=5), [-1, 8]),
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, st=5), [0, 0]),     # groups, hoisted gather
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, st=5), [-1, 0]),    # same, rows of 18 chunks swizzled
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=48, sk=4, wk=1, st=5), [-1, 0]),  # 12 chunks, 4 k-groups
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=144, st=5, ks=1), [-1, 0]),   # 36 chunks, K streaming
    ((1, 8, 17, 13, 24, 3, 2, 1, 1, 1), dict(wm=1, rm=2, wn=4, rn=1, mf=16, bk=16, st=5), [-1, 4]),     # stride 2, K tail
    ((3, 8, 11, 11, 20, 3, 1, 2, 2, 1), dict(wm=1, rm=2, wn=2, rn=2, mf=16, bk=16, st=5, ks=1), [-1, 4]),   # dilation, K streaming
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, st=5), [-1, 8]),      # 1x1, N=392
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=16, sk=4, wk=1, st=5), [0, 0]),   # BN=16, 4 k-groups
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=32, bk=72, sk=2, wk=1, st=5), [0, 0]),   # BN=32, whole windows
    # K streaming with whole tiles between two shared ones: the tile store reads the
    # accumulators right after the last MFMA (the store once came 19 issue slots too early)
    ((8, 512, 7, 7, 2048, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64, st=5, ks=1), [-1, 0]),
    ((8, 512, 7, 7, 2048, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=32, st=2, ks=1), [-1, 0]),
    # three and four buffers
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=16, st=6), [-1, 8]),
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=1, rn=1, mf=32, bk=72, st=6), [0, 0]),
    ((8, 512, 7, 7, 2048, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=32, st=7, ks=1), [-1, 0]),
    # the same in workgroups of one wavefront (the ring's buffer index once reached the
    # load instruction in a vector register there, and the kernel did not assemble)
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=2, wn=1, rn=5, mf=16, bk=16, st=7), [-1, 0]),
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=1, rn=3, mf=32, bk=16, st=6), [-1, 0]),
    ((2, 32, 16, 16, 64, 3, 1, 0, 1, 4), dict(wm=1, rm=1, wn=1, rn=4, mf=16, bk=16, st=6), [-1, 0]),
    # unpadded B rows permuted against bank conflicts: every row width / MFMA shape of the permutation
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=16, st=5), [-1, 0]),    # 32 floats, 16x16x4
    ((2, 16, 14, 14, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=4, rn=1, mf=16, bk=16, st=5), [-1, 0]),    # 64 floats, 16x16x4
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=2, rn=2, mf=32, bk=16, st=5), [-1, 0]),    # 128 floats, 32x32x2
    ((1, 8, 17, 13, 24, 3, 2, 1, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16, st=5), [-1, 0]),     # 16 floats, stride 2, K tail
    # rows that neither divide nor are multiples of 64 floats: the tile lands flat, not permuted
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=1, rn=5, mf=16, bk=32, st=5), [-1, 0]),      # 80 floats, N=392
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=1, rn=3, mf=16, bk=16, st=5), [0, 0]),     # 48 floats
    # depth 8 (operands of the next tile read ahead of the last MFMAs)
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, st=8), [-1, 0]),    # groups, whole windows
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=144, st=8), [0, 0]),    # 16 columns, four tiles of 144
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=32, st=8), [-1, 0]),      # 1x1, N=392
    ((3, 8, 11, 11, 20, 3, 1, 2, 2, 1), dict(wm=1, rm=2, wn=2, rn=2, mf=16, bk=16, st=8, ks=1), [-1, 4]),   # dilation, K tail, K streaming
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=144, st=8, ks=1), [-1, 0]),  # 36 chunks, K streaming
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=144, st=8, ls=6), [-1, 0]),   # loads spread over six k blocks
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=144, st=8, ks=1, ls=4), [-1, 0]),  # the same with K streaming
])
def test_conv2d_direct_to_lds(oracle, args, kn, pad):
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    key = key_of("conv2d", "t", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    ref = oracle.conv2d_nchw_c(x, w, st, pd, dl, g)
    M, N, K = ko // g, nb * ref.shape[2] * ref.shape[3], (c // g) * ks * ks
    kp = K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16
    cfg = gcfg(M, N, kp, **kn)
    for inline in ([1, 0], [0, 0]):
        out = run_plan(key, conv_cfgs(cfg, inline, [pad]), [x, w])
        assert rel(out, ref) <= TOL, inline


def _conv_bias(N, C, H, W, K, k, stride=1, padding=0, dilation=1, groups=1):
    from flextensor_amd.nn import conv2d_nchw
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, k, k), name="W")
    bias = placeholder((K,), name="bias")
    Out = conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Out.op], [Img, Wt, bias, Out]


@pytest.mark.parametrize("args,kn,pad", [
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=16), [4, -1]),
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=16, sk=3), [4, -1]),          # grid split-K: bias once
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=32, sk=2, wk=1, st=4), [4, -1]),   # in-workgroup split
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, ks=1, st=5), [0, 0]),      # groups, K streaming, straight into LDS
    ((4, 6, 7, 7, 9, 3, 2, 1, 2, 3), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16), [4, -1]),                    # the reference's test case
])
def test_conv2d_with_bias(oracle, args, kn, pad):
    """[Padding, conv, bias]: bias merged into the convolution's epilogue, and as its own kernel."""
    register(_conv_bias, "conv2d", "bias", args, "rocm", 0)
    key = key_of("conv2d", "bias", args)
    TASK_TABLE[key].set_specific_space("lds_pad", "enum", [pad])
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w, bias = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    ref = oracle.bias_add_nchw_np(oracle.conv2d_nchw_c(x, w, st, pd, dl, g), bias)
    M, N, K = ko // g, nb * ref.shape[2] * ref.shape[3], (c // g) * ks * ks
    kp = K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16
    cfg = gcfg(M, N, kp, **kn)
    for merge in ([0, 0, 1], [0, 0, 0]):
        gc = {k: [] for k in KEYS}
        gc["inline"], gc["merge"], gc["special"] = [[1, 0, 0]], [merge], [pad]
        configs = Config([{k: [] for k in KEYS}, cfg, {k: [] for k in KEYS}], gc)
        s, _ = schedule_with_config(key, configs)
        assert ("bias_add_nchw_f32" in [x_.kernel for x_ in s.specs]) == (merge[2] == 0)
        out = run_plan(key, configs, [x, w, bias])
        assert rel(out, ref) <= TOL, merge
    # the default-schedule kernels of the three-stage graph
    dev = [torch.from_numpy(a).cuda() for a in (x, w, bias)]
    out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
    run_default_schedule(ops, dev + [out], stream=current_stream())
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), ref) <= TOL


def _depthwise_bias(N, C, H, W, factor, k, stride=1, padding=0, dilation=1):
    from flextensor_amd.nn import depthwise_conv2d_nchw
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((C, factor, k, k), name="W")
    bias = placeholder((C * factor,), name="bias")
    Out = depthwise_conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation)
    return [Out.op], [Img, Wt, bias, Out]


def test_depthwise_and_one_channel_groups_with_bias(oracle):
    """[Padding, depthwise, bias] (flextensor/nn/ops.py:673-677): the bias is added in the stores of
    the depthwise kernel (merge 1, the default) or runs as its own kernel behind it (merge 0), in
    every variant of the kernel; conv2d_nchw with groups = channels and a bias builds the same graph."""
    for args in ((2, 6, 12, 16, 1, 3, 1, 1, 1), (1, 4, 14, 16, 6, 3, 2, 1, 1)):
        register(_depthwise_bias, "conv2d", "dw_bias", args, "rocm", 0)
        key = key_of("conv2d", "dw_bias", args)
        for name, knobs in special_knobs("depthwise_conv2d_nchw").items():
            TASK_TABLE[key].set_specific_space(name, "enum", knobs)
        ops, bufs = TASK_TABLE[key].func(*args)
        x, w, bias = seeded_inputs(bufs, seed=sum(args))
        ref = oracle.bias_add_nchw_np(oracle.depthwise_nchw_c(x, w, args[6], args[7], args[8]), bias)
        b_, co, p, q = ref.shape
        s, _ = schedule_with_config(key, Config([], None))
        assert [k.kernel for k in s.specs] == ["depthwise_f32"] and s.specs[0].defines["HAS_BIAS"] == 1
        assert rel(run_plan(key, Config([], None), [x, w, bias]), ref) <= TOL
        none = {k: [] for k in KEYS}
        for merge in (0, 1):
            # special: nt_store, halo_shfl, lds_planes, lane_items, row_exchange, kernel_fuse
            variants = [[[0], [0], [0], [1], [0], [1]], [[1], [0], [0], [2], [0], [0]]]
            if args[4] == 1 and args[6] == 1:
                variants += [[[0], [1], [0], [1], [0], [1]],      # shuffled halo
                             [[0], [0], [2], [1], [0], [1]],      # planes staged through LDS
                             [[1], [0], [0], [1], [2], [1]]]      # row exchange
            for special in variants:
                gc = {k: [] for k in KEYS}
                gc["inline"], gc["merge"], gc["special"] = [[1, 0, 0]], [[0, 0, merge]], special
                configs = Config([none, dcfg(b_, co, p, q, 2, 4, 2), none], gc)
                s, _ = schedule_with_config(key, configs)
                want = ["depthwise_f32"] if merge else ["depthwise_f32", "bias_add_nchw_f32"]
                assert [k.kernel for k in s.specs] == want
                assert rel(run_plan(key, configs, [x, w, bias]), ref) <= TOL, (merge, special)
        dev = [torch.from_numpy(a).cuda() for a in (x, w, bias)]
        out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
        run_default_schedule(ops, dev + [out], stream=current_stream())
        torch.cuda.synchronize()
        assert rel(out.cpu().numpy(), ref) <= TOL
    args = (2, 6, 12, 16, 12, 3, 1, 1, 1, 6)       # conv2d, groups = channels, two kernels per channel
    register(_conv_bias, "conv2d", "bias", args, "rocm", 0)
    key = key_of("conv2d", "bias", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w, bias = seeded_inputs(bufs, seed=sum(args))
    ref = oracle.bias_add_nchw_np(oracle.conv2d_nchw_c(x, w, 1, 1, 1, 6), bias)
    s, _ = schedule_with_config(key, Config([], None))
    assert [k.kernel for k in s.specs] == ["depthwise_f32"]
    assert rel(run_plan(key, Config([], None), [x, w, bias]), ref) <= TOL


def _gemm_conv_bias(N, C, H, W, K, k, stride=1, padding=0, dilation=1, groups=1):
    from flextensor_amd.nn import gemm_conv2d_nchw
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, k, k), name="W")
    bias = placeholder((K,), name="bias")
    Out = gemm_conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Out.op], [Img, Wt, bias, Out]


@pytest.mark.parametrize("args,kn,pad,with_bias", [
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=16), [4, -1], False),
    ((1, 384, 27, 27, 64, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=32, st=3), [-1, -1], True),   # the reference's test case
    ((4, 6, 11, 9, 9, 3, 2, 1, 2, 3), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16), [4, -1], True),            # groups, stride, dilation, K tail
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, st=5, ks=1), [0, 0], False),   # straight into LDS, K streaming
    ((1, 16, 14, 14, 48, 3, 1, 1, 1, 2), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=8, sk=3, st=3), [4, -1], False),  # one image, groups, split K
])
def test_gemm_conv2d_vs_oracle(oracle, args, kn, pad, with_bias):
    """[Padding, Img2Col, ComputeGemm, (ComputeBias,) Col2Img] under every
    combination of graph flags that has a kernel sequence: from one implicit
    GEMM kernel to pad, im2col, batched GEMM, bias, col2img as five kernels;
    intermediates are checked through the final result."""
    from flextensor_amd.task import gemm_conv2d
    from flextensor_amd.templates.gfx950 import InvalidConfig
    func = _gemm_conv_bias if with_bias else gemm_conv2d
    register(func, "gemm_conv2d", "t", args, "rocm", 0, override=True)
    key = key_of("gemm_conv2d", "t", args)
    TASK_TABLE[key].set_specific_space("lds_pad", "enum", [pad])
    ops, bufs = TASK_TABLE[key].func(*args)
    host = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    x, w = host[0], host[1]
    bias = host[2] if with_bias else None
    ref = oracle.gemm_conv2d_nchw_np(x, w, bias, st, pd, dl, g)[0]
    direct = oracle.conv2d_nchw_c(x, w, st, pd, dl, g)
    if with_bias:
        direct = oracle.bias_add_nchw_np(direct, bias)
    assert rel(direct, ref) <= 1e-6
    M, N, K = ko // g, nb * ref.shape[2] * ref.shape[3], (c // g) * ks * ks
    kp = K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16
    cfg = gcfg(M, N, kp, **kn)
    nops = 5 if with_bias else 4
    empty = {k: [] for k in KEYS}
    op_cfgs = [dict(empty), dict(empty), cfg] + [dict(empty)] * (nops - 3)
    ran = 0
    for pad_in in (1, 0):
        for col_in in (1, 0):
            for bias_m in ((1, 0) if with_bias else (0,)):
                for img_m in (1, 0):
                    gc = {k: [] for k in KEYS}
                    gc["inline"] = [[pad_in, col_in] + [0] * (nops - 2)]
                    gc["merge"] = [[0, 0, 0] + ([bias_m] if with_bias else []) + [img_m]]
                    gc["special"] = [pad]
                    configs = Config(op_cfgs, gc)
                    try:
                        plan, _ = schedule_with_config(key, configs)
                    except InvalidConfig:
                        # col2img merges only behind a merged bias, and into the GEMM over stored
                        # columns only for one image (where [groups][M][P*Q] is NCHW already)
                        assert img_m == 1 and ((col_in == 0 and nb > 1) or (with_bias and bias_m == 0)), gc
                        continue
                    kernels = [k_.kernel for k_ in plan.specs]
                    assert ("zero_pad2d_f32" in kernels) == (pad_in == 0)
                    assert ("im2col_nchw_f32" in kernels) == (col_in == 0)
                    assert ("col2img_nchw_f32" in kernels) == (img_m == 0)
                    if with_bias:
                        assert ("bias_add_nchw_f32" in kernels) == (bias_m == 0)
                    out = run_plan(key, configs, list(host))
                    assert rel(out, ref) <= TOL, (gc["inline"], gc["merge"], kernels)
                    ran += 1
    assert ran == (10 if with_bias else 6) + ((2 if with_bias else 2) if nb == 1 else 0)
    # untuned replay and the default-schedule reference of the correctness gate
    out = run_plan(key, Config([], None), list(host))
    assert rel(out, ref) <= TOL
    dev = [torch.from_numpy(a).cuda() for a in host]
    out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
    run_default_schedule(ops, dev + [out], stream=current_stream())
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("args,kn,pad", [
    ((5, 96, 80, 67), dict(wm=1, rm=1, wn=2, rn=1, mf=16, bk=16), [4, -1]),                  # ragged, scalar B loads
    ((3, 200, 136, 328), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=8, st=3), [-1, -1]),
    ((4, 128, 256, 128), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=32, sk=2), [4, -1]),          # grid split-K atomics
    ((4, 128, 512, 128), dict(wm=1, rm=2, wn=2, rn=2, mf=16, bk=32, ks=1, st=5), [-1, -1]),   # K streaming, straight into LDS
    ((7, 64, 64, 64), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=16, sk=2, wk=1), [4, -1]),       # k-groups
])
def test_batch_gemm_vs_oracle(oracle, args, kn, pad):
    """C[b] = A[b] @ B[b]: the batch index is the kernel's group index."""
    from flextensor_amd.task import batch_gemm
    register(batch_gemm, "gemm", "batch_gemm", args, "rocm", 0)
    key = key_of("gemm", "batch_gemm", args)
    nb, M, K, N = args
    ops, bufs = TASK_TABLE[key].func(*args)
    a, b = seeded_inputs(bufs, seed=sum(args))
    ref = np.stack([oracle.gemm_f32_c(a[i], b[i]) for i in range(nb)])
    assert rel(ref, np.matmul(a.astype(np.float64), b.astype(np.float64))) <= TOL
    kp = K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[0]], [pad]
    for cfg in (Config([], None), Config([gcfg(M, N, kp, **kn)], g)):
        out = run_plan(key, cfg, [a, b])
        assert rel(out, ref) <= TOL
    dev = [torch.from_numpy(x).cuda() for x in (a, b)]
    out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
    run_default_schedule(ops, dev + [out], stream=current_stream())
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), ref) <= TOL


def test_batch_gemm_transposed_operands_vs_oracle(oracle):
    """batch_gemm with A stored [b,k,i] and / or B stored [b,j,k] (flextensor/nn/ops.py:1131-1145)."""
    from flextensor_amd.nn import batch_gemm as op_batch_gemm
    nb, M, K, N = 3, 40, 48, 72
    for ta, tb in ((True, False), (True, True), (False, True)):
        def wrap(nb, M, K, N, ta=ta, tb=tb):
            A = placeholder((nb, K, M) if ta else (nb, M, K), name="A")
            B = placeholder((nb, N, K) if tb else (nb, K, N), name="B")
            C = op_batch_gemm(A, B, transposeA=ta, transposeB=tb)
            return [C.op], [A, B, C]
        name = "batch_gemm_%d%d" % (ta, tb)
        register(wrap, "gemm", name, (nb, M, K, N), "rocm", 0)
        key = key_of("gemm", name, (nb, M, K, N))
        ops, bufs = wrap(nb, M, K, N)
        a, b = seeded_inputs(bufs, seed=5)
        ref = np.stack([oracle.gemm_f32_c(a[i], b[i], transA=ta, transB=tb) for i in range(nb)])
        a64 = a.astype(np.float64).transpose(0, 2, 1) if ta else a.astype(np.float64)
        b64 = b.astype(np.float64).transpose(0, 2, 1) if tb else b.astype(np.float64)
        assert rel(ref, np.matmul(a64, b64)) <= TOL
        for cfg in (Config([], None), Config([gcfg(M, N, K, 1, 1, 2, 1, 16, 16, st=3)], None)):
            out = run_plan(key, cfg, [a, b])
            assert rel(out, ref) <= TOL, (ta, tb)
        dev = [torch.from_numpy(x).cuda() for x in (a, b)]
        out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
        run_default_schedule(ops, dev + [out], stream=current_stream())
        torch.cuda.synchronize()
        assert rel(out.cpu().numpy(), ref) <= TOL


def test_gemm_transpose_b_vs_oracle(oracle):
    def wrap(M, K, N):
        A = placeholder((M, K), name="A")
        B = placeholder((N, K), name="B")
        C = op_gemm(A, B, transposeB=True)
        return [C.op], [A, B, C]
    register(wrap, "gemm", "gemm_nt", (160, 96, 224), "rocm", 0)
    key = key_of("gemm", "gemm_nt", (160, 96, 224))
    _, bufs = wrap(160, 96, 224)
    a, b = seeded_inputs(bufs, seed=9)
    for cfg in (None, gcfg(160, 224, 96, 2, 1, 2, 1, 32, 16), gcfg(160, 224, 96, 1, 2, 2, 2, 16, 32, sk=3)):
        out = run_plan(key, Config([cfg] if cfg else [], None), [a, b])
        assert rel(out, oracle.gemm_f32_c(a, b, transB=True)) <= TOL


def test_gemm_transpose_a_vs_oracle(oracle):
    """The transposeA branches (flextensor/nn/ops.py:1093-1100): A stored [K][M], with B stored
    either way; ragged M (vector and scalar transposing loads), split K, default config."""
    for (M, K, N), tb in (((160, 96, 224), False), ((160, 96, 224), True), ((50, 72, 90), False),
                          ((37, 64, 29), True)):
        def wrap(M, K, N, tb=tb):
            A = placeholder((K, M), name="A")
            B = placeholder((N, K) if tb else (K, N), name="B")
            C = op_gemm(A, B, transposeA=True, transposeB=tb)
            return [C.op], [A, B, C]
        name = "gemm_t%s" % ("t" if tb else "n")
        register(wrap, "gemm", name, (M, K, N), "rocm", 0)
        key = key_of("gemm", name, (M, K, N))
        ops, bufs = wrap(M, K, N)
        assert bufs[-1].shape == (M, N)
        a, b = seeded_inputs(bufs, seed=M + K)
        ref = oracle.gemm_f32_c(a, b, transA=True, transB=tb)
        assert rel(ref, a.astype(np.float64).T @ (b.astype(np.float64).T if tb else b.astype(np.float64))) < 1e-5
        kp = ceil_div(K, 16) * 16
        cfgs = [None, gcfg(M, N, kp, 2, 1, 2, 1, 16, 16, st=3), gcfg(M, N, kp, 1, 2, 1, 1, 32, 16, st=1)]
        if kp % 48 == 0:
            cfgs.append(gcfg(M, N, kp, 1, 2, 2, 2, 16, 16, sk=3, st=2))
        for cfg in cfgs:
            out = run_plan(key, Config([cfg] if cfg else [], None), [a, b])
            assert rel(out, ref) <= TOL, (M, K, N, tb, cfg)
        with pytest.raises(Exception):      # tiles straight into LDS: a transposed A needs tile rows of 64 floats
            schedule_with_config(key, Config([gcfg(M, N, kp, 2, 1, 2, 1, 16, 16, st=5)], None))
        if M % 4 == 0:
            # tiles straight into LDS: the [K][M] tile lands as it lies in memory, fragments read as scalars
            dtl = [gcfg(M, N, kp, 4, 1, 2, 1, 16, 16, st=5), gcfg(M, N, kp, 2, 1, 1, 2, 32, 32, st=8),
                   gcfg(M, N, kp, 2, 2, 2, 1, 16, 32, st=6), gcfg(M, N, kp, 4, 1, 4, 1, 16, 32, st=8)]
            for cfg in dtl:
                out = run_plan(key, Config([cfg], None), [a, b])       # default LDS layout: swizzled, unpadded rows
                assert rel(out, ref) <= TOL, (M, K, N, tb, cfg)
        # and the default-schedule kernel the search checks candidates against
        dev = [torch.from_numpy(x).cuda() for x in (a, b)]
        out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
        run_default_schedule(ops, dev + [out], stream=current_stream())
        torch.cuda.synchronize()
        assert rel(out.cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("M,K,N,kn", [
    (256, 256, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=64)),
    (256, 512, 384, dict(wm=1, rm=4, wn=2, rn=2, mf=16, bk=128, st=1)),
    (136, 208, 72, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64)),      # ragged everywhere, K tail
    (512, 256, 512, dict(wm=2, rm=4, wn=2, rn=4, mf=32, bk=128, gm=2, xcd=0)),
    (512, 512, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=128, st=5)),      # fragment-prefetch pipeline
    (200, 320, 136, dict(wm=2, rm=2, wn=1, rn=2, mf=16, bk=64, st=5)),       # same, ragged, one k-step per tile
    (256, 64, 256, dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=64, st=5)),        # same, a single tile
    (256, 768, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=128, st=4)),      # prefetch 3 tiles
    (512, 512, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=128, st=6)),      # tiles straight into LDS
    (200, 336, 136, dict(wm=2, rm=2, wn=1, rn=4, mf=16, bk=64, st=6)),       # same, ragged M, N and K tail
    (256, 64, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=16, bk=64, st=6)),        # same, a single tile
    (512, 512, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=128, st=7)),      # straight into LDS + fragment prefetch
    (200, 336, 136, dict(wm=2, rm=2, wn=1, rn=4, mf=16, bk=64, st=7)),       # same, ragged, one step per tile
    (256, 64, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=16, bk=64, st=7)),        # same, a single tile
    (512, 1024, 512, dict(wm=4, rm=1, wn=4, rn=1, mf=16, bk=256, st=7)),     # same, 16 wavefronts, four steps per tile
    (512, 512, 512, dict(wm=2, rm=4, wn=2, rn=4, mf=16, bk=128, st=8)),      # written-out instruction order, four tiles
    (200, 336, 136, dict(wm=2, rm=4, wn=1, rn=4, mf=16, bk=128, st=8)),      # same, ragged M and N, K tail, three tiles
    (256, 128, 256, dict(wm=2, rm=4, wn=2, rn=4, mf=16, bk=128, st=8)),      # same, a single tile
    (256, 256, 256, dict(wm=2, rm=4, wn=2, rn=4, mf=16, bk=128, st=8)),      # same, two tiles
    (512, 512, 256, dict(wm=2, rm=2, wn=2, rn=4, mf=32, bk=64, st=8)),       # same, 32x32x32, two k-steps per tile
])
def test_gemm_int8_vs_oracle(oracle, M, K, N, kn):
    _gemm_int8_case(oracle, M, K, N, kn, None)


@pytest.mark.parametrize("M,K,N,kn,store", [
    (136, 208, 72, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64), 2),           # 128-bit row stores, ragged
    (200, 320, 136, dict(wm=2, rm=2, wn=1, rn=2, mf=16, bk=64, st=5), 2),
    (256, 512, 384, dict(wm=1, rm=4, wn=2, rn=2, mf=16, bk=128), 3),         # same, non-temporal
    (512, 256, 512, dict(wm=2, rm=4, wn=2, rn=4, mf=32, bk=128, gm=2), 3),
    # bit 2: the last tile block by block, every block stored as soon as it is complete
    (512, 512, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=64, st=7), 4),        # eight tiles, 32x32x32
    (200, 336, 136, dict(wm=2, rm=2, wn=1, rn=4, mf=16, bk=128, st=7), 4),       # ragged M and N, K tail, three tiles
    (256, 256, 256, dict(wm=2, rm=4, wn=2, rn=4, mf=16, bk=128, st=7), 6),       # with 128-bit row stores, two tiles
    (200, 336, 136, dict(wm=1, rm=3, wn=2, rn=1, mf=16, bk=128, st=7), 7),       # three blocks per wavefront: a ragged last group
    (512, 1024, 512, dict(wm=4, rm=4, wn=2, rn=8, mf=16, bk=128, st=7), 4),      # the benchmark's tile
])
def test_gemm_int8_row_vector_stores(oracle, M, K, N, kn, store):
    """nt_store bit 1: the MFMA computes the transposed tile so that a lane
    holds four consecutive columns of one row; bit 2: early stores in the last tile."""
    _gemm_int8_case(oracle, M, K, N, kn, store)


@pytest.mark.parametrize("M,K,N,kn", [
    (136, 200, 72, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64)),              # K % 16 = 8: rows 8-byte aligned, dword loads
    (96, 100, 80, dict(wm=1, rm=2, wn=1, rn=1, mf=16, bk=64, st=1)),         # K % 16 = 4: a 4-byte tail
    (64, 67, 48, dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=64, st=3)),          # odd K: byte loads, one tile
    (80, 333, 96, dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=128, st=5)),        # odd K, three tiles, fragment prefetch
    (48, 18, 40, dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=64)),                # K below one MFMA step
])
def test_gemm_int8_k_not_a_multiple_of_16(oracle, M, K, N, kn):
    """The operator is defined for any reduce length (legacy/gemm_int8.py:15-21): rows that are not
    16-byte aligned are loaded in dwords or bytes, the bytes of the last chunk beyond the row (they
    belong to the next row) are replaced by zeros. Tiles straight into LDS refuse such a K."""
    _gemm_int8_case(oracle, M, K, N, kn, None)
    a = np.full((M, K), -128, np.int8)
    b = np.full((N, K), -128, np.int8)
    key = key_of("gemm", "gemm_int8", (M, K, N))
    out = run_plan(key, Config([gcfg(M, N, ceil_div(K, 64) * 64, **kn)], None), [a, b])
    assert np.array_equal(out, np.full((M, N), K * 16384, np.int32))          # every tail byte counted once
    with pytest.raises(Exception):
        schedule_with_config(key, Config([gcfg(M, N, ceil_div(K, 64) * 64, **dict(kn, st=6))], None))


@pytest.mark.parametrize("M,K,N,kn", [
    # K across workgroups: integer atomic adds into a zero-filled C
    (136, 512, 72, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64, sk=4)),                # ragged, register-staged
    (64, 1024, 96, dict(wm=1, rm=2, wn=1, rn=2, mf=16, bk=128, sk=8, st=5)),         # fragment prefetch, one tile per part
    (200, 1000, 136, dict(wm=2, rm=2, wn=1, rn=2, mf=16, bk=64, sk=4, st=3)),        # K tail in the last part only
    (256, 2048, 256, dict(wm=2, rm=2, wn=2, rn=2, mf=32, bk=128, sk=4, st=7)),       # tiles straight into LDS
    (256, 2048, 256, dict(wm=2, rm=4, wn=2, rn=4, mf=16, bk=128, sk=2, st=8)),       # written-out instruction order
    (80, 333, 96, dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=128, sk=3, st=2)),          # odd K: byte loads in every part
    # K across wavefront groups of one workgroup: summed through LDS
    (136, 512, 72, dict(wm=2, rm=1, wn=1, rn=1, mf=32, bk=64, sk=4, wk=1)),
    (64, 1024, 96, dict(wm=1, rm=2, wn=1, rn=2, mf=16, bk=128, sk=8, wk=1, st=5)),
    (200, 1000, 136, dict(wm=2, rm=2, wn=1, rn=2, mf=16, bk=64, sk=4, wk=1, st=3)),
    (128, 2048, 128, dict(wm=2, rm=2, wn=2, rn=2, mf=16, bk=128, sk=4, wk=1, st=7)),   # 16 wavefronts, direct to LDS
    (128, 2048, 256, dict(wm=2, rm=4, wn=1, rn=4, mf=16, bk=128, sk=2, wk=1, st=8)),   # written-out order: no barrier ends its last tile
    (256, 1024, 128, dict(wm=1, rm=4, wn=1, rn=4, mf=32, bk=64, sk=2, wk=1, st=1)),    # 256 accumulators, one buffer: the sum area exceeds the tiles
])
def test_gemm_int8_k_divisions(oracle, M, K, N, kn):
    """The reduce split of the int8 operator: across workgroups (exact whatever the order of the
    atomic adds) and across wavefront groups; twice through one plan, the second launch over the
    first one's result (the zero fill is part of the plan)."""
    _gemm_int8_case(oracle, M, K, N, kn, None)
    key = key_of("gemm", "gemm_int8", (M, K, N))
    _, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=K + 1)
    g = None
    if kn.get("st") in (6, 7, 8):
        g = {k: [] for k in KEYS}
        g["inline"], g["special"] = [[0]], [[-1, 0], [0]]
    s, _ = schedule_with_config(key, Config([gcfg(M, N, ceil_div(K, 64) * 64, **kn)], g))
    func = build(s, bufs, "rocm")
    ins = [torch.from_numpy(x).cuda() for x in (a, b)]
    out = torch.full((M, N), -77, dtype=torch.int32, device="cuda")
    for _ in range(2):
        func(*ins, out)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), oracle.gemm_i8_c(a, b))
    func.close()
    # stores that write finished sums do not combine with a divided K
    if kn.get("st") == 7 and kn["bk"] == 2 * (32 if kn["mf"] == 32 else 64):
        with pytest.raises(InvalidConfig):
            g2 = {k: [] for k in KEYS}
            g2["inline"], g2["special"] = [[0]], [[-1, 0], [4]]
            schedule_with_config(key, Config([gcfg(M, N, ceil_div(K, 64) * 64, **kn)], g2))


def _gemm_int8_case(oracle, M, K, N, kn, store):
    register(gemm_int8, "gemm", "gemm_int8", (M, K, N), "rocm", 0)
    key = key_of("gemm", "gemm_int8", (M, K, N))
    _, bufs = TASK_TABLE[key].func(M, K, N)
    a, b = seeded_inputs(bufs, seed=K)
    assert a.min() == -128 and a.max() == 127
    g = None
    if store is not None or kn.get("st") in (6, 7, 8):       # direct-to-LDS tiles need the swizzled (unpadded) layout
        g = {k: [] for k in KEYS}
        g["inline"], g["special"] = [[0]], [[-1, 0], [store or 0]]
    out = run_plan(key, Config([gcfg(M, N, ceil_div(K, 64) * 64, **kn)], g), [a, b])
    assert np.array_equal(out, oracle.gemm_i8_c(a, b))
    assert np.array_equal(out, oracle.gemm_i8_np(a, b))


CONV_CASES = [
    # batch, C, H, W, K, k, stride, pad, dil, knobs
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=16)),
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=2, rn=2, mf=16, bk=16, sk=3)),
    ((1, 8, 17, 13, 24, 3, 2, 1, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16)),   # stride 2, K=72 -> 80
    ((3, 6, 11, 11, 20, 3, 1, 2, 2, 1), dict(wm=1, rm=2, wn=2, rn=1, mf=16, bk=32)),   # dilation 2
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=32)),    # 1x1, N=392
    ((1, 3, 32, 32, 16, 7, 2, 3, 1, 1), dict(wm=1, rm=1, wn=4, rn=1, mf=16, bk=16)),   # 7x7 s2 p3, K=147
    ((2, 16, 14, 14, 32, 3, 1, 1, 1, 1), dict(wm=2, rm=1, wn=1, rn=1, mf=16, bk=16, sk=3, wk=1, st=3)),
    ((1, 64, 28, 28, 64, 3, 1, 1, 1, 1), dict(wm=4, rm=1, wn=1, rn=1, mf=16, bk=32, sk=2, wk=1, st=4)),
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72)),              # groups 4, whole windows
    ((2, 24, 10, 10, 24, 3, 1, 1, 1, 12), dict(wm=1, rm=1, wn=1, rn=2, mf=16, bk=16)),             # two channels per group, K=18 -> 32
    # K = 400 has no LDS tile wider than 16: zero-padded to 448 = 7 x 64 and 432 = 3 x 144 (the last tile holds 16 real columns)
    ((2, 16, 14, 14, 48, 5, 1, 2, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=16, bk=64, st=3, kp=448)),
    ((2, 16, 14, 14, 48, 5, 1, 2, 1, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=16, bk=144, st=5, kp=432)),
    ((2, 16, 14, 14, 48, 5, 1, 2, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=144, st=8, ls=4, kp=432)),
    ((2, 16, 14, 14, 48, 5, 1, 2, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=32, st=2, kp=416, wk=1, sk=13)),
    ((1, 16, 14, 14, 32, 3, 2, 1, 1, 2), dict(wm=1, rm=1, wn=1, rn=1, mf=32, bk=8, sk=3)),         # groups 2, split-K atomics
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), dict(wm=1, rm=1, wn=2, rn=1, mf=32, bk=72, ks=1)),        # groups 4, K streaming
    ((1, 8, 17, 13, 24, 3, 2, 1, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16, ks=1, st=3)),   # K streaming, padded K
    ((8, 64, 7, 7, 96, 1, 1, 0, 1, 1), dict(wm=1, rm=2, wn=2, rn=1, mf=16, bk=32, ks=2)),          # 1x1, K streaming
    # 98 tiles of 36 k-steps over 256 workgroups: most tiles have three sharers and most workgroups
    # end one tile and begin the next (an early version of the exchange summed this one wrong)
    ((1, 64, 56, 56, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=2, wn=2, rn=1, mf=16, bk=16, st=3, ks=1)),
    ((1, 64, 56, 56, 64, 3, 1, 1, 1, 1), dict(wm=2, rm=2, wn=2, rn=1, mf=16, bk=16, st=2, ks=2)),
    # one wavefront, 224 columns, two register sets of 56 gathered elements, 112 accumulators: every
    # register in use (the compiler once split live ranges inside the divergent address arithmetic
    # of this kernel and lanes outside the image kept stale rows)
    ((3, 6, 11, 11, 20, 3, 1, 2, 2, 1), dict(wm=1, rm=1, wn=1, rn=7, mf=32, bk=16, st=3)),
]


@pytest.mark.parametrize("args,kn", CONV_CASES)
def test_conv2d_vs_oracle(oracle, args, kn):
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    key = key_of("conv2d", "t", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    ref = oracle.conv2d_nchw_c(x, w, st, pd, dl, g)
    assert ref.shape == bufs[-1].shape
    M, N, K = ko // g, nb * ref.shape[2] * ref.shape[3], (c // g) * ks * ks
    kn = dict(kn)
    kp = kn.pop("kp", K if K % kn["bk"] == 0 else ceil_div(K, 16) * 16)
    cfg = gcfg(M, N, kp, **kn)
    for inline in ([1, 0], [0, 0]):
        out = run_plan(key, conv_cfgs(cfg, inline), [x, w])
        assert rel(out, ref) <= TOL, inline
        assert rel(out, oracle.conv2d_nchw_np(x, w, st, pd, dl, g)) <= TOL


@pytest.mark.parametrize("args,kn", [
    ((1, 64, 14, 14, 96, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=16, bk=32, st=3)),         # 196 pixels: 16-byte image rows
    ((1, 64, 14, 14, 96, 1, 1, 0, 1, 1), dict(wm=1, rm=1, wn=4, rn=1, mf=16, bk=64, st=8, ls=2)),   # tiles straight into LDS
    ((1, 48, 7, 7, 40, 1, 1, 0, 1, 1), dict(wm=1, rm=1, wn=1, rn=1, mf=16, bk=16, st=2, sk=3, wk=1)),  # 49 pixels: single floats
    ((1, 48, 13, 13, 24, 1, 1, 0, 2, 1), dict(wm=1, rm=1, wn=2, rn=1, mf=16, bk=16, st=5)),         # dilation has no meaning at 1x1
    ((1, 72, 28, 28, 64, 1, 1, 0, 1, 1), dict(wm=2, rm=1, wn=2, rn=1, mf=32, bk=72, st=3, ks=1)),   # K streaming
])
def test_pointwise_conv2d_over_one_image_as_a_gemm(oracle, args, kn):
    """1x1 / stride 1 / unpadded convolution of one image: O [K][H*W] = W [K][C] x X [C][H*W] in the
    tensors' own layouts. image_as_matrix 1 lowers it in the GEMM addressing mode, 0 as the gather."""
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    key = key_of("conv2d", "t", args)
    assert list(TASK_TABLE[key].special_space) == ["lds_pad", "image_as_matrix"]
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    ref = oracle.conv2d_nchw_c(x, w, st, pd, dl, g)
    cfg = gcfg(ko, h * wd, c, **kn)
    for flag in (1, 0):
        for inline in ([1, 0], [0, 0]):
            cfgs = conv_cfgs(cfg, inline, special=[[-1, -1], [flag]])
            s, _ = schedule_with_config(key, cfgs)
            assert s.specs[-1].defines["MODE"] == (0 if flag else 1)
            assert rel(run_plan(key, cfgs, [x, w]), ref) <= TOL, (flag, inline)
    s, _ = schedule_with_config(key, Config([], None))               # the default is the GEMM mode
    assert s.specs[-1].defines["MODE"] == 0
    assert rel(run_plan(key, Config([], None), [x, w]), ref) <= TOL


@pytest.mark.parametrize("args", [
    (2, 24, 10, 10, 24, 3, 1, 1, 1, 24),          # groups = channels, one kernel per channel
    (1, 8, 12, 16, 48, 3, 2, 1, 1, 8),            # six kernels per channel, stride 2 (a MobileNet stage)
    (2, 5, 9, 11, 10, 3, 1, 1, 2, 5),             # two kernels per channel, dilation 2
])
def test_conv2d_with_one_channel_per_group_takes_the_depthwise_kernel(oracle, args):
    """conv2d_nchw with groups = input channels is the depthwise operator (weight
    [K, 1, kh, kw] = [C, K/C, kh, kw] in memory): the plan holds the depthwise
    kernel and its result is the grouped convolution's."""
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    key = key_of("conv2d", "t", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    assert ops[0].kind == "depthwise_conv2d_nchw" and ops[0].attrs["factor"] == args[4] // args[1]
    assert "row_exchange" in TASK_TABLE[key].special_space
    x, w = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, ko, ks, st, pd, dl, g = args
    ref = oracle.conv2d_nchw_c(x, w, st, pd, dl, g)
    assert ref.shape == bufs[-1].shape
    b_, co, p, q = ref.shape
    s, _ = schedule_with_config(key, Config([], None))
    assert [sp.kernel for sp in s.specs] == ["depthwise_f32"]
    assert rel(run_plan(key, Config([], None), [x, w]), ref) <= TOL
    for inline in ([1, 0], [0, 0]):
        for fuse in (1, 0):
            cfgs = conv_cfgs(dcfg(b_, co, p, q, min(2, p), min(4, q), 2), inline, special=[[0], [0], [0], [1], [0], [fuse]])
            assert rel(run_plan(key, cfgs, [x, w]), ref) <= TOL, (inline, fuse)


def test_conv2d_and_depthwise_with_row_column_pairs(oracle):
    """stride / padding / dilation as (rows, columns) pairs (flextensor/nn/ops.py:448-459), through
    the implicit GEMM (folded and materialised padding, register-staged and straight-into-LDS
    tiles, hoisted and per-tile gather), the im2col form and the direct depthwise kernel."""
    from flextensor_amd.nn import conv2d_nchw, depthwise_conv2d_nchw, gemm_conv2d_nchw

    def wrap(kind, N, C, H, W, K, r, s, st, pd, dl, g=1, f=1):
        Img = placeholder((N, C, H, W), name="Img")
        if kind == "depthwise":
            Wt = placeholder((C, f, r, s), name="W")
            Out = depthwise_conv2d_nchw(Img, Wt, stride=st, padding=pd, dilation=dl)
        else:
            Wt = placeholder((K, C // g, r, s), name="W")
            fn = conv2d_nchw if kind == "conv" else gemm_conv2d_nchw
            Out = fn(Img, Wt, stride=st, padding=pd, dilation=dl, groups=g)
        return [Out.op], [Img, Wt, Out]

    cases = [("conv", (2, 8, 11, 14, 32, 3, 3, (2, 1), (1, 2), (1, 2), 1)),
             ("conv", (1, 8, 13, 9, 16, 3, 5, (1, 2), (0, 2), (2, 1), 2)),
             ("im2col", (2, 8, 11, 14, 32, 3, 3, (2, 1), (1, 2), (1, 2), 1))]
    for kind, a in cases:
        name = "pairs_" + kind
        register(lambda *args, kind=kind: wrap(kind, *args), "conv2d", name, a, "rocm", 0)
        key = key_of("conv2d", name, a)
        # a task built on a function of its own carries the knobs it declares
        TASK_TABLE[key].set_specific_space("lds_pad", "enum", [[4, -1], [0, 0]])
        ops, bufs = TASK_TABLE[key].func(*a)
        x, w = seeded_inputs(bufs, seed=31)
        ref = oracle.conv2d_nchw_c(x, w, a[7], a[8], a[9], a[10])
        assert ref.shape == bufs[-1].shape
        M, N, K = a[4] // a[10], a[0] * ref.shape[2] * ref.shape[3], (a[1] // a[10]) * a[5] * a[6]
        kp = ceil_div(K, 16) * 16
        plans = [Config([], None)]
        if kind == "conv":
            for st_, bk, pad in ((3, 16, [4, -1]), (5, 16, [0, 0])):
                if kp % bk == 0:
                    for inline in ([1, 0], [0, 0]):
                        plans.append(conv_cfgs(gcfg(M, N, kp, 1, 1, 2, 1, 16, bk, st=st_), inline, [pad]))
        for cfg in plans:
            out = run_plan(key, cfg, [x, w])
            assert rel(out, ref) <= TOL, (kind, a, cfg)
        dev = [torch.from_numpy(t).cuda() for t in (x, w)]
        out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
        run_default_schedule(ops, dev + [out], stream=current_stream())
        torch.cuda.synchronize()
        assert rel(out.cpu().numpy(), ref) <= TOL
    for a, th, tw in (((2, 6, 11, 14, 0, 3, 3, (2, 1), (1, 2), (1, 2), 1, 2), 2, 2),
                      ((1, 5, 9, 12, 0, 3, 3, (1, 1), (1, 1), (1, 1), 1, 1), 3, 4),
                      ((1, 5, 9, 12, 0, 3, 3, (2, 1), (0, 1), (1, 1), 1, 1), 2, 4)):
        register(lambda *args: wrap("depthwise", *args), "conv2d", "pairs_dw", a, "rocm", 0)
        key = key_of("conv2d", "pairs_dw", a)
        ops, bufs = TASK_TABLE[key].func(*a)
        x, w = seeded_inputs(bufs, seed=17)
        ref = oracle.depthwise_nchw_c(x, w, a[7], a[8], a[9])
        b_, co, p, q = ref.shape
        assert ref.shape == bufs[-1].shape
        for inline in ([1, 0], [0, 0]):
            out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, min(th, p), min(tw, q), 2), inline), [x, w])
            assert rel(out, ref) <= TOL, (a, inline)


@pytest.mark.parametrize("args,th,tw,waves", [
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 4, 4, 4),
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 7, 4, 1),
    ((1, 8, 15, 13, 2, 3, 1, 1, 1), 4, 4, 2),      # odd plane, factor 2
    ((1, 8, 15, 13, 2, 3, 2, 1, 1), 2, 2, 1),      # stride 2
    ((2, 4, 9, 9, 1, 5, 1, 2, 1), 1, 4, 1),        # 5x5
])
def test_depthwise_vs_oracle(oracle, args, th, tw, waves):
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    nb, c, h, wd, f, ks, st, pd, dl = args
    ref = oracle.depthwise_nchw_c(x, w, st, pd, dl)
    b_, co, p, q = ref.shape
    out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, min(th, p), min(tw, q), waves)), [x, w])
    assert rel(out, ref) <= TOL


@pytest.mark.parametrize("args,th,tw,waves", [
    ((2, 6, 16, 32, 6, 3, 2, 1, 1), 2, 4, 2),     # stride 2, rows of whole vectors: two 128-bit loads per patch row
    ((1, 5, 14, 28, 6, 3, 2, 1, 1), 1, 4, 1),     # 14 output columns: the last patch of a row is ragged
    ((1, 4, 14, 14, 6, 3, 1, 1, 1), 2, 4, 1),     # stride 1, rows that are no multiple of four floats (scalar loads)
    ((2, 3, 12, 16, 3, 3, 1, 1, 1), 3, 4, 2),     # stride 1, one 128-bit load per patch row, factor 3
    ((1, 4, 16, 16, 2, 3, 2, 2, 2), 2, 4, 1),     # stride 2, dilation 2, padding 2: two halo columns on the left
    ((1, 4, 13, 16, 2, 3, 2, 1, 2), 2, 4, 1),     # stride 2, dilation 2, padding 1: output rows are not half rows
    ((1, 3, 9, 11, 4, 3, 2, 1, 1), 2, 2, 1),      # odd plane, two outputs per lane row
    # a ragged last patch whose last stored column reads the right padding through the vectors
    ((1, 4, 28, 28, 1, 5, 2, 2, 1), 2, 4, 1),     # 5x5, stride 2, padding 2: 14 output columns
    ((1, 4, 12, 12, 2, 3, 2, 2, 2), 1, 4, 1),     # 3x3, stride 2, dilation 2, padding 2: 6 output columns
    ((1, 2, 20, 20, 1, 7, 2, 3, 1), 1, 4, 1),     # 7x7, stride 2, padding 3: 10 output columns
    ((1, 4, 28, 28, 1, 5, 2, 2, 1), 1, 4, 2),
])
def test_depthwise_kernels_of_a_channel_fused_vs_oracle(oracle, args, th, tw, waves):
    """Several kernels per input channel: a lane loads its input patch once and
    computes the patch of every output plane of the channel (kernel_fuse 1),
    or lanes own single output planes (0); stride 2 reads two vectors per row."""
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    ref = oracle.depthwise_nchw_c(x, w, args[6], args[7], args[8])
    b_, co, p, q = ref.shape
    # the halo through lane shifts where the layer admits it (stride 1, rows of whole vectors)
    shuffles = (0, 1) if (args[6] == 1 and args[8] == 1 and args[3] % 4 == 0 and tw == 4) else (0,)
    for fuse in (1, 0):
        for items in (1, 2):
            for shfl in shuffles:
                cfgs = conv_cfgs(dcfg(b_, co, p, q, min(th, p), min(tw, q), waves),
                                 special=[[0], [shfl], [0], [items], [0], [fuse]])
                if items == 2 and args[5] >= 7:
                    with pytest.raises(InvalidConfig):      # two 7x7 patches per lane do not fit the registers
                        schedule_with_config(key, cfgs)
                    continue
                s, _ = schedule_with_config(key, cfgs)
                assert s.specs[-1].defines.get("MFUSE", 0) == (fuse if args[4] > 1 else 0)
                assert s.specs[-1].defines["SHFL"] == shfl
                out = run_plan(key, cfgs, [x, w])
                assert rel(out, ref) <= TOL, (fuse, items, shfl)
    # borders: a constant image must give border sums with missing taps
    ones = np.ones_like(x)
    out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, min(th, p), min(tw, q), waves)), [ones, w])
    assert rel(out, oracle.depthwise_nchw_np(ones, w, args[6], args[7], args[8])) <= TOL


@pytest.mark.parametrize("args,th,waves", [
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 7, 4),       # 7 lanes per row, 63 lanes per wavefront
    ((1, 5, 8, 12, 1, 3, 1, 1, 1), 4, 1),         # 3 lanes per row, last wavefront partly idle
    ((3, 7, 16, 64, 1, 3, 1, 1, 1), 2, 2),        # 16 lanes per row
    ((1, 3, 9, 20, 2, 3, 1, 1, 1), 3, 1),         # factor 2, ragged rows per lane
])
def test_depthwise_shuffled_halo_vs_oracle(oracle, args, th, waves):
    """Halo columns taken from neighbouring lanes (DPP shifts) instead of loads."""
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    ref = oracle.depthwise_nchw_c(x, w, args[6], args[7], args[8])
    b_, co, p, q = ref.shape
    for nt_store in (0, 1, 3):                    # bit 0: non-temporal stores, bit 1: non-temporal loads
        out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, th, 4, waves), special=[[nt_store], [1]]), [x, w])
        assert rel(out, ref) <= TOL, nt_store
    # borders: a constant image must give border sums with missing taps
    ones = np.ones_like(x)
    out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, th, 4, waves), special=[[0], [1]]), [ones, w])
    assert rel(out, oracle.depthwise_nchw_np(ones, w, args[6], args[7], args[8])) <= TOL
    # several patches per lane (lane_items), requested up front: shuffled halo, loaded halo, scalar path
    for items, shfl, tw in ((3, 1, 4), (2, 0, 4), (4, 0, 2)):
        out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, th, tw, waves), special=[[1], [shfl], [0], [items]]), [x, w])
        assert rel(out, ref) <= TOL, (items, shfl, tw)


@pytest.mark.parametrize("args,chunks,waves,rows_per_load", [
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 2, 4, 7),     # 14 rows per wavefront: two spans tile a plane
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 4, 2, 7),     # a whole plane per wavefront: every halo row is padding
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 3, 1, 9),     # 27 rows + a ragged span of one row
    ((1, 5, 8, 12, 1, 3, 1, 1, 1), 1, 1, 8),       # 3 chunks per row, 24 of 64 lanes busy; 5 planes
    ((3, 7, 16, 64, 1, 3, 1, 1, 1), 2, 2, 4),      # 16 chunks per row; 21 planes x 2 spans on 2-wavefront workgroups
    ((2, 3, 7, 4, 1, 3, 1, 1, 1), 8, 4, 7),        # one chunk per row: every chunk is left and right edge; more rows than the plane
    ((1, 2, 5, 128, 1, 3, 1, 1, 1), 3, 1, 2),      # 32 chunks per row: the two halo rows take all 64 lanes
])
def test_depthwise_row_exchange_vs_oracle(oracle, args, chunks, waves, rows_per_load):
    """Rows pass between lanes through a wavefront-private LDS window; every chunk is loaded once."""
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    ref = oracle.depthwise_nchw_c(x, w, args[6], args[7], args[8])
    b_, co, p, q = ref.shape
    for nt_store in (0, 1, 3):
        cfgs = conv_cfgs(dcfg(b_, co, p, q, 1, 4, waves), special=[[nt_store], [0], [0], [1], [chunks]])
        s, _ = schedule_with_config(key, cfgs)
        assert s.specs[-1].defines["WX"] == chunks and s.specs[-1].defines["WXR"] == rows_per_load
        out = run_plan(key, cfgs, [x, w])
        assert rel(out, ref) <= TOL, nt_store
    # borders: a constant image must give border sums with missing taps
    ones = np.ones_like(x)
    out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, 1, 4, waves), special=[[0], [0], [0], [1], [chunks]]), [ones, w])
    assert rel(out, oracle.depthwise_nchw_np(ones, w, args[6], args[7], args[8])) <= TOL
    # a layer it does not fit is refused, not mis-computed
    for bad in ((1, 4, 9, 20, 2, 3, 1, 1, 1), (1, 4, 9, 20, 1, 3, 2, 1, 1), (1, 4, 9, 18, 1, 3, 1, 1, 1)):   # factor 2; stride 2; ragged rows
        register(depthwise_conv2d, "conv2d", "depthwise", bad, "rocm", 0)
        bo = oracle.depthwise_nchw_np(np.zeros((bad[0], bad[1], bad[2], bad[3]), np.float32),
                                      np.zeros((bad[1], bad[4], 3, 3), np.float32), bad[6], bad[7], bad[8]).shape
        with pytest.raises(Exception):
            schedule_with_config(key_of("conv2d", "depthwise", bad),
                                 conv_cfgs(dcfg(bo[0], bo[1], bo[2], bo[3], 1, 4, 1), special=[[0], [0], [0], [1], [2]]))


@pytest.mark.parametrize("args,planes,waves", [
    ((2, 16, 28, 28, 1, 3, 1, 1, 1), 4, 4),
    ((1, 5, 8, 12, 1, 3, 1, 1, 1), 2, 1),         # 5 planes, 2 per workgroup: the last workgroup is half empty
    ((3, 7, 16, 64, 1, 3, 1, 1, 1), 1, 2),
    ((2, 3, 7, 4, 1, 3, 1, 1, 1), 8, 1),          # one vector per row, more slots than planes
])
def test_depthwise_plane_staged_vs_oracle(oracle, args, planes, waves):
    """Whole planes staged through LDS in copy order; a zero border is the padding."""
    register(depthwise_conv2d, "conv2d", "depthwise", args, "rocm", 0)
    key = key_of("conv2d", "depthwise", args)
    ops, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, seed=sum(args))
    ref = oracle.depthwise_nchw_c(x, w, args[6], args[7], args[8])
    b_, co, p, q = ref.shape
    for nt_store in (0, 1, 2):
        cfgs = conv_cfgs(dcfg(b_, co, p, q, 1, 4, waves), special=[[nt_store], [0], [planes]])
        s, _ = schedule_with_config(key, cfgs)
        assert s.specs[-1].defines["LDSP"] == planes
        out = run_plan(key, cfgs, [x, w])
        assert rel(out, ref) <= TOL, nt_store
    ones = np.ones_like(x)
    out = run_plan(key, conv_cfgs(dcfg(b_, co, p, q, 1, 4, waves), special=[[0], [0], [planes]]), [ones, w])
    assert rel(out, oracle.depthwise_nchw_np(ones, w, args[6], args[7], args[8])) <= TOL
    # a layer it does not fit is refused, not mis-computed
    bad = (1, 4, 9, 20, 2, 3, 1, 1, 1)            # factor 2
    register(depthwise_conv2d, "conv2d", "depthwise", bad, "rocm", 0)
    with pytest.raises(Exception):
        schedule_with_config(key_of("conv2d", "depthwise", bad),
                             conv_cfgs(dcfg(1, 8, 9, 20, 1, 4, 1), special=[[0], [0], [2]]))


DEGENERATE = [
    (gemm, "gemm", "gemm", (1, 1, 1)), (gemm, "gemm", "gemm", (1, 17, 3)), (gemm, "gemm", "gemm", (3, 5, 1)),
    (gemm_int8, "gemm", "gemm_int8", (1, 1, 1)), (gemm_int8, "gemm", "gemm_int8", (2, 3, 5)),
    (conv2d, "conv2d", "t", (1, 1, 1, 1, 1, 1, 1, 0, 1, 1)),          # one pixel, one channel, one tap
    (conv2d, "conv2d", "t", (1, 3, 5, 5, 2, 3, 1, 0, 1, 1)),          # 3x3 output
    (conv2d, "conv2d", "t", (1, 2, 3, 3, 4, 3, 1, 1, 1, 2)),          # one channel per group: the depthwise kernel
    (depthwise_conv2d, "conv2d", "depthwise", (1, 1, 1, 1, 1, 1, 1, 0, 1)),
    (depthwise_conv2d, "conv2d", "depthwise", (1, 3, 3, 3, 2, 3, 1, 1, 1)),
    (depthwise_conv2d, "conv2d", "depthwise", (2, 2, 5, 7, 1, 3, 2, 0, 1)),
]


@pytest.mark.parametrize("func,category,name,args", DEGENERATE)
def test_smallest_extents(oracle, func, category, name, args):
    """Extents of one and a few: every tile is an edge tile, most lanes idle, K far below one MFMA step."""
    register(func, category, name, args, "rocm", 0)
    key = key_of(category, name, args)
    ops, bufs = TASK_TABLE[key].func(*args)
    host = seeded_inputs(bufs, seed=sum(args) + 1)
    out = run_plan(key, Config([], None), host)
    if func is gemm_int8:
        assert np.array_equal(out, oracle.gemm_i8_c(host[0], host[1]))
        ref = oracle.gemm_i8_np(host[0], host[1])
    elif func is gemm:
        ref = oracle.gemm_f32_c(host[0], host[1])
    elif func is conv2d:
        ref = oracle.conv2d_nchw_c(host[0], host[1], args[6], args[7], args[8], args[9])
    else:
        ref = oracle.depthwise_nchw_c(host[0], host[1], args[6], args[7], args[8])
    assert out.shape == np.asarray(ref).shape
    assert rel(out, ref) <= TOL
    # the default-schedule kernels the search gates candidates against
    tdt = {"float32": torch.float32, "int32": torch.int32}[bufs[-1].dtype]
    dev = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in host]
    gate = torch.full(bufs[-1].shape, -77, dtype=tdt, device="cuda")
    run_default_schedule(ops, dev + [gate], stream=current_stream())
    torch.cuda.synchronize()
    assert rel(gate.cpu().numpy(), ref) <= TOL


def test_empty_extents_are_refused_on_the_host():
    for func, category, name, args in ((gemm, "gemm", "gemm", (0, 4, 4)), (gemm, "gemm", "gemm", (4, 0, 4)),
                                       (gemm_int8, "gemm", "gemm_int8", (4, 4, 0))):
        with pytest.raises(Exception):
            register(func, category, name, args, "rocm", 0)
            schedule_with_config(key_of(category, name, args), Config([], None))


def test_default_schedule_kernels_vs_oracle(oracle):
    """The plain kernels every candidate is gated against are themselves right."""
    s = current_stream()
    for args in [(2, 6, 9, 11, 9, 3, 2, 1, 2, 3), (1, 4, 8, 8, 6, 3, 1, 1, 1, 1)]:
        ops, bufs = conv2d(*args)
        x, w = seeded_inputs(bufs, 1)
        out = torch.empty(bufs[-1].shape, device="cuda")
        run_default_schedule(ops, [torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), out], s)
        ref = oracle.conv2d_nchw_c(x, w, args[6], args[7], args[8], args[9])
        assert rel(out.cpu().numpy(), ref) <= 1e-6
    ops, bufs = depthwise_conv2d(2, 6, 9, 11, 3, 3, 2, 1, 2)
    x, w = seeded_inputs(bufs, 2)
    out = torch.empty(bufs[-1].shape, device="cuda")
    run_default_schedule(ops, [torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), out], s)
    assert rel(out.cpu().numpy(), oracle.depthwise_nchw_c(x, w, 2, 1, 2)) <= 1e-6
    ops, bufs = gemm(70, 50, 90)
    a, b = seeded_inputs(bufs, 3)
    out = torch.empty(bufs[-1].shape, device="cuda")
    run_default_schedule(ops, [torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), out], s)
    assert rel(out.cpu().numpy(), oracle.gemm_f32_c(a, b)) <= 1e-6
    ops, bufs = gemm_int8(70, 64, 90)
    a, b = seeded_inputs(bufs, 4)
    out = torch.empty(bufs[-1].shape, dtype=torch.int32, device="cuda")
    run_default_schedule(ops, [torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), out], s)
    assert np.array_equal(out.cpu().numpy(), oracle.gemm_i8_c(a, b))


# ------------------------------------------- the five benchmark configs ---

FULL = {
    "gemm": "gemm_gemm_(1024, 1024, 1024)_rocm(0)",
    "conv2": "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)",
    "conv3a": "conv2d_baseline1_(8, 256, 14, 14, 512, 3, 1, 1, 1, 1)_rocm(0)",
    "conv3b": "conv2d_baseline2_(8, 512, 7, 7, 2048, 1, 1, 0, 1, 1)_rocm(0)",
    "dw": "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)",
    "i8": "gemm_gemm_int8_(4096, 4096, 4096)_rocm(0)",
}


def tuned_configs(key):
    from flextensor_amd.tuned import lookup
    cfg = lookup(key)
    return cfg if cfg is not None else Config([], None)


def test_full_size_gemm_fp32(oracle):
    key = FULL["gemm"]
    _, bufs = TASK_TABLE[key].func(*TASK_TABLE[key].args)
    a, b = seeded_inputs(bufs, 0)
    out = run_plan(key, tuned_configs(key), [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL
    rows = oracle.gemm_f32_c(a[:48], b)           # fp32 sequential-k oracle on a row sample
    assert rel(out[:48], rows) <= TOL


@pytest.mark.parametrize("name", ["conv2", "conv3a", "conv3b"])
def test_full_size_conv2d(oracle, name):
    key = FULL[name]
    args = TASK_TABLE[key].args
    _, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, 0)
    out = run_plan(key, tuned_configs(key), [x, w])
    ref = oracle.conv2d_nchw_c(x, w, args[6], args[7], args[8], args[9])
    assert rel(out, ref) <= TOL
    assert rel(out, oracle.conv2d_nchw_np(x, w, args[6], args[7], args[8], args[9])) <= TOL


def test_full_size_depthwise(oracle):
    key = FULL["dw"]
    args = TASK_TABLE[key].args
    _, bufs = TASK_TABLE[key].func(*args)
    x, w = seeded_inputs(bufs, 0)
    out = run_plan(key, tuned_configs(key), [x, w])
    assert rel(out, oracle.depthwise_nchw_c(x, w, 1, 1, 1)) <= TOL
    # linearity in the input, a size-independent property
    x2 = np.random.default_rng(5).uniform(-1, 1, x.shape).astype(np.float32)
    o2 = run_plan(key, tuned_configs(key), [x2, w])
    o12 = run_plan(key, tuned_configs(key), [x + x2, w])
    assert rel(o12, out.astype(np.float64) + o2) <= TOL


def test_full_size_gemm_int8_bit_exact(oracle):
    key = FULL["i8"]
    _, bufs = TASK_TABLE[key].func(*TASK_TABLE[key].args)
    a, b = seeded_inputs(bufs, 0)
    out = run_plan(key, tuned_configs(key), [a, b])
    assert np.array_equal(out, oracle.gemm_i8_np(a, b))              # exact, float64 BLAS
    assert np.array_equal(out[100:132], oracle.gemm_i8_c(a, b, 100, 132)[100:132])
    # size-independent properties: worst-case magnitude and a permutation operand
    a2 = np.full_like(a, -128)
    out2 = run_plan(key, tuned_configs(key), [a2, a2])
    assert out2.min() == out2.max() == 4096 * 128 * 128              # 2^26, no overflow
    eye = np.eye(4096, dtype=np.int8)
    out3 = run_plan(key, tuned_configs(key), [a, eye])
    assert np.array_equal(out3, a.astype(np.int32))                  # A · Iᵀ = A
    out4 = run_plan(key, tuned_configs(key), [a, b])
    assert np.array_equal(out4, out)                                 # deterministic


# --------------------------------------------------- measure / search path --

def _registered_layer_keys():
    keys = [k for k, t in TASK_TABLE.items() if t.dev_id == 0 and t.target == "rocm" and t.category == "conv2d"
            and not k.startswith("conv2d_t_") and not k.startswith("conv2d_bias") and not k.startswith("conv2d_smoke")]
    # yolo at batch 8 repeats the batch-1 layers with 8x the work: keep every third of them
    b8 = [k for k in keys if k.startswith("conv2d_yolo_b8")]
    keys = [k for k in keys if not k.startswith("conv2d_yolo_b8")] + b8[::3]
    # the other networks' tables: every fourth layer of each (all of the short ones)
    for prefix, step in (("conv2d_google", 4), ("conv2d_res", 4), ("conv2d_squeeze", 4), ("conv2d_vgg-16", 3),
                         ("conv2d_overfeat", 2), ("conv2d_mobile_v2", 2)):
        net = sorted(k for k in keys if k.startswith(prefix))
        keys = [k for k in keys if not k.startswith(prefix)] + net[::step]
    return sorted(keys) + ["gemm_gemm_(32, 32, 32)_rocm(0)", "gemm_gemm_(4096, 32, 64)_rocm(0)",
                           "gemm_gemm_(64, 4096, 4096)_rocm(0)", "gemm_gemm_(2048, 2048, 2048)_rocm(0)"]


@pytest.mark.parametrize("key", _registered_layer_keys())
def test_registered_tasks_default_config_passes_the_gate(key):
    """Registered convolution layers (all of YOLO, grouped, dilated, depthwise
    and the benchmark shapes, a sample of the other networks' tables) and a
    few GEMM shapes: the untuned plan matches the default-schedule kernels on
    the device."""
    s, bufs = schedule_with_config(key, Config([], None))
    s.compile()                                   # from the on-disk cache when built ahead of time
    ms = Measurer(key).evaluate(s, number=3, warmup=1, warm_ms=0)
    assert 0 < ms < 1e3


def _shipped_keys():
    from flextensor_amd.tuned import load
    return sorted(load())


@pytest.mark.parametrize("key", _shipped_keys())
def test_every_shipped_entry_passes_the_gate(key):
    """Each line of the shipped log of tuned points lowers with today's
    templates and its kernels match the default-schedule kernels on the
    device (fp32 within 1e-5 of the largest value, int32 identical)."""
    s, bufs = schedule_with_config(key, tuned_configs(key))
    s.compile()
    ms = Measurer(key).evaluate(s, number=3, warmup=1, warm_ms=0)
    assert 0 < ms < 1e3


def test_correctness_gate_rejects_wrong_output():
    key = "gemm_gemm_(256, 256, 256)_rocm(0)"
    m = Measurer(key)
    s, _ = schedule_with_config(key, Config([], None))
    ms = m.evaluate(s, number=3)
    assert 0 < ms < 10
    ok, metric = m.check(m.sets[0][-1])
    assert ok and metric <= TOL
    m.ref += 1.0                                   # corrupt the default-schedule result
    with pytest.raises(WrongResult):
        m.evaluate(s, number=1)
    bad = m.sets[0][-1].clone()
    bad[3, 5] = float("nan")
    assert compare_on_device(bad, m.sets[0][-1], current_stream())[0] is False


def test_plan_verify_runs_the_gate_and_the_static_checks():
    """KernelPlan.verify(): what a replayed or hand-written config is checked with (the candidates of
    a search pass the same gate inside the measurer)."""
    import flextensor_amd.measure as measure
    for key in ("gemm_gemm_(256, 256, 256)_rocm(0)", "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)",
                "gemm_gemm_int8_(4096, 4096, 4096)_rocm(0)"):
        s, _ = schedule_with_config(key, Config([], None))
        assert s.verify() <= TOL
    key = "gemm_gemm_(256, 256, 256)_rocm(0)"
    s, _ = schedule_with_config(key, Config([], None))
    m = measure.get_measurer(key)
    keep = m.ref.clone()
    m.ref += 1.0                                   # corrupt the default-schedule result
    try:
        with pytest.raises(WrongResult):
            s.verify(static=False)
    finally:
        m.ref.copy_(keep)
    assert s.verify(static=False) <= TOL


def test_builtplan_rejects_mismatched_tensors():
    key = "gemm_gemm_(256, 256, 256)_rocm(0)"
    s, bufs = schedule_with_config(key, Config([], None))
    f = build(s, bufs, "rocm")
    a = torch.zeros(256, 256, device="cuda")
    with pytest.raises(ValueError):
        f(a, a)
    with pytest.raises(ValueError):
        f(a, a, torch.zeros(256, 128, device="cuda"))
    with pytest.raises(ValueError):
        f(a, a, torch.zeros(256, 256, device="cuda", dtype=torch.int32))
    with pytest.raises(ValueError):
        f(a, a.t(), torch.zeros(256, 256, device="cuda")) if not a.t().is_contiguous() else None
    with pytest.raises(ValueError):
        f(a.cpu(), a, a)
    f.close()


def test_schedule_with_the_performance_model_on_device(oracle, tmp_path):
    """use_model=True end to end on the GPU (flextensor/model.py:448-456, train.py:27-62): a first
    search measures on the device and leaves its data, the offline trainer fits the ranking
    network, a second search lets the network rank candidates and measures only its best points;
    what comes back is a checked, timed kernel that matches the oracle."""
    from flextensor_amd import train
    if os.environ.get("FT_TESTS_COMPILE_ONLY") == "1":
        pytest.skip("needs measured costs: nothing to compile ahead for a search")
    np.random.seed(1)
    torch.manual_seed(1)
    key = "gemm_gemm_(512, 256, 512)_rocm(0)"
    d = str(tmp_path)
    schedule(key, op_trial=2, graph_trial=1, op_stop=2, parallel=8, number=5, timeout=20, warm_up=(1, 8),
             verbose=False, method="searching", perf_path=d)
    assert "performance_judger_data_gemm_op0.txt" in os.listdir(d)
    train.train_for_schedule(key, perf=True, perf_path=d)
    assert "performance_judger_model_gemm_op0.pkl" in os.listdir(d)
    s, bufs, configs = schedule(key, op_trial=3, graph_trial=1, op_stop=3, parallel=8, number=5, timeout=20,
                                warm_up=(1, 8), verbose=False, method="searching", use_model=True, perf_path=d)
    a, b = seeded_inputs(bufs, 13)
    out = run_plan(key, configs, [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL
    assert s.specs[-1].kernel == "igemm_f32"


@pytest.mark.parametrize("method", ["searching", "q"])
def test_schedule_on_device_small_gemm(oracle, method):
    """End to end: search a few points on the GPU, replay the winner, check it."""
    np.random.seed(0)
    key = "gemm_gemm_(512, 256, 512)_rocm(0)"
    s, bufs, configs = schedule(key, op_trial=2, graph_trial=1, op_stop=2, parallel=8, number=5,
                                timeout=20, warm_up=(1, 8), verbose=False, method=method)
    a, b = seeded_inputs(bufs, 11)
    out = run_plan(key, configs, [a, b])
    assert rel(out, oracle.gemm_np(a, b)) <= TOL
    s2, _ = schedule_with_config(key, Config(*__import__("json").loads(__import__("json").dumps(configs))))
    assert s2.describe() == s.describe()
