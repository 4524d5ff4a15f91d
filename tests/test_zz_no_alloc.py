"""The entry point that allocates nothing (ftr_launch_seq_static_ws) against
ftr_launch_seq with caller-owned workspaces: K-streaming convolutions, two
calls in a row on the same static array, the second on a smaller input.
K streaming sums in a fixed order, so the two paths must agree bit for bit."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available() and os.environ.get("FT_TESTS_COMPILE_ONLY") != "1":
    pytest.skip("no GPU visible", allow_module_level=True)

from flextensor_amd import runtime as rt  # noqa: E402
from flextensor_amd.measure import seeded_inputs  # noqa: E402
from flextensor_amd.scheduler import schedule_with_config  # noqa: E402
from flextensor_amd.task import Task, register, conv2d  # noqa: E402
from flextensor_amd.utils import Config, ceil_div  # noqa: E402

KEYS = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]
COMPILE_ONLY = os.environ.get("FT_TESTS_COMPILE_ONLY") == "1"


def streaming_plan(args, wm, rm, wn, rn, mf, bk, per_cu):
    register(conv2d, "conv2d", "noalloc", args, "rocm", 0)
    key = Task("conv2d", "noalloc", None, args, "rocm", 0).key
    nb, c, h, w, ko, ks, st, pd, dl, g = args
    p = (h + 2 * pd - dl * (ks - 1) - 1) // st + 1
    q = (w + 2 * pd - dl * (ks - 1) - 1) // st + 1
    M, N, K = ko // g, nb * p * q, (c // g) * ks * ks
    cfg = {k: [] for k in KEYS}
    cfg["spatial"] = [[ceil_div(M, wm * rm * mf), wm, rm, mf], [ceil_div(N, wn * rn * mf), wn, rn, mf]]
    cfg["reduce"] = [[1, K // bk, bk]]
    cfg["unroll"], cfg["fuse"], cfg["reorder"] = [[3, 1]], [[4]], [[1, 0, per_cu]]
    s, bufs = schedule_with_config(key, Config([{k: [] for k in KEYS}, cfg], None))
    assert s.workspaces, "the case must need a workspace"
    return s, bufs


CASES = [
    ((1, 64, 56, 56, 64, 3, 1, 1, 1, 1), (2, 2, 2, 1, 16, 16, 1)),    # 98 tiles, 3528 units
    ((2, 32, 14, 14, 64, 3, 1, 1, 1, 4), (1, 1, 2, 1, 32, 72, 1)),    # smaller: grouped, other layout
]


def test_static_workspace_matches_owned_workspace():
    plans = [streaming_plan(a, *k) for a, k in CASES]
    if COMPILE_ONLY:
        for s, _ in plans:
            s.compile()
        pytest.skip("compile only")
    for rounds in range(2):                     # twice over both: the array keeps the previous contents
        for (s, bufs), (args, _) in zip(plans, CASES):
            x, w = [torch.from_numpy(a).cuda() for a in seeded_inputs(bufs, seed=3 + rounds)]
            owned = s.build()
            static = s.build(static_workspace=True)
            out_o = torch.full(bufs[-1].shape, -5.0, device="cuda")
            out_s = torch.full(bufs[-1].shape, -7.0, device="cuda")
            owned(x, w, out_o)
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            static(x, w, out_s)
            static(x, w, out_s)                 # back to back on one stream: counters return to zero
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
            assert torch.equal(out_o, out_s), args
            ref = torch.nn.functional.conv2d(x.double(), w.double(), stride=args[6], padding=args[7],
                                             dilation=args[8], groups=args[9])
            assert float((out_s.double() - ref).abs().max() / ref.abs().max()) <= 1e-5
            owned.close()
            static.close()


def test_static_workspace_rejects_what_does_not_fit():
    if COMPILE_ONLY:
        pytest.skip("compile only")
    L = rt.lib()
    src = 'extern "C" __global__ void k(unsigned* p) { p[threadIdx.x] = 1u; }'
    mod = rt.Module.from_source(src, "k")
    launch = rt.Launch(mod, (1,), (64,), [ctypes.c_void_p(0)])
    for off, nbytes in ((0, rt.STATIC_WS_BYTES + 16), (rt.STATIC_WS_BYTES, 16), (128, 16), (0, 8)):
        with pytest.raises(rt.RuntimeError_):
            rt.launch_seq_static_ws([launch], [(0, 0, off, nbytes, 1)])
    with pytest.raises(rt.RuntimeError_):
        rt.launch_seq_static_ws([launch], [(1, 0, 0, 256, 1)])
    rt.launch_seq_static_ws([launch], [(0, 0, rt.STATIC_WS_BYTES - 256, 256, 1)])   # the last 256 bytes
    torch.cuda.synchronize()
    assert L.ftr_last_error() is not None
    mod.close()
