"""Random points of the schedule spaces against the CPU oracle.

The hand-picked cases of test_gpu_parity.py cover the knobs one by one; here
points are drawn from the operators' own spaces (the same sub-spaces the search
walks: tile splits, K splits, pipeline depths, traversal, K division, plus the
task-level knobs and the graph-level inline and merge flags), so that combinations
nobody thought of are run too. Points the templates refuse on the host are redrawn,
as the search does. The draw is seeded by the case, so the points are the same
in every process (and can be compiled ahead of time without a device).

Acceptance as everywhere: fp32 max|out - ref| / max|ref| <= 1e-5, int32 bit-exact.
"""
import os
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available() and os.environ.get("FT_TESTS_COMPILE_ONLY") != "1":
    pytest.skip("no GPU visible", allow_module_level=True)

from flextensor_amd.measure import seeded_inputs  # noqa: E402
from flextensor_amd.plan import build  # noqa: E402
from flextensor_amd.task import TASK_TABLE  # noqa: E402

from random_points import CASES, point as draw_point  # noqa: E402

TOL = 1e-5


@pytest.mark.parametrize("shape_index,point", CASES)
def test_random_point_vs_oracle(oracle, shape_index, point):
    kind, key, args, configs, plan = draw_point(shape_index, point)
    _, bufs = TASK_TABLE[key].func(*args)
    host = seeded_inputs(bufs, seed=shape_index * 31 + point)
    func_ = build(plan, bufs, "rocm")
    tdt = {"float32": torch.float32, "int32": torch.int32}[bufs[-1].dtype]
    out = torch.full(bufs[-1].shape, -77, dtype=tdt, device="cuda")
    func_(*[torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in host], out)
    torch.cuda.synchronize()
    func_.close()
    out = out.cpu().numpy()
    what = (key, [dict((k, v) for k, v in c.items() if v) for c in configs.op_config_lst], configs.graph_config)
    if kind == "int8":
        assert np.array_equal(out, oracle.gemm_i8_c(host[0], host[1])), what
        return
    if kind in ("gemm", "gemm_tn", "gemm_tt", "gemm_nt"):
        ref = oracle.gemm_f32_c(host[0], host[1], transA=kind[-2] == "t", transB=kind[-1] == "t")
    elif kind == "bgemm":
        ref = np.stack([oracle.gemm_f32_c(host[0][b], host[1][b]) for b in range(args[0])])
    elif kind in ("conv", "gconv", "convb"):
        ref = oracle.conv2d_nchw_c(host[0], host[1], args[6], args[7], args[8], args[9])
    else:
        ref = oracle.depthwise_nchw_c(host[0], host[1], args[6], args[7], args[8])
    if kind in ("convb", "dwb"):
        ref = oracle.bias_add_nchw_np(ref, host[2])
    ref = np.asarray(ref, np.float64)
    err = float(np.max(np.abs(out.astype(np.float64) - ref)) / np.max(np.abs(ref)))
    assert err <= TOL, (err,) + what
