"""The distance between the last MFMA of the main loop and the first read of
its result registers, checked in the generated ISA (no GPU needed).

A 16-pass MFMA's results may not be read for 19 issue slots and the hardware
does not interlock. In the segment loop of balanced K streaming the compiler's
padding missed the short branch from the main loop to the tile store; the
templates therefore place the slots themselves. This test compiles the
configuration that once failed and looks at the instruction stream."""
import os
import re
import shutil
import subprocess

import pytest

from flextensor_amd import isa_check as isa_hazards

from flextensor_amd.scheduler import schedule_with_config
from flextensor_amd.task import TASK_TABLE  # noqa: F401  (registers the tasks)
from flextensor_amd.utils import Config, ceil_div

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
KEYS = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]


def _isa(spec, tmp_path):
    src = tmp_path / "kernel.hip"
    src.write_text(spec.source())
    out = tmp_path / "kernel.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-S", "--cuda-device-only", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-include", "hip/hip_runtime.h", "-o", str(out), str(src)] + spec.options()
    subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    return out.read_text().split("\n")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_k_streaming_tile_store_waits_for_the_last_mfma(tmp_path):
    key = "conv2d_baseline2_(8, 512, 7, 7, 2048, 1, 1, 0, 1, 1)_rocm(0)"
    M, N, K = 2048, 392, 512
    c = {k: [] for k in KEYS}
    c["spatial"] = [[ceil_div(M, 64), 2, 1, 32], [ceil_div(N, 32), 1, 1, 32]]
    c["reduce"], c["unroll"], c["fuse"], c["reorder"] = [[1, K // 64, 64]], [[5, 1]], [[1]], [[0, 0, 1]]
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[1, 0]], [[-1, 0]]
    plan, _ = schedule_with_config(key, Config([{k: [] for k in KEYS}, c], g))
    spec = plan.specs[-1]
    assert spec.defines["SK_PER"] > 0 and spec.defines["DTL"] == 1 and spec.defines["MFMA"] == 32
    lines = _isa(spec, tmp_path)
    mfma = [i for i, l in enumerate(lines) if "v_mfma_f32_32x32x2" in l]
    assert mfma, "no MFMA in the kernel"
    last = mfma[-1]
    nop = [i for i, l in enumerate(lines) if re.search(r"\bs_nop 15\b", l) and i > last]
    reads = [i for i, l in enumerate(lines) if "v_accvgpr_read" in l and i > last]
    assert nop and reads
    # the explicit slots (16 + 4) stand between the loop and every later accumulator read
    assert re.search(r"\bs_nop 3\b", lines[nop[0] + 1])
    assert last < nop[0] < reads[0]
    # and nothing reads an accumulator between the loop's first MFMA and its last
    assert not [i for i, l in enumerate(lines) if "v_accvgpr_read" in l and mfma[0] < i < last]
    # every path from every MFMA, with the control-flow graph rebuilt from the text
    found, _ = isa_hazards.find_early_reads("\n".join(lines), "igemm_f32")
    assert found == []


SNIPPET = """
k:
	v_mfma_f32_32x32x2_f32 a[0:15], v1, v2, a[0:15]
	s_cbranch_scc1 .LBB0_2
	s_nop 15
	s_nop 1
	v_accvgpr_read_b32 v3, a15
	s_endpgm
.LBB0_2:
	s_add_i32 s0, s0, 1
%s	v_accvgpr_read_b32 v4, a0
	s_endpgm
.Lfunc_end0:
"""


def test_checker_follows_branches_and_counts_nops():
    found, insts = isa_hazards.find_early_reads(SNIPPET % "", "k")
    assert [(insts[j][1], used) for _, j, used in found] == [("v4, a0", 2)]       # the padded fall-through passes
    found, _ = isa_hazards.find_early_reads(SNIPPET % "\ts_nop 15\n", "k")
    assert found == []
    # the next MFMA may accumulate onto the result at once, but not multiply with it
    chain = "k:\n\tv_mfma_f32_16x16x4_f32 v[0:3], v8, v9, v[0:3]\n\tv_mfma_f32_16x16x4_f32 v[0:3], v8, v9, v[0:3]\n" \
            "\tv_mfma_f32_16x16x4_f32 v[4:7], v0, v9, v[4:7]\n\ts_endpgm\n.Lfunc_end0:\n"
    found, insts = isa_hazards.find_early_reads(chain, "k")
    assert [(i, j) for i, j, _ in found] == [(1, 2)]
    # an early overwrite of the result registers by another instruction counts as well
    waw = "k:\n\tv_mfma_f32_16x16x4_f32 a[0:3], v8, v9, a[0:3]\n\ts_nop 3\n\tv_accvgpr_write_b32 a2, 0\n\ts_endpgm\n.Lfunc_end0:\n"
    found, _ = isa_hazards.find_early_reads(waw, "k")
    assert [(i, j, used) for i, j, used in found] == [(0, 2, 4)]
    found, _ = isa_hazards.find_early_reads(waw.replace("s_nop 3", "s_nop 9"), "k")
    assert found == []


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_benchmark_kernels_have_no_early_accumulator_reads(tmp_path):
    """Every MFMA kernel of the shipped benchmark configurations, all paths."""
    import __graft_entry__ as g
    from flextensor_amd.tuned import lookup
    checked = 0
    for n, key in enumerate(g.BENCH_KEYS):
        plan, _ = schedule_with_config(key, lookup(key))
        for spec in plan.specs:
            if spec.kernel not in ("igemm_f32", "gemm_i8"):
                continue
            d = tmp_path / str(n)
            d.mkdir()
            found, insts = isa_hazards.find_early_reads("\n".join(_isa(spec, d)), spec.kernel)
            assert found == [], (key, [(insts[i], insts[j], used) for i, j, used in found[:3]])
            checked += 1
    assert checked == 5


ARRIVAL = """
k:
	global_store_dword v1, v2, s[0:1] sc1
	s_cbranch_scc1 .LBB0_2
%s	s_barrier
	global_atomic_add v3, v4, v5, s[2:3] sc0
	s_endpgm
.LBB0_2:
	s_waitcnt vmcnt(0)
	s_barrier
	global_atomic_add v3, v4, v5, s[2:3] sc0
	s_endpgm
.Lfunc_end0:
"""


def test_arrival_checker_wants_a_wait_then_a_barrier_on_every_path():
    found, insts = isa_hazards.find_unordered_arrivals(ARRIVAL % "", "k")
    assert [(i, insts[j][0]) for i, j in found] == [(0, "global_atomic_add")] and found[0][1] == 3
    found, _ = isa_hazards.find_unordered_arrivals(ARRIVAL % "\ts_waitcnt lgkmcnt(0)\n", "k")
    assert len(found) == 1                                    # a wait for LDS only does not count
    found, _ = isa_hazards.find_unordered_arrivals(ARRIVAL % "\ts_waitcnt vmcnt(0) lgkmcnt(0)\n", "k")
    assert found == []
    # the wait has to come before the barrier, not after it
    late = ARRIVAL.replace("%s\ts_barrier\n", "\ts_barrier\n\ts_waitcnt vmcnt(0)\n")
    found, _ = isa_hazards.find_unordered_arrivals(late, "k")
    assert len(found) == 1


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_k_streaming_arrivals_wait_for_the_slot_stores(tmp_path):
    """Both ways a tile can travel to LDS, on the shipped K-streaming entry and on a
    register-staged variant of it: every slot store is waited for before its arrival is
    counted, in the run's last segment and in the prologue of a following one."""
    from flextensor_amd.tuned import lookup
    key = "conv2d_baseline1_(8, 256, 14, 14, 512, 3, 1, 1, 1, 1)_rocm(0)"
    shipped = lookup(key)
    staged = Config([dict(c) for c in shipped.op_config_lst], dict(shipped.graph_config))
    staged.op_config_lst[1]["unroll"] = [[3, 1]]
    staged.op_config_lst[1]["reduce"] = [[1, 72, 32]]
    for n, cfg in enumerate((shipped, staged)):
        plan, _ = schedule_with_config(key, cfg)
        spec = plan.specs[-1]
        assert spec.defines["SK_PER"] > 0
        d = tmp_path / str(n)
        d.mkdir()
        text = "\n".join(_isa(spec, d))
        assert re.search(r"global_store_dword.*sc1", text) and "global_atomic_add" in text
        found, insts = isa_hazards.find_unordered_arrivals(text, spec.kernel)
        assert found == [], [(insts[i], insts[j]) for i, j in found[:3]]


MASKED = """k:
\tv_cmp_ne_u32_e32 vcc, 0, v12
\tv_mov_b32_e32 v23, 0
%s.LBB0_2:
\ts_or_b64 exec, exec, s[2:3]
\tv_mov_b32_dpp v24, v7 wave_shl:1 row_mask:0xf bank_mask:0xf
\ts_endpgm
.Lfunc_end0:
"""


def test_lane_shift_checker_flags_a_shift_behind_a_narrowed_mask():
    branchy = ("\ts_and_saveexec_b64 s[2:3], vcc\n\ts_cbranch_execz .LBB0_2\n"
               "\tv_mov_b32_dpp v23, v11 wave_shr:1 row_mask:0xf bank_mask:0xf\n")
    found, insts = isa_hazards.find_masked_lane_shifts(MASKED % branchy, "k")
    # the shift inside the branch is found; the one after exec is whole again is not
    assert [(insts[i][0], insts[j][1].split()[0]) for i, j in found] == [("s_and_saveexec_b64", "v23,")]
    plain = "\tv_mov_b32_dpp v23, v11 wave_shr:1 row_mask:0xf bank_mask:0xf\n\tv_cndmask_b32_e32 v23, 0, v23, vcc\n"
    found, _ = isa_hazards.find_masked_lane_shifts(MASKED % plain, "k")
    assert found == []


JOIN = """k:
\tv_bfrev_b32_e32 v60, 1
\ts_and_saveexec_b64 s[18:19], s[34:35]
; %%bb.229:
\tv_mul_i32_i24_e32 v56, 11, v56
\tv_lshl_add_u32 v60, v56, 2, v59
; %%bb.230:
%s\ts_or_b64 exec, exec, s[18:19]
\tbuffer_load_dword a233, v60, s[56:59], 0 offen
\ts_and_saveexec_b64 s[4:5], s[6:7]
\ts_cbranch_execz .LBB0_2
; %%bb.231:
\tv_mov_b32_e32 v5, v7
\tglobal_store_dword v[126:127], v5, off
.LBB0_2:
\ts_or_b64 exec, exec, s[4:5]
\ts_endpgm
.Lfunc_end0:
"""


def test_copy_checker_flags_copies_between_a_join_block_and_its_exec_restore():
    """The form the compiler produced in a register-starved gather kernel: copies of unrelated live
    values at the top of the join block, ahead of the restore, so that only the lanes of the branch
    execute them. A block that works under the mask and restores it at its own end is not that."""
    split = "\tv_accvgpr_write_b32 a18, v240\n\tv_mov_b32_e32 v28, v93\n\ts_mov_b64 s[42:43], s[40:41]\n"
    found = isa_hazards.find_copies_ahead_of_exec_restore(JOIN % split, "k")
    assert [copies for _, copies in found] == [["v_accvgpr_write_b32 a18, v240", "v_mov_b32_e32 v28, v93"]]
    assert isa_hazards.find_copies_ahead_of_exec_restore(JOIN % "", "k") == []
    # SGPR spills into lanes ignore exec and do not count
    lanes = "\tv_writelane_b32 v254, s18, 46\n"
    assert isa_hazards.find_copies_ahead_of_exec_restore(JOIN % lanes, "k") == []


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_register_starved_gather_kernel_has_no_divergent_address_arithmetic():
    """224 columns, two register sets of 56 gathered elements each, 112 accumulators: the kernel in
    which the copies were found (wrong rows in the tiles loaded inside the loop). The offsets are
    selects now, so the address set-up has no divergent branch for the compiler to split around."""
    from flextensor_amd.task import Task, conv2d, register
    args = (3, 6, 11, 11, 20, 3, 1, 2, 2, 1)
    register(conv2d, "conv2d", "rnd", args, "rocm", 0)
    key = Task("conv2d", "rnd", None, args, "rocm", 0).key
    c = {k: [] for k in KEYS}
    c.update(fuse=[[8]], spatial=[[1, 1, 1, 32], [2, 1, 7, 32]], reduce=[[1, 4, 16]], reorder=[[0, 1, 0]],
             unroll=[[3, 1]])
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[1, 0]], [[4, -1]]
    plan, _ = schedule_with_config(key, Config([{k: [] for k in KEYS}, c], g))
    text = isa_hazards.assembly_of(plan.specs[-1])
    first_mfma = text.index("v_mfma")
    assert "s_and_saveexec" not in text[:first_mfma]
    assert isa_hazards.check_plan(plan) == []


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("special", [[[1], [0], [0], [1], [2]],      # row exchange (the shipped variant)
                                     [[1], [0], [0], [1], [3]],      # ragged last span
                                     [[1], [1], [0], [1], [0]],      # direct kernel, shuffled halo
                                     [[1], [1], [0], [3], [0]]])     # the same, three patches per lane
def test_depthwise_lane_shifts_run_with_every_lane_switched_on(special):
    key = "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)"
    c = {k: [] for k in KEYS}
    c["spatial"] = [[8, 1, 1, 1], [512, 1, 1, 1], [28, 1, 1, 1], [7, 1, 1, 4]]
    c["fuse"] = [[4]]
    g = {k: [] for k in KEYS}
    g["inline"], g["special"] = [[1, 0]], special
    plan, _ = schedule_with_config(key, Config([{k: [] for k in KEYS}, c], g))
    text = isa_hazards.assembly_of(plan.specs[-1])
    assert "_dpp" in text, "the kernel is expected to shift lanes with DPP"
    assert isa_hazards.check_plan(plan) == []


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("shape_index", [0, 3, 4, 7, 8, 11, 13, 14, 18, 20, 22, 25, 27, 29])
def test_random_points_of_the_spaces_pass_the_static_checks(shape_index):
    """The generated assembly of points drawn at random from the schedule spaces (the same points
    the device parity test runs): no accumulator read before the matrix core has written it, no
    arrival counted ahead of the slot stores, no lane shift under a narrowed exec mask, no register
    copies between a join block's start and its exec restore."""
    from random_points import point
    for number in (0, 4):
        kind, key, args, configs, plan = point(shape_index, number)
        assert isa_hazards.check_plan(plan) == [], (key, configs)
