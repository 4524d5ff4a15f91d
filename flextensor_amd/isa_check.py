"""Static checks of generated gfx950 ISA.

1. A software-managed hazard: a read (or an overwrite by another instruction)
of an MFMA's result registers before the matrix core has written them.
2. The hand-off of balanced K streaming: on every path from a store to a
workspace slot (a device-scope store, ``sc1``) to the next arrival count (a
``global_atomic_add``) the wavefront waits for its stores (``s_waitcnt``
with ``vmcnt(0)``) and then passes an ``s_barrier``; neither a barrier nor a
workgroup-scope fence waits for vector stores by itself.

3. Lane shifts under a narrowed execution mask: a DPP instruction reads a
neighbouring lane's register, and a lane that a divergent branch has switched
off cannot be read (the reader keeps its old value). The compiler is free to
sink a shift into the arm of a select; the depthwise kernels therefore compute
their shifts before any select, and this check looks for a DPP instruction
between an ``s_and_saveexec`` and the instruction that restores ``exec``.

4. Register copies ahead of an execution-mask restore. The join block of a divergent
``if`` begins with ``s_or_b64 exec, exec, <saved>``. Under register pressure the compiler
has placed its own copies of unrelated live values (live-range splits, spills into
accumulation registers) at the top of that block, in front of the restore, where only the
lanes that took the branch execute them: the other lanes keep stale registers. The sign in
the assembly text is a basic block whose vector instructions up to the restore are nothing
but register-to-register copies.

For 1: the hardware does not interlock this case; the compiler pads it with s_nop,
but its padding follows the control-flow graph with a visited set per block
and can lose a short path. This module rebuilds the graph from the assembly
text and walks every path forward from each MFMA for the required number of
issue slots.

    python -m flextensor_amd.isa_check [tuned.log]     # every MFMA kernel of a key:json log

needs hipcc (the kernels are compiled to assembly text on the host; no GPU)."""
import os
import re
import shutil
import subprocess
import sys
import tempfile

# issue slots before another instruction may read the result, as the compiler's own hazard table
# for gfx950 enforces them in straight-line code: passes + 2 for the fp32 shapes (16 and 8 passes),
# passes + 4 for the integer ones (32x32x32: 8 passes, 16x16x64: 4 passes; the distances it leaves
# between such an MFMA and a v_accvgpr_read of its result are exactly 12 and 8). A larger number
# here would flag the compiler's correct code; the point of the walk is to find the paths on which
# its padding got lost.
NEED = {"f32_32x32x2": 18, "f32_16x16x4": 10, "i32_32x32x32": 12, "i32_16x16x64": 8}
REG = re.compile(r"\b([av])(?:\[(\d+):(\d+)\]|(\d+)\b)")
BRANCH = re.compile(r"^s_(branch|cbranch_\w+)\s+(\S+)")


def _regs(text):
    out = set()
    for m in REG.finditer(text):
        kind = m.group(1)
        if m.group(4) is not None:
            out.add((kind, int(m.group(4))))
        else:
            out.update((kind, i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def parse(asm_text, kernel):
    """Instructions of one kernel: list of (mnemonic, operand text), label -> index."""
    lines = asm_text.split("\n")
    start = next(i for i, l in enumerate(lines) if l.startswith(kernel + ":"))
    insts, labels = [], {}
    for l in lines[start + 1:]:
        s = l.split(";")[0].strip()
        if l.startswith(".Lfunc_end") or s.startswith(".Lfunc_end") or s == "s_endpgm" and False:
            break
        if not s:
            continue
        if s.endswith(":"):
            labels[s[:-1]] = len(insts)
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        insts.append((parts[0], parts[1] if len(parts) > 1 else ""))
    return insts, labels


def _slots(inst):
    if inst[0] == "s_nop":
        return int(inst[1].strip(), 0) + 1
    return 1


def _reads(inst):
    """Registers an instruction reads (every operand but the destination of
    an instruction that has one; stores and MFMA sources read all of theirs)."""
    name, ops = inst
    if not ops:
        return set()
    parts = [p.strip() for p in ops.split(",")]
    if name.startswith(("global_store", "buffer_store", "ds_write", "flat_store", "scratch_store", "global_atomic")):
        return _regs(ops)
    return _regs(",".join(parts[1:]))


def find_early_reads(asm_text, kernel):
    """List of (mfma index, reader index, slots between) for reads that come too early."""
    insts, labels = parse(asm_text, kernel)
    found = []
    for i, (name, ops) in enumerate(insts):
        if not name.startswith("v_mfma"):
            continue
        shape = next((k for k in NEED if k in name), None)
        if shape is None:
            raise ValueError("unknown MFMA shape: " + name)
        need = NEED[shape]
        dst = _regs(ops.split(",")[0])
        # walk forward over every path until `need` slots have passed
        stack, seen = [(i + 1, 0)], {}
        while stack:
            j, used = stack.pop()
            while j < len(insts) and used < need:
                if seen.get(j, need + 1) <= used:
                    break
                seen[j] = used
                jn, jo = insts[j]
                if jn.startswith("v_mfma"):
                    # the next MFMA: reading the result as its own accumulator is interlocked;
                    # as a multiplicand it is not
                    parts = [p.strip() for p in jo.split(",")]
                    if _regs(",".join(parts[1:3])) & dst:
                        found.append((i, j, used))
                    if _regs(parts[0]) & dst:
                        break        # the registers get a new producer: this walk ends
                elif _reads((jn, jo)) & dst:
                    found.append((i, j, used))
                    break
                elif jn.startswith(("v_", "ds_read", "global_load", "buffer_load")) and not jn.startswith("v_cmp") \
                        and _regs(jo.split(",")[0]) & dst:
                    # another instruction writes a result register while the MFMA may still be
                    # writing it: the same distance applies to this write-after-write
                    found.append((i, j, used))
                    break
                b = BRANCH.match(jn + " " + jo)
                used += _slots((jn, jo))
                if b:
                    target = labels.get(b.group(2))
                    if target is not None:
                        stack.append((target, used))
                    if b.group(1) == "branch":
                        break
                if jn == "s_endpgm":
                    break
                j += 1
    return found, insts


def _successors(insts, labels, j):
    """Indices control can reach from instruction j."""
    name, ops = insts[j]
    if name == "s_endpgm":
        return []
    b = BRANCH.match(name + " " + ops)
    out = []
    if b:
        target = labels.get(b.group(2))
        if target is not None:
            out.append(target)
        if b.group(1) == "branch":
            return out
    if j + 1 < len(insts):
        out.append(j + 1)
    return out


def find_unordered_arrivals(asm_text, kernel, single_wavefront=False):
    """[(slot store index, arrival index)] for arrival counts that a slot store can
    reach without the wavefront having waited for its stores and passed a barrier.
    A workgroup of one wavefront has nobody to collect (the compiler drops the barrier
    instruction): there the wait alone is asked for."""
    insts, labels = parse(asm_text, kernel)
    found = []
    enough = 1 if single_wavefront else 2
    for i, (name, ops) in enumerate(insts):
        if not (name.startswith("global_store") and re.search(r"\bsc1\b", ops)):
            continue
        # stage 0: store outstanding; 1: waited for; 2: waited for and a barrier passed
        stack, seen = [(j, 0) for j in _successors(insts, labels, i)], set()
        while stack:
            j, stage = stack.pop()
            if (j, stage) in seen:
                continue
            seen.add((j, stage))
            jn, jo = insts[j]
            if jn.startswith("global_atomic_add"):
                if stage < enough:
                    found.append((i, j))
                continue                      # the arrival is counted: this walk ends
            if jn.startswith("global_store") and re.search(r"\bsc1\b", jo):
                stage = 0                     # a later slot store is outstanding again
            elif jn == "s_waitcnt" and re.search(r"\bvmcnt\(0\)", jo):
                stage = max(stage, 1)
            elif jn == "s_barrier" and stage == 1:
                stage = 2
            stack.extend((k, stage) for k in _successors(insts, labels, j))
    return found, insts


NARROWS = re.compile(r"^s_(and|andn2|xor)_saveexec_b64$")


def _restores_exec(name, ops):
    """exec is whole again: or-ed with the saved mask, or re-loaded."""
    return name in ("s_or_b64", "s_mov_b64", "s_or_saveexec_b64") and re.match(r"\s*exec\b", ops) is not None


def find_masked_lane_shifts(asm_text, kernel):
    """[(mask instruction index, DPP instruction index)] for DPP instructions that control
    can reach from an instruction that narrows exec before exec is restored."""
    insts, labels = parse(asm_text, kernel)
    found = []
    for i, (name, ops) in enumerate(insts):
        if not NARROWS.match(name):
            continue
        stack, seen = list(_successors(insts, labels, i)), set()
        while stack:
            j = stack.pop()
            if j in seen:
                continue
            seen.add(j)
            jn, jo = insts[j]
            if _restores_exec(jn, jo):
                continue
            if jn.endswith("_dpp"):
                found.append((i, j))
            stack.extend(_successors(insts, labels, j))
    return found, insts


BLOCK_START = re.compile(r"^\s*(\.LBB\d+_\d+:|; %bb\.\d+:)")
VECTOR = re.compile(r"^(v_|ds_|buffer_|global_|scratch_|flat_)")
LANE_ACCESS = ("v_readlane", "v_writelane")          # SGPR spills: these ignore exec
COPY = re.compile(r"^(v_mov_b32_e32 v\d+, v\d+|v_mov_b64_e32 v\[\d+:\d+\], v\[\d+:\d+\]"
                  r"|v_accvgpr_(write|read|mov)_b32 [av]\d+, [av]\d+)$")


def find_copies_ahead_of_exec_restore(asm_text, kernel):
    """[(line number of the restore, [copy instructions])] for basic blocks in which
    nothing but register copies stands between the block's start and its
    ``s_or_b64 exec, exec, ...``. (A block that does real work under the narrowed mask
    and then restores it, a predicated store merged with its join block, is the
    ordinary case and is not reported.)"""
    lines = asm_text.split("\n")
    start = next(i for i, l in enumerate(lines) if l.startswith(kernel + ":"))
    found, vec = [], []
    for n, l in enumerate(lines[start + 1:], start + 2):
        if l.startswith(".Lfunc_end"):
            break
        if BLOCK_START.match(l):
            vec = []
            continue
        s = l.split(";")[0].strip()
        if not s or s.startswith(".") or s.endswith(":"):
            continue
        name = s.split(None, 1)[0]
        if name == "s_or_b64" and re.match(r"\s*exec\b", s[len(name):]):
            if vec and all(COPY.match(x) for x in vec):
                found.append((n, list(vec)))
            vec = []
        elif VECTOR.match(name) and not name.startswith(LANE_ACCESS):
            vec.append(s)
    return found


HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def assembly_of(spec, workdir=None):
    """Assembly text of one KernelSpec for gfx950 (hipcc -S with the options hiprtc gets)."""
    d = workdir or tempfile.mkdtemp(prefix="ft_isa_")
    src, out = os.path.join(d, "kernel.hip"), os.path.join(d, "kernel.s")
    with open(src, "w") as f:
        f.write(spec.source())
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-S", "--cuda-device-only", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-include", "hip/hip_runtime.h", "-o", out, src] + spec.options()
    subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    with open(out) as f:
        text = f.read()
    if workdir is None:
        shutil.rmtree(d, ignore_errors=True)
    return text


def check_plan(plan):
    """[(kernel, first instruction, second instruction, detail)] over the kernels of a plan:
    early reads of MFMA results (detail = issue slots between), arrival counts of the
    K-streaming exchange that do not wait for the slot stores (detail = "arrival"), in
    the depthwise kernels DPP lane shifts under a narrowed exec mask (detail = "masked shift"),
    and in all of them register copies ahead of an exec restore (detail = "masked copy";
    the two instructions are then the first copy and the line number of the restore)."""
    out = []
    for spec in plan.specs:
        if spec.kernel not in ("igemm_f32", "gemm_i8", "depthwise_f32"):
            continue
        text = assembly_of(spec)
        out.extend((spec.kernel, (copies[0], ""), ("s_or_b64", "exec, line %d" % n), "masked copy")
                   for n, copies in find_copies_ahead_of_exec_restore(text, spec.kernel))
        if spec.kernel == "depthwise_f32":
            found, insts = find_masked_lane_shifts(text, spec.kernel)
            out.extend((spec.kernel, insts[i], insts[j], "masked shift") for i, j in found)
            continue
        found, insts = find_early_reads(text, spec.kernel)
        out.extend((spec.kernel, insts[i], insts[j], used) for i, j, used in found)
        if spec.defines.get("SK_PER", 0):
            threads = spec.block[0] * spec.block[1] * spec.block[2]
            found, insts = find_unordered_arrivals(text, spec.kernel, single_wavefront=threads <= 64)
            out.extend((spec.kernel, insts[i], insts[j], "arrival") for i, j in found)
    return out


def main(argv):
    from .scheduler import schedule_with_config
    from .task import TASK_TABLE
    from .tuned import LOG, load
    table = load(argv[1] if len(argv) > 1 else LOG)
    seen, bad = set(), 0
    for key, cfg in table.items():
        if key not in TASK_TABLE:
            print("skipped (not registered):", key)
            continue
        plan, _ = schedule_with_config(key, cfg)
        sig = tuple((sp.template, tuple(sp.options())) for sp in plan.specs)
        if sig in seen:
            continue
        seen.add(sig)
        for kernel, mfma, reader, used in check_plan(plan):
            bad += 1
            if used == "arrival":
                print("UNORDERED ARRIVAL %s %s: %s %s -> %s %s" % ((key, kernel) + mfma + reader))
            elif used == "masked copy":
                print("REGISTER COPY AHEAD OF AN EXEC RESTORE %s %s: %s %s -> %s %s" % ((key, kernel) + mfma + reader))
            elif used == "masked shift":
                print("LANE SHIFT UNDER A NARROWED EXEC MASK %s %s: %s %s -> %s %s" % ((key, kernel) + mfma + reader))
            else:
                print("EARLY READ %s %s: %s %s -> %s %s after %d slots" % ((key, kernel) + mfma + reader + (used,)))
    print("%d plans checked, %d findings" % (len(seen), bad))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
