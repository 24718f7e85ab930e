"""Static check of the compiled decode kernels for one hazard the compiler does not cover.

A VALU, LDS or memory instruction that reads the result of a matrix op (v_mfma) too early sees
the register's old contents.  Within straight-line code the compiler pads with wait states; it
does not when a taken branch sits between the matrix op and the first reader (observed: a
uniform `if` right after the score matrix ops made `v_max_f32` read stale scores, intermittently
wrong outputs for chunk_size 128).  The source therefore keeps branches away from matrix-op
results; this test compiles csrc/kernels.hip to assembly and fails if the pattern reappears:
a branch within a few instructions after a v_mfma whose target (or fall-through) reads the
matrix op's destination within its first few instructions.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "chunk-attention_amd", "csrc", "kernels.hip")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

AFTER_MFMA = 6     # instructions after a matrix op in which a branch is looked for
AT_TARGET = 6      # instructions at the branch target / fall-through that are inspected


def regs_of(operand: str):
    """Vector registers named by one operand: v12 or v[12:15]."""
    m = re.fullmatch(r"-?\|?v(\d+)\|?", operand)
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    return set()


def parse(path):
    """[(label or None, mnemonic, [operands])] for every instruction and label line."""
    out = []
    for line in open(path):
        line = line.split(";")[0].rstrip()
        if not line.strip():
            continue
        m = re.match(r"^([.\w$]+):\s*$", line)
        if m:
            out.append((m.group(1), None, []))
            continue
        if not line.startswith("\t") or line.strip().startswith("."):
            continue
        parts = line.strip().split(None, 1)
        ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        out.append((None, parts[0], ops))
    return out


def readers(insts, start, count, dst):
    """Instructions among the first `count` at `start` that read a register of `dst`
    (first operand = destination for everything but stores and matrix-op accumulate chains)."""
    found, seen = [], 0
    i = start
    while i < len(insts) and seen < count:
        label, mn, ops = insts[i]
        i += 1
        if mn is None:
            continue
        seen += 1
        if mn.startswith("s_") and not mn.startswith("s_waitcnt"):
            if mn in ("s_branch", "s_endpgm") or mn.startswith("s_cbranch"):
                break
            continue
        if mn.startswith("v_mfma"):
            continue   # matrix op to matrix op dependencies are interlocked in hardware
        srcs = ops if mn.startswith(("global_store", "ds_write", "scratch_store", "buffer_store")) else ops[1:]
        used = set()
        for o in srcs:
            used |= regs_of(o.split(" ")[0])
        if used & dst:
            found.append((mn, ops))
        if ops and not mn.startswith(("global_store", "ds_write")):
            dst = dst - regs_of(ops[0])   # overwritten: later reads are of the new value
    return found


@pytest.mark.skipif(not shutil.which(HIPCC) and not os.path.exists(HIPCC), reason="hipcc not available")
def test_no_branch_between_matrix_op_and_first_reader(tmp_path):
    asm = tmp_path / "kernels.s"
    import importlib.util
    spec = importlib.util.spec_from_file_location("ca_build", os.path.join(ROOT, "chunk-attention_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)           # the library's own compiler flags
    flags = [f for f in build.HIP_FLAGS if f != "-fPIC"]
    subprocess.check_call([HIPCC] + flags + ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.dirname(SRC), "-S",
                                             "--cuda-device-only", "-o", str(asm), SRC], stderr=subprocess.DEVNULL)
    insts = parse(asm)
    labels = {lab: i for i, (lab, mn, _) in enumerate(insts) if lab}
    n_mfma, problems = 0, []
    for i, (lab, mn, ops) in enumerate(insts):
        if not mn or not mn.startswith("v_mfma"):
            continue
        n_mfma += 1
        dst = regs_of(ops[0])
        seen, j = 0, i + 1
        while j < len(insts) and seen < AFTER_MFMA:
            l2, m2, o2 = insts[j]
            j += 1
            if m2 is None:
                continue
            seen += 1
            if m2.startswith("s_cbranch") or m2 == "s_branch":
                target = labels.get(o2[0])
                spots = [("target " + o2[0], target)] if target is not None else []
                if m2 != "s_branch":
                    spots.append(("fall-through", j))
                for name, at in spots:
                    for rmn, rops in readers(insts, at, AT_TARGET, set(dst)):
                        problems.append("%s %s -> %s after %s: %s %s" % (mn, ops[0], name, m2, rmn, ", ".join(rops)))
                break
    assert n_mfma > 100, "the kernels' matrix ops were not found in the assembly"
    assert not problems, "matrix-op result read right after a branch:\n" + "\n".join(problems[:20])
