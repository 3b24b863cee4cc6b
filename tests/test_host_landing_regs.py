"""The gate/up row-tile kernel (fm_pf_rows) requests a task's scales and biases one task
ahead with loads that land in v[240:255], registers its inline statements name themselves,
and copies them out behind the wait that covers those loads.  That is only sound while the
compiler's own values never live in those sixteen registers: this test compiles the kernels
to gfx950 assembly (no GPU needed) and reads every instruction of every instantiation.

Why the registers are named at all: a value that an asynchronous load is still writing must
not sit in a register the compiler allocates.  With compiler-allocated outputs the kernel was
compiled with the "next task" value in one register block inside the loop and another at the
loop header, and the copy between them, at the back edge, ran before the wait: a late load
then left stale scales in the copy (a chunk's result changed from one call to the next)."""
import os
import re
import subprocess

import pytest

from finchmoe_amd import build as fb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LAND_LO, LAND_HI = 240, 255


def _vregs(code):
    out = [(int(m.group(1)), int(m.group(2))) for m in re.finditer(r"\bv\[(\d+):(\d+)\]", code)]
    out += [(int(m.group(1)), int(m.group(1))) for m in re.finditer(r"\bv(\d+)\b", code)]
    return out


def _device_asm(src, tmp):
    """{function: [instruction text or ';;#ASMSTART' / ';;#ASMEND' marker]} of one source."""
    if not os.path.exists(fb.HIPCC):
        pytest.skip("no hipcc")
    out = os.path.join(str(tmp), src + ".s")
    flags = [f for f in fb.FLAGS if f not in ("-fPIC", "-fvisibility=hidden")]
    cmd = [fb.HIPCC] + flags + ["--offload-device-only", "-S", "-I", os.path.join(ROOT, "include"),
                                os.path.join(fb.CSRC, src), "-o", out]
    subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    funcs, cur = {}, None
    for ln in open(out):
        m = re.match(r"^(_Z\S+|fm_\w+):", ln)
        if m:
            cur = m.group(1)
            funcs[cur] = []
        elif cur is not None:
            if ln.startswith(".Lfunc_end"):
                cur = None
            else:
                t = ln.strip()
                funcs[cur].append(t if t.startswith(";;#ASM") else ln.split(";")[0].strip())
    os.unlink(out)
    return funcs


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    funcs = _device_asm("fm_prefill.hip", tmp_path_factory.mktemp("asm"))
    rows = {k: v for k, v in funcs.items() if "fm_pf_rowsILi" in k}
    assert len(rows) == 12, sorted(rows)          # {gate/up bf16 X, gate/up fp32 X, down} x {3,4} bits x {bf16,fp16}
    return rows


def test_landing_registers_are_named_by_the_loads_and_the_copy_only(kernels):
    for name, body in kernels.items():
        gate_up = "fm_pf_rowsILi0E" in name
        loads = copies = 0
        for code in body:
            if not code or code.startswith(".") or code.startswith(";;#"):
                continue
            touched = [r for r in _vregs(code) if r[1] >= LAND_LO]
            if not touched:
                continue
            assert gate_up, (name, code)           # the down kernel never reaches them
            op = code.split()[0]
            if op == "global_load_dwordx4":
                m = re.match(r"global_load_dwordx4 v\[(\d+):(\d+)\], v(\d+), s\[\d+:\d+\]$", code)
                assert m and LAND_LO <= int(m.group(1)) and int(m.group(2)) <= LAND_HI and int(m.group(3)) < LAND_LO, (name, code)
                loads += 1
            else:
                m = re.match(r"v_mov_b32(?:_e32)? v(\d+), v(\d+)$", code)
                assert m and int(m.group(1)) < LAND_LO <= int(m.group(2)) <= LAND_HI, (name, code)
                copies += 1
        if gate_up:
            assert loads >= 8 and loads % 4 == 0 and copies == 16, (name, loads, copies)


def test_copy_out_sits_directly_behind_the_waits(kernels):
    """Walking back from the sixteen copies, only scalar instructions and labels (the choice
    between the alternative waits) come before the waits on the load counter: no vector or
    LDS instruction, and so no other use of a register, lies between wait and copy."""
    for name, body in kernels.items():
        if "fm_pf_rowsILi0E" not in name:
            continue
        first = next(i for i, c in enumerate(body) if re.match(r"v_mov_b32(?:_e32)? v\d+, v240$", c))
        waits = 0
        for c in body[:first][::-1]:
            if not c or c.endswith(":") or c.startswith(";;#"):
                continue
            if c.startswith("s_waitcnt") and "vmcnt" in c:
                waits += 1
                continue
            if not c.startswith("s_"):
                break
        assert waits >= 2, (name, waits)


def test_no_accumulation_registers_in_the_row_tile_kernels(kernels):
    for name, body in kernels.items():
        for code in body:
            if code.startswith(".") or code.startswith(";;#"):
                continue
            assert not re.search(r"\ba\[?\d", code), (name, code)


@pytest.mark.parametrize("src", [s for s in fb.SOURCES if s != "fm_api.hip"])
def test_nothing_touches_the_destination_of_an_inline_load_before_a_wait(src, tmp_path):
    """Every kernel, read top to bottom: the registers an inline statement's LDS read, lane
    permutation or memory load writes are named by no later instruction until a wait on that
    counter has passed (lgkmcnt(0) for LDS, any vmcnt wait for memory)."""
    for name, body in _device_asm(src, tmp_path).items():
        pend_l, pend_v, inside = set(), set(), False
        for c in body:
            if c.startswith(";;#ASMSTART") or c.startswith(";;#ASMEND"):
                inside = c.startswith(";;#ASMSTART")
                continue
            if not c or c.endswith(":") or c.startswith("."):
                continue
            op = c.split()[0]
            if op == "s_waitcnt":
                if "lgkmcnt(0)" in c:
                    pend_l = set()
                if "vmcnt(" in c:
                    pend_v = set()
                continue
            regs = set()
            for lo, hi in _vregs(c):
                regs |= set(range(lo, hi + 1))
            if inside and (op.startswith("ds_read") or op.startswith("ds_bpermute")):
                dst = set()
                for lo, hi in _vregs(c.split()[1]):
                    dst |= set(range(lo, hi + 1))
                assert not (regs - dst) & (pend_l | pend_v), (name, c)
                pend_l |= dst
                continue
            if inside and re.match(r"(global|buffer|flat)_load", op) and "lds" not in op:
                dst = set()
                for lo, hi in _vregs(c.split()[1]):
                    dst |= set(range(lo, hi + 1))
                assert not (regs - dst) & (pend_l | pend_v), (name, c)
                pend_v |= dst
                continue
            assert not regs & (pend_l | pend_v), (name, c)
