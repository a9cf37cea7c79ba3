"""The short-K L_inf forward (csrc/inf_forward_shortk.hip) issues the loads of its input panel and the waits for
them as inline assembly, so the compiler does not know that a parked register has a load in flight.  That is safe
only as long as the generated code never reads such a register between the load and the wait that stands in front
of the panel write.  This test compiles the file to assembly (no GPU needed) and checks exactly that, for every
instantiation of the kernel."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "l_inf-dist-net_amd", "csrc", "inf_forward_shortk.hip")

LOAD = re.compile(r"^\s*buffer_load_dwordx4 v\[(\d+):(\d+)\], v(\d+), ")
WRITE = re.compile(r"^\s*ds_write_b128 v(\d+), v\[(\d+):(\d+)\]")
WAIT = re.compile(r"^\s*s_waitcnt vmcnt\((\d+)\)\s*$")


def library_flags():
    """The compiler flags of the library's Makefile (FLAGS := ... with its continuation line), ARCH filled in."""
    text = open(os.path.join(os.path.dirname(SRC), "Makefile")).read()
    arch = re.search(r"^ARCH\s*\?=\s*(\S+)", text, re.M).group(1)
    flags = re.search(r"^FLAGS\s*:=\s*((?:.*\\\n)*.*)$", text, re.M).group(1).replace("\\\n", " ")
    return flags.replace("$(ARCH)", arch).split()


def registers(text):
    """Vector registers named in an operand string."""
    regs = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(lo), int(hi) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", text))
    return regs


def kernels(asm):
    """name -> instruction lines (comments and directives dropped) of every shortk kernel in the listing."""
    out, name = {}, None
    for line in asm.splitlines():
        m = re.match(r"^(_ZN5ldist25inf_forward_shortk_kernelILi(\d+)E\S*):", line)
        if m:
            name = int(m.group(2))
            out[name] = []
            continue
        if name is None:
            continue
        code = line.split(";")[0].rstrip()
        if re.match(r"^\s+s_endpgm", code):
            out[name].append(code)
            name = None
            continue
        if re.match(r"^\s+[a-z]", code):
            out[name].append(code)
    return out


def check_kernel(nw, lines):
    loads = [i for i, l in enumerate(lines) if LOAD.match(l)]
    assert loads, "no buffer loads found"
    parks = set()
    for i in loads:
        lo, hi, _ = map(int, LOAD.match(lines[i]).groups())
        assert hi - lo == 3
        parks.update(range(lo, hi + 1))
    assert len(parks) == 4 * nw, (nw, sorted(parks))
    writes = 0
    pending = set()      # registers with a load in flight, in listing order (every straight run of the loop is in order)
    # the region in which the parked registers are live: first load .. last load (the tile loop and its prologue)
    for i in range(loads[0], loads[-1] + 1):
        line = lines[i]
        ld = LOAD.match(line)
        if ld:
            lo, hi, addr = map(int, ld.groups())
            assert addr not in pending, f"address register has a load in flight: {line.strip()}"
            assert not (set(range(lo, hi + 1)) & pending), f"second load into registers in flight: {line.strip()}"
            pending.update(range(lo, hi + 1))
            continue
        if not (registers(line) & parks):
            continue
        w = WRITE.match(line)
        if w and set(range(int(w.group(2)), int(w.group(3)) + 1)) <= parks:
            addr, lo, hi = map(int, w.groups())
            assert addr not in pending, line
            # the wait stands in front of the write; what the scheduler put between them must leave the data alone
            j = i - 1
            while not WAIT.match(lines[j]):
                assert not (registers(lines[j]) & set(range(lo, hi + 1))), (lines[j], line)
                j -= 1
                assert j >= loads[0], f"no wait in front of {line.strip()}"
            assert int(WAIT.match(lines[j]).group(1)) <= nw - 1, (lines[j], line)
            pending.difference_update(range(lo, hi + 1))
            writes += 1
            continue
        # anything else may use a parked register only while no load into it is in flight (the offset of the next
        # load is computed there, between the panel write and the load)
        assert not (registers(line) & pending), f"touches a register with a load in flight: {line.strip()}"
    assert writes == nw, (nw, writes)


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_read_of_a_parked_register_before_its_wait(tmp_path):
    out = tmp_path / "shortk.s"
    cmd = ["hipcc"] + library_flags() + ["-S", "--cuda-device-only", SRC, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    asm = out.read_text()
    found = kernels(asm)
    assert sorted(found) == list(range(1, 11))
    for nw, lines in found.items():
        check_kernel(nw, lines)
    # the window loop is unrolled over the parked registers: none of them may have gone to scratch memory
    spills = re.findall(r"\.vgpr_spill_count:\s*(\d+)", asm)
    assert len(spills) == 10 and all(int(n) == 0 for n in spills), spills


def test_the_check_itself_flags_an_early_read():
    good = ["\tbuffer_load_dwordx4 v[2:5], v9, s[0:3], s4 offen",
            "\tv_add_f32_e32 v20, v21, v22",
            "\ts_waitcnt vmcnt(0)",
            "\tds_write_b128 v30, v[2:5]",
            "\tv_cndmask_b32_e64 v2, -1, v40, s[4:5]",
            "\tbuffer_load_dwordx4 v[2:5], v2, s[0:3], s4 offen"]
    check_kernel(1, good)
    for bad_line in ("\tv_mov_b32_e32 v20, v3", "\tv_mov_b32_e32 v4, v20"):
        bad = good[:1] + [bad_line] + good[1:]
        with pytest.raises(AssertionError):
            check_kernel(1, bad)
    with pytest.raises(AssertionError):      # the write without its wait
        check_kernel(1, good[:2] + good[3:])
