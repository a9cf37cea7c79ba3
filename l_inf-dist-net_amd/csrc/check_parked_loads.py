#!/usr/bin/env python3
"""Build-time check of inf_forward_shortk.hip's generated code (run by the Makefile before the library is linked).

The short-K L_inf forward issues the loads of its input panel and the waits for them as inline assembly, so the
compiler does not know that a parked register has a load in flight.  That is safe only as long as the generated code
never reads or writes such a register between the load and the wait that stands in front of the panel write; if it
did, the kernel would silently reduce stale data.  This script reads the assembly listing of the file (compiled with
the library's own flags) and checks exactly that for every instantiation of the kernel, and that none of the parked
registers was spilled.  Any change of compiler or flags re-runs it through `make`.

usage: check_parked_loads.py <listing.s>     exit status 0 when every kernel passes
"""
import re
import sys

LOAD = re.compile(r"^\s*buffer_load_dwordx4 v\[(\d+):(\d+)\], v(\d+), ")
WRITE = re.compile(r"^\s*ds_write_b128 v(\d+), v\[(\d+):(\d+)\]")
WAIT = re.compile(r"^\s*s_waitcnt vmcnt\((\d+)\)\s*$")


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



def check_listing(asm):
    """Raises AssertionError when a kernel of the listing violates the rule; returns the instantiations checked."""
    found = kernels(asm)
    assert sorted(found) == list(range(1, 11)), sorted(found)
    for nw, lines in found.items():
        check_kernel(nw, lines)
    # the window loop is unrolled over the parked registers: none of them may have gone to scratch memory
    spills = re.findall(r"\.vgpr_spill_count:\s*(\d+)", asm)
    assert len(spills) == 10 and all(int(n) == 0 for n in spills), spills
    return sorted(found)


if __name__ == "__main__":
    try:
        done = check_listing(open(sys.argv[1]).read())
    except AssertionError as e:
        sys.exit(f"check_parked_loads: {sys.argv[1]}: a parked register is touched while its load is in flight: {e}")
    print(f"check_parked_loads: {len(done)} instantiations of inf_forward_shortk_kernel pass")
