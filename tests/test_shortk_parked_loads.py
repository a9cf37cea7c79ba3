"""The short-K L_inf forward (csrc/inf_forward_shortk.hip) issues the loads of its input panel and the waits for
them as inline assembly, so the compiler does not know that a parked register has a load in flight.  The library's
Makefile checks the generated code with csrc/check_parked_loads.py before it links; this test runs the same check on a
fresh compile (no GPU needed) and tests the checker itself."""
import importlib.util
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "l_inf-dist-net_amd", "csrc")
SRC = os.path.join(CSRC, "inf_forward_shortk.hip")

_spec = importlib.util.spec_from_file_location("check_parked_loads", os.path.join(CSRC, "check_parked_loads.py"))
checker = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(checker)
check_kernel = checker.check_kernel


def library_flags():
    """The compiler flags of the library's Makefile (FLAGS := ... with its continuation line), ARCH filled in."""
    text = open(os.path.join(CSRC, "Makefile")).read()
    arch = re.search(r"^ARCH\s*\?=\s*(\S+)", text, re.M).group(1)
    flags = re.search(r"^FLAGS\s*:=\s*((?:.*\\\n)*.*)$", text, re.M).group(1).replace("\\\n", " ")
    return flags.replace("$(ARCH)", arch).split()


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_read_of_a_parked_register_before_its_wait(tmp_path):
    out = tmp_path / "shortk.s"
    cmd = ["hipcc"] + library_flags() + ["-S", "--cuda-device-only", SRC, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    assert checker.check_listing(out.read_text()) == list(range(1, 11))


def test_the_makefile_runs_the_check_before_it_links():
    text = open(os.path.join(CSRC, "Makefile")).read()
    assert "check_parked_loads.py" in text
    assert re.search(r"^\$\(OUT\):.*\$\(SHORTK_OK\)", text, re.M), "the library must depend on the check's stamp"

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
