"""The C ABI bound by a plain C++ host program (pcf-nat_amd/csrc/abi_check.cpp): no Python and no torch between the
caller and the library.  The program compares every un-fused entry point, the fused forward and the dense forward
with index loops of its own and exits 0 when all agree."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "pcf-nat_amd", "lib", "na1d_abi_check")


@pytest.mark.gpu
def test_host_program_binds_the_c_abi_and_agrees_with_its_own_loops():
    assert os.path.exists(PROGRAM), "build it with `make -C pcf-nat_amd/csrc`"
    r = subprocess.run([PROGRAM], capture_output=True, text=True, timeout=120)
    print(r.stdout[-3000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-1000:]
    assert "all checks passed" in r.stdout and "FAILED" not in r.stdout
