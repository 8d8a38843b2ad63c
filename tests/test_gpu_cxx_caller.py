"""The reference's C++ call sites on top of the C ABI: a program that includes include/vsparse_shim.hpp,
links libvsparse.so and calls spmm::wmmaSpmm / spmm::cudaSpmm / sddmm::wmmaSddmm / sddmm::cudaSddmm with
hipMalloc'ed buffers (no Python, no torch in that process) must reproduce the host loops."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cxx", "reference_call_sites")


def test_cxx_program_through_the_shim(gpu):
    # a missing executable is a failure, not a skip: it is the only C++-caller evidence for the shim
    assert os.path.exists(EXE), "tests/cxx/reference_call_sites is not built (python -m vectorsparse_amd.build)"
    proc = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout
    assert "PASSED" in proc.stdout and "FAILED" not in proc.stdout
