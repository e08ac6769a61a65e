"""Runs the C++ scenario program (tests/cpp/hip_executor_scenarios.cpp): the reference's
test_paged_flash scenarios through the C++ HipExecutor class."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "hip_executor_scenarios")


@pytest.mark.gpu
def test_cpp_scenarios(exe):
    assert os.path.exists(EXE), "build it with __graft_entry__.build()"
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.count(" ok") == 9
