"""Host arithmetic of the persistent grids' tile assignment (sentinel_amd/csrc/grid_plan.h), run on the CPU.

The compiled check (tests/cpp/test_grid_plan.cpp) walks tile_of_slot over many grid shapes: every tile of an XCD must go to
exactly one (round, workgroup) under both orders, and plan_persistent_grid must pick the order the measurements asked for.
"""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "test_grid_plan")


def test_every_tile_is_assigned_once():
    if not os.path.exists(EXE):  # plain C++ (g++): no HIP compiler needed
        if shutil.which("make") is None or shutil.which(os.environ.get("CXX", "g++")) is None:
            pytest.skip("tests/cpp/test_grid_plan is not built and there is no make / C++ compiler to build it")
        subprocess.run(["make", "-C", os.path.join(HERE, "cpp"), EXE], check=True, capture_output=True, timeout=300)
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "grid plan ok" in proc.stdout
