"""Host arithmetic of the persistent grids' tile assignment (sentinel_amd/csrc/mfma_tile.h), run on the CPU.

The compiled check (tests/cpp/test_grid_plan.cpp) walks tile_of_slot over many grid shapes: every tile of an XCD must go to
exactly one (round, workgroup) under both orders, and plan_persistent_grid must pick the order the measurements asked for.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "test_grid_plan")


def test_every_tile_is_assigned_once():
    if not os.path.exists(EXE):
        subprocess.run(["make", "-C", os.path.join(HERE, "cpp"), EXE], check=True, capture_output=True, timeout=300)
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "grid plan ok" in proc.stdout
