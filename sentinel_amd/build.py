"""Builds libsentinel_hip_attn.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m sentinel_amd.build          # compile everything
The library is written to sentinel_amd/lib/ and is what tests, bench.py and the C++ shim load.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsentinel_hip_attn.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SOURCES = ["capi.hip", "flash_fp32.hip", "flash_mfma_fwd.hip", "flash_mfma_bwd.hip", "layout_adapter.hip", "decode_attention.hip",
           "dense_softmax.hip", "kernel_timing.hip"]
# packed-fp32 instruction selection is switched off for every device translation unit
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _compile(src):
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + os.environ.get("SENTINEL_HIPCC_EXTRA", "").split() + ["-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    return obj


def build_library(jobs=None):
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 8)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objects
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
    sys.exit(0)
