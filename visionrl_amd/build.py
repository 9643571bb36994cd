"""Build the HIP libraries in-tree: ``python -m visionrl_amd.build``.

hipcc cross-compiles for gfx950 without a GPU.  Packed-FP32 instruction
selection is switched off for the device pass, as this GPU pool requires.
The sources compile side by side (one hipcc process each), then link into
``csrc/libvrl_int4.so`` (the product) and ``csrc/libvrl_bench.so`` (measurement
helpers that only ``bench.py`` loads).
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_NAME = "libvrl_int4.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)
BENCH_LIB_PATH = os.path.join(CSRC, "libvrl_bench.so")
SOURCES = ["int4_gemv.hip", "cfg_sample.hip", "decode_layer.hip", "head_sample.hip"]
BENCH_SOURCES = ["bench_kernels.hip"]

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-fPIC",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go straight to VGPRs: the dequant path converts them at once
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]
NOISE = "is not a recognized feature for this target"


def hipcc_path() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found: a ROCm toolchain is required to build visionrl_amd")
    return found


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    log = "\n".join(line for line in (proc.stdout + proc.stderr).splitlines() if NOISE not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log, flush=True)


def build(verbose: bool = True) -> str:
    hipcc = hipcc_path()
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = [s for s in SOURCES + BENCH_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    missing = [s for s in SOURCES + BENCH_SOURCES if s not in sources]
    if missing:
        raise RuntimeError(f"missing sources: {missing}")
    objs = {s: os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in sources}
    with ThreadPoolExecutor(max_workers=min(4, len(sources))) as pool:
        jobs = [pool.submit(_run, [hipcc, *HIPCC_FLAGS, "-c", "-o", objs[s], os.path.join(CSRC, s)], verbose)
                for s in sources]
        for job in jobs:
            job.result()
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", LIB_PATH, *[objs[s] for s in SOURCES]], verbose)
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", BENCH_LIB_PATH,
          *[objs[s] for s in BENCH_SOURCES]], verbose)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
