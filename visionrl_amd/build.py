"""Build the HIP library in-tree: ``python -m visionrl_amd.build``.

hipcc cross-compiles for gfx950 without a GPU.  Packed-FP32 instruction
selection is switched off for the device pass, as this GPU pool requires.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libvrl_int4.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)
SOURCES = ["int4_gemv.hip", "cfg_sample.hip", "decode_layer.hip"]

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go straight to VGPRs: the dequant path converts them at once
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def hipcc_path() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found: a ROCm toolchain is required to build visionrl_amd")
    return found


def build(verbose: bool = True) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIB_PATH, *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(line for line in (proc.stdout + proc.stderr).splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log, flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
