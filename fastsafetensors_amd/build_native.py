# SPDX-License-Identifier: Apache-2.0
"""Builds ``libfstx.so`` for gfx950 with hipcc, in-tree next to this file.

    python -m fastsafetensors_amd.build_native

hipcc cross-compiles without a GPU.  ``-packed-fp32-ops`` is switched off for
device code on purpose: the conversion kernel's float arithmetic must not be
compiled into packed FP32 instructions.
"""
import os
import shutil
import subprocess
import sys
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["fstx_kernels.hip", "fstx_device_hip.cpp", "fstx_pipeline.cpp"]
OUTPUT = os.path.join(HERE, "libfstx.so")


def hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return found


def command() -> List[str]:
    return [
        hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        # the kernels' leading scalar argument (granule_log2) arrives in a register
        "-mllvm", "-amdgpu-kernarg-preload-count=1",
        f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
        "-o", OUTPUT, *[os.path.join(CSRC, s) for s in SOURCES], "-lpthread",
    ]


def build(verbose: bool = False) -> str:
    cmd = command()
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return OUTPUT


if __name__ == "__main__":
    print(build(verbose=True))
