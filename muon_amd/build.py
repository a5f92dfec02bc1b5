"""Builds muon_amd/libmuon_amd.so from muon_amd/csrc/*.hip with hipcc for gfx950.

    python -m muon_amd.build
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmuon_amd.so")
SOURCES = ["capi.hip", "elementwise.hip", "aol.hip", "ns_gemm.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # hipcc -O3 must not form packed-fp32 instructions on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = True) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = OUT + ".tmp"
    cmd = [hipcc, *FLAGS, *[os.path.join(CSRC, s) for s in SOURCES], "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libmuon_amd.so")
    os.replace(tmp, OUT)
    return OUT


if __name__ == "__main__":
    print(build())
