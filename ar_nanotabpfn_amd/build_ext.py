"""Build ``libartab_attention.so`` for gfx950 with hipcc (cross-compiles without a GPU).

    python -m ar_nanotabpfn_amd.build_ext
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "artab_api.hip")
OUT = os.path.join(HERE, "libartab_attention.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    # packed-FP32 VALU forms are switched off for device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators live in VGPRs (no AGPR<->VGPR copies around every product)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def find_hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def build(verbose: bool = True) -> str:
    """Compile the library from source every time it is called; returns the .so path."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-o", OUT + ".tmp", SRC]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    os.replace(OUT + ".tmp", OUT)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
