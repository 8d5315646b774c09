"""Build ``libartab_attention.so`` for gfx950 with hipcc (cross-compiles without a GPU).

    python -m ar_nanotabpfn_amd.build_ext

The device code is split over several translation units (the C ABI with the small kernels, the
matrix-core attention kernel, the fused layer kernels per element type and kernel group) that are
compiled side by side and linked into one shared library.
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
OUT = os.path.join(HERE, "libartab_attention.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed-FP32 VALU forms are switched off for device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators live in VGPRs (no AGPR<->VGPR copies around every product)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]

# (source, extra defines, object name)
UNITS = [("artab_api.hip", [], "artab_api.o"), ("flash_launch.hip", [], "flash_launch.o"),
         ("mix_bench.hip", [], "mix_bench.o"), ("backward_launch.hip", [], "backward_launch.o")]
for _bf16 in (1, 0):
    for _group in (0, 1, 2, 3):
        UNITS.append(("layer_launch.hip", [f"-DARTAB_LAYER_BF16={_bf16}", f"-DARTAB_LAYER_GROUP={_group}"],
                      f"layer_launch_{'bf16' if _bf16 else 'f16'}_{_group}.o"))


def find_hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{log}")
    if verbose and log.strip():
        print(log)


def build(verbose: bool = True, jobs: int = 0) -> str:
    """Compile every translation unit from source (every time it is called) and link the
    library; returns the .so path."""
    hipcc = find_hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(len(UNITS), max(1, (os.cpu_count() or 2)), 8)
    objs = [os.path.join(OBJ_DIR, o) for _, _, o in UNITS]
    cmds = [[hipcc, *HIPCC_FLAGS, *defs, "-c", os.path.join(CSRC, src), "-o", obj]
            for (src, defs, _), obj in zip(UNITS, objs)]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT + ".tmp", *objs], verbose)
    os.replace(OUT + ".tmp", OUT)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
