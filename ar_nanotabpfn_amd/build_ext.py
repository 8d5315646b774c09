"""Build ``libartab_attention.so`` and ``libartab_bench.so`` for gfx950 with hipcc (cross-compiles
without a GPU).

    python -m ar_nanotabpfn_amd.build_ext

The device code is split over several translation units (the C ABI with the small kernels, the
matrix-core attention kernel, the fused layer kernels per element type and kernel group) that are
compiled side by side.  The same objects are linked twice: with a launch observer that observes
nothing into the drop-in library (exports: the ``artab_*`` functions of
``include/artab_attention.h``), and with the benchmark hooks and the instruction-mix kernel into
``libartab_bench.so`` (``include/artab_bench.h``), which only ``bench.py`` loads.
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
OUT_BENCH = os.path.join(HERE, "libartab_bench.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed-FP32 VALU forms are switched off for device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators live in VGPRs (no AGPR<->VGPR copies around every product)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # leading scalar kernel arguments (up to 8 of them) arrive in SGPRs, placed there by the command
    # processor, instead of being loaded from the argument segment by the kernel's first
    # instructions; kernels whose first argument is a struct are unaffected
    "-mllvm", "-amdgpu-kernarg-preload-count=8",
    # only the extern "C" entry points leave the library (see EXPORTS below)
    "-fvisibility=hidden",
]

# linker version script: the C ABI is every artab_* symbol, nothing else is exported
EXPORTS = "{ global: artab_*; local: *; };\n"

# (source, extra defines, object name)
UNITS = [("artab_api.hip", [], "artab_api.o"), ("flash_launch.hip", [], "flash_launch.o"),
         ("backward_launch.hip", [], "backward_launch.o")]
# objects that differ between the two libraries
PRODUCT_ONLY = [("launch_observer_none.hip", [], "launch_observer_none.o")]
BENCH_ONLY = [("bench_hooks.hip", [], "bench_hooks.o"), ("mix_bench.hip", [], "mix_bench.o")]
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
    """Compile every translation unit from source (every time it is called) and link the two
    libraries; returns the path of the drop-in library."""
    hipcc = find_hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    units = UNITS + PRODUCT_ONLY + BENCH_ONLY
    jobs = jobs or min(len(units), max(1, (os.cpu_count() or 2)), 8)

    def obj(u):
        return os.path.join(OBJ_DIR, u[2])

    cmds = [[hipcc, *HIPCC_FLAGS, *defs, "-c", os.path.join(CSRC, src), "-o", os.path.join(OBJ_DIR, o)]
            for src, defs, o in units]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    exports = os.path.join(OBJ_DIR, "exports.map")
    with open(exports, "w") as f:
        f.write(EXPORTS)
    for out, extra in ((OUT, PRODUCT_ONLY), (OUT_BENCH, BENCH_ONLY)):
        objs = [obj(u) for u in UNITS + extra]
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", f"-Wl,--version-script={exports}",
              "-o", out + ".tmp", *objs], verbose)
        os.replace(out + ".tmp", out)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
