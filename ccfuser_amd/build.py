"""Build libccfuser_moe.so from the HIP sources with hipcc for gfx950.

    python -m ccfuser_amd.build          # compile every source, link the library

hipcc cross-compiles without a GPU.  Objects go to ``ccfuser_amd/csrc/_obj`` and
the library next to this file, so it travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libccfuser_moe.so"
SOURCES = ["api.hip", "gate.hip", "route.hip", "rows.hip", "bwd.hip", "ffn.hip", "probe.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
PER_FILE = {
    # the gate's fp32 accumulation order must survive the optimiser
    "gate.hip": ["-ffp-contract=off"],
    # the 16x16x32 main loop names its accumulation registers itself: nothing of the compiler's may live there
    "ffn.hip": ["-mllvm", "-amdgpu-spill-vgpr-to-agpr=0"],
    "probe.hip": ["-mllvm", "-amdgpu-spill-vgpr-to-agpr=0"],
}


def _compile(src: str) -> Path:
    obj_dir = CSRC / "_obj"
    obj_dir.mkdir(exist_ok=True)
    obj = obj_dir / (src + ".o")
    cmd = [HIPCC, *COMMON, *PER_FILE.get(src, []), "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> Path:
    """Compile every HIP source and link the shared library.  Always recompiles."""
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
           "-Wno-unused-command-line-argument", *map(str, objs), "-o", str(LIB)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes)")
    return LIB


if __name__ == "__main__":
    build()
