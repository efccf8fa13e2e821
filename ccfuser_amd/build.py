"""Build libccfuser_moe.so (the product) and libccfuser_probe.so (measurement probes) from the
HIP sources with hipcc for gfx950.

    python -m ccfuser_amd.build          # compile every source, check, link both libraries

hipcc cross-compiles without a GPU.  Objects go to ``ccfuser_amd/csrc/_obj`` and the
libraries next to this file, so they travel with the source tree.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libccfuser_moe.so"
PROBE_LIB = HERE / "libccfuser_probe.so"
SOURCES = ["api.hip", "gate.hip", "route.hip", "rows.hip", "bwd.hip", "ffn.hip"]
PROBE_SOURCES = ["probe.hip"]

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
# Sources whose kernels name accumulation registers (AGPRs) literally in inline asm, and the
# kernels (regex on the mangled name) that do.  If the compiler parks a value of its own in
# such a register, or spills, the asm overwrites it; both times that happened the value was an
# address and the kernel faulted the GPU.  So these are compiled to assembly and scanned, and a
# library that fails the scan is never linked.
ACC_CHECKED = {
    "ffn.hip": r"_ZN3ccf\S*grouped_gemm\S*",
    "probe.hip": r"_ZN3ccf\S*mfma_probe_kernel\S*",
}
_NOISE = "is not a recognized feature for this target"


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if _NOISE not in l)
    return res.returncode, err


def _compile(src: str) -> Path:
    obj_dir = CSRC / "_obj"
    obj_dir.mkdir(exist_ok=True)
    obj = obj_dir / (src + ".o")
    rc, err = _run([HIPCC, *COMMON, *PER_FILE.get(src, []), "-c", str(CSRC / src), "-o", str(obj)])
    if rc != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def kernel_bodies(asm_text: str, name_regex: str):
    """(name, assembly text) of every kernel whose mangled name matches: from its label to the
    end-of-function label, so code behind an early s_endpgm is part of the body."""
    out = []
    for m in re.finditer(r"^(" + name_regex + r"):[^\n]*\n", asm_text, flags=re.M):
        end = asm_text.find(".Lfunc_end", m.end())
        out.append((m.group(1), asm_text[m.end(): end if end >= 0 else len(asm_text)]))
    return out


def acc_register_violations(asm_text: str, name_regex: str):
    """Accumulation-register moves of the compiler's own, and scratch accesses, in the kernels
    that name those registers themselves.  The hand-written asm uses the bracket form a[N]; the
    compiler prints aN."""
    bad = []
    for name, body in kernel_bodies(asm_text, name_regex):
        stray = re.findall(r"^\s*(v_accvgpr_(?:write_b32 a\d+, v\d+|read_b32 v\d+, a\d+|mov_b32 .*))$", body, flags=re.M)
        if stray:
            bad.append((name, stray[:5]))
        if "scratch_" in body:
            bad.append((name, ["scratch access"]))
    return bad


def device_assembly(src: str, out: Path) -> str:
    rc, err = _run([HIPCC, *COMMON, *PER_FILE.get(src, []), "-S", "--cuda-device-only", str(CSRC / src), "-o", str(out)])
    if rc != 0:
        raise RuntimeError(f"hipcc -S failed on {src}:\n{err}")
    return out.read_text()


def _check(src: str) -> None:
    obj_dir = CSRC / "_obj"
    obj_dir.mkdir(exist_ok=True)
    text = device_assembly(src, obj_dir / (src + ".s"))
    bad = acc_register_violations(text, ACC_CHECKED[src])
    if bad:
        raise RuntimeError(f"{src}: the compiler uses accumulation registers that the kernels name themselves, "
                           f"or spills; such a binary faults the GPU and is not linked: {bad[:3]}")


def _link(objs, lib: Path) -> None:
    rc, err = _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
                    "-Wno-unused-command-line-argument", *map(str, objs), "-o", str(lib)])
    if rc != 0:
        raise RuntimeError(f"link failed:\n{err}")


def build(verbose: bool = True) -> Path:
    """Compile every HIP source, scan the kernels that own their accumulation registers, and
    link both shared libraries.  Always recompiles."""
    srcs = SOURCES + PROBE_SOURCES
    with ThreadPoolExecutor(max_workers=8) as pool:
        checks = [pool.submit(_check, s) for s in ACC_CHECKED]
        objs = dict(zip(srcs, pool.map(_compile, srcs)))
        for c in checks:
            c.result()
    _link([objs[s] for s in SOURCES], LIB)
    _link([objs[s] for s in PROBE_SOURCES], PROBE_LIB)
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes), {PROBE_LIB} ({PROBE_LIB.stat().st_size} bytes)")
    return LIB


if __name__ == "__main__":
    build()
