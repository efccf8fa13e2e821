"""Static checks of the compiled GEMM kernels (CPU only, needs hipcc).

The 16x16x32 main loop names its accumulation registers (AGPRs) literally in
inline asm, so the compiler must never place a value of its own there.  It
does so only under register pressure (a copy `v_accvgpr_write_b32 aN, vM` and
back); this test compiles ffn.hip to assembly and fails if any such copy
appears in the kernels that use that main loop, or if they spill to scratch.
"""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                    reason="hipcc not available")
def test_no_compiler_values_in_accumulation_registers(tmp_path):
    from ccfuser_amd import build as B
    out = tmp_path / "ffn.s"
    cmd = [B.HIPCC, *B.COMMON, *B.PER_FILE.get("ffn.hip", []), "-S", "--cuda-device-only",
           str(B.CSRC / "ffn.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    text = out.read_text()
    # kernels built on Ring16Mainloop: SCHED = 4 in the GemmCfg mangling, plain and persistent
    kernels = re.findall(r"^(_ZN3ccf\S*grouped_gemm\S*GemmCfgILi256ELi256ELi64ELi2ELi2ELi2ELi1ELi8ELi4EEE\S*):[^\n]*\n(.*?)s_endpgm",
                         text, flags=re.S | re.M)
    assert len(kernels) >= 4, [k for k, _ in kernels]
    for name, body in kernels:
        # the hand-written asm uses the bracket form a[N]; the compiler prints aN
        stray = re.findall(r"^\s*(v_accvgpr_(?:write_b32 a\d+, v\d+|read_b32 v\d+, a\d+|mov_b32 .*))$", body, flags=re.M)
        assert not stray, (name, stray[:5])
        assert "scratch_" not in body, name
        assert body.count("v_mfma_f32_16x16x32_f16") >= 128, name


@pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                    reason="hipcc not available")
def test_probe_kernel_keeps_the_accumulation_registers_to_itself(tmp_path):
    """The MFMA-only probe names all 256 accumulation registers in inline asm too: the compiler
    must hold nothing of its own there (a value parked in one would be overwritten: it was the
    index of the kernel's only store once), and must not spill."""
    from ccfuser_amd import build as B
    out = tmp_path / "probe.s"
    cmd = [B.HIPCC, *B.COMMON, *B.PER_FILE.get("probe.hip", []), "-S", "--cuda-device-only",
           str(B.CSRC / "probe.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    text = out.read_text()
    m = re.search(r"^(_ZN3ccf\S*mfma_probe_kernel\S*):[^\n]*\n(.*?)s_endpgm", text, flags=re.S | re.M)
    assert m
    body = m.group(2)
    stray = re.findall(r"^\s*(v_accvgpr_(?:write_b32 a\d+, v\d+|read_b32 v\d+, a\d+|mov_b32 .*))$", body, flags=re.M)
    assert not stray, stray[:5]
    assert "scratch_" not in body
    assert body.count("v_mfma_f32_16x16x32_f16") == 64
