"""Static checks of the compiled GEMM kernels (CPU only, needs hipcc).

The 16x16x32 main loop names its accumulation registers (AGPRs) literally in
inline asm, so the compiler must never place a value of its own there.  It
does so only under register pressure (a copy `v_accvgpr_write_b32 aN, vM` and
back).  ccfuser_amd.build runs this scan on every build and refuses to link a
library that fails it; these tests run the same scan and also check that it
sees the kernels it is meant for.
"""
import shutil
from pathlib import Path

import pytest

needs_hipcc = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                 reason="hipcc not available")


@needs_hipcc
def test_no_compiler_values_in_accumulation_registers(tmp_path):
    from ccfuser_amd import build as B
    text = B.device_assembly("ffn.hip", tmp_path / "ffn.s")
    kernels = B.kernel_bodies(text, B.ACC_CHECKED["ffn.hip"])
    # plain, persistent, split-tail kernels, each in several epilogue forms
    assert len(kernels) >= 10, [k for k, _ in kernels]
    assert any("persistent" in k for k, _ in kernels) and any("tail" in k for k, _ in kernels)
    for name, body in kernels:
        assert body.count("v_mfma_f32_16x16x32_f16") >= 128, name
        assert "s_endpgm" in body, name
    assert B.acc_register_violations(text, B.ACC_CHECKED["ffn.hip"]) == []


@needs_hipcc
def test_probe_kernel_keeps_the_accumulation_registers_to_itself(tmp_path):
    """The MFMA-only probe names all 256 accumulation registers in inline asm too: the compiler
    must hold nothing of its own there (a value parked in one would be overwritten: it was the
    index of the kernel's only store once), and must not spill."""
    from ccfuser_amd import build as B
    text = B.device_assembly("probe.hip", tmp_path / "probe.s")
    kernels = B.kernel_bodies(text, B.ACC_CHECKED["probe.hip"])
    assert len(kernels) == 1
    assert kernels[0][1].count("v_mfma_f32_16x16x32_f16") == 64
    assert B.acc_register_violations(text, B.ACC_CHECKED["probe.hip"]) == []


def test_the_scan_flags_a_parked_value_and_code_behind_an_early_exit():
    """The scan itself, on hand-made assembly: a compiler-style accumulation-register copy is
    found also when it sits behind the kernel's first s_endpgm."""
    from ccfuser_amd import build as B
    asm = """
_ZN3ccf12_GLOBAL__N_119grouped_gemm_kernelIXX:        ; @kernel
\ts_cbranch_scc1 .LBB0_2
\ts_endpgm
.LBB0_2:
\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
\tv_accvgpr_write_b32 a17, v3
\ts_endpgm
.Lfunc_end0:
_ZN3ccf5otherE:
\tv_accvgpr_write_b32 a1, v1
.Lfunc_end1:
"""
    bad = B.acc_register_violations(asm, B.ACC_CHECKED["ffn.hip"])
    assert len(bad) == 1 and "a17" in bad[0][1][0]
    clean = asm.replace("\tv_accvgpr_write_b32 a17, v3\n", "\tv_accvgpr_write_b32 a[17], 0\n")
    assert B.acc_register_violations(clean, B.ACC_CHECKED["ffn.hip"]) == []


@needs_hipcc
def test_gate_kernels_keep_their_values_in_registers(tmp_path):
    """Both forms of the fp16 gate (wavefronts sharing K, and every wavefront alone through all of K
    with four sets of loads in flight) are built for a register budget: none of their instantiations
    may spill (the kernel metadata's private segment size is what a spill would need)."""
    import re
    from ccfuser_amd import build as B
    text = B.device_assembly("gate.hip", tmp_path / "gate.s")
    sizes = {}
    for m in re.finditer(r"\.name:\s+(\S*gate_(?:mfma|stream)_kernel\S*)(.*?)\.private_segment_fixed_size:\s+(\d+)", text, flags=re.S):
        if ".name:" in m.group(2):                      # ran into the next kernel's record
            continue
        sizes[m.group(1)] = int(m.group(3))
    forms = {"mfma": 0, "stream": 0}
    for name, size in sizes.items():
        assert size == 0, f"{name} spills {size} bytes"
        forms["stream" if "stream" in name else "mfma"] += 1
    # tile widths 16 and 32, 1/2/4 slots, three list lengths of the selection
    assert forms["mfma"] >= 15 and forms["stream"] >= 15, forms
