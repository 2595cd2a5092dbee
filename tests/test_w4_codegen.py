"""The 4-wavefront kernel keeps its accumulators in the accumulation registers a0..a255, which it names only
inside inline assembly: the compiler is told they are taken, but nothing stops it from parking other values
there when it runs short of ordinary registers (it did once, in the fused-LayerNorm form, and the accumulators
came out overwritten).  This test compiles the kernels to assembly and checks that the compiler itself never
writes an accumulation register and never spills."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "general-nvgpu-testing_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


import pytest


# fp16 and bf16: plain, streaming stores, fused LayerNorm; B as [K][N]: plain, streaming stores
@pytest.mark.parametrize("source,count", [("gemm_inst_w4.hip", 6), ("gemm_inst_w4_kmajor.hip", 4)])
def test_compiler_never_touches_the_accumulators(tmp_path, source, count):
    out = tmp_path / "w4.s"
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Wno-unused-command-line-argument",
                    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only",
                    "-o", str(out), os.path.join(CSRC, source)], check=True, capture_output=True, timeout=600)
    text = out.read_text()
    kernels = re.findall(r"^(_ZN4beam16gemmrc_w4_kernel\w+):", text, flags=re.M)
    assert len(kernels) >= count, kernels
    assert "v_mfma_f32_16x16x32" in text
    for bad in ("v_accvgpr_write", "v_accvgpr_mov", "scratch_load", "scratch_store"):
        assert bad not in text, f"the compiler emitted {bad} in a 4-wavefront kernel"
    assert set(re.findall(r"\.vgpr_spill_count:\s*(\d+)", text)) == {"0"}
    assert set(re.findall(r"\.sgpr_spill_count:\s*(\d+)", text)) == {"0"}
    assert set(re.findall(r"\.private_segment_fixed_size:\s*(\d+)", text)) == {"0"}
