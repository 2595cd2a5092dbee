"""The 4-wavefront kernel keeps its accumulators in the accumulation registers a0..a255, which it names only
inside inline assembly: the compiler is told they are taken, but nothing stops it from parking other values
there when it runs short of ordinary registers (it did once, in the fused-LayerNorm form, and the accumulators
came out overwritten).  This test compiles the kernels to assembly and checks that the compiler itself never
writes an accumulation register and never spills a vector register.  Scalar registers parked in the lanes of a
vector register (v_writelane / v_readlane) are harmless where they happen once per output tile -- the form of the
fused LayerNorm that walks its tiles keeps two operand streams, the next tile's descriptors and the epilogue's
arguments alive at once -- but not in the steady K loop: no block that holds a whole K tile's 128 MFMAs may contain
one."""
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
    assert set(re.findall(r"\.private_segment_fixed_size:\s*(\d+)", text)) == {"0"}
    # basic blocks (label to label): the steady K loop is the one with a whole K tile's MFMAs
    steady = [b for b in re.split(r"^\.LBB\d+_\d+:", text, flags=re.M) if b.count("v_mfma_f32_16x16x32") >= 128]
    assert len(steady) >= len(kernels), (len(steady), len(kernels))
    for b in steady:
        assert "v_readlane" not in b and "v_writelane" not in b, "a scalar register is reloaded inside the steady K loop"
    # An inline-assembly statement that writes the scalar condition bit says so: between the statement that sets
    # M0 by an add and the next instruction that tests the bit, something the compiler emitted must have set it.
    lines = [l.strip() for l in text.splitlines()]
    reads = re.compile(r"^(s_cselect_|s_cbranch_scc|s_addc_|s_subb_)")
    writes = re.compile(r"^s_(cmp|cmpk|add|sub|and|or|xor|andn2|orn2|not|lshl|lshr|ashr|bfe|min|max|mul_i32\b.*scc|abs|bitcmp|addk|cmov)")
    adds = [i for i, l in enumerate(lines) if l.startswith("s_add_u32 m0")]
    assert len(adds) > 100
    for i in adds:
        for l in lines[i + 1:]:
            if l.startswith(("s_add_u32 m0", ".LBB", "s_branch", "s_endpgm")) or writes.match(l):
                break
            assert not reads.match(l), f"line {i}: `{l}` tests the condition bit an M0 add in inline assembly has overwritten"
