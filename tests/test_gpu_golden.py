"""The HIP path against the committed float64 fixtures (tests/golden), the reference-shaped
Python operators on torch tensors, and the tuner end to end."""
import glob
import os

import numpy as np
import pytest

from test_gpu_gemm import BF16, run_gemm
from test_gpu_ln import run_ln

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def bits_to_f64(bits, dtype):
    if dtype == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return bits.view(np.float16).astype(np.float64)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "gemm_*.npz"))))
def test_gemm_fixture(gpu, beamc, path):
    f = np.load(path)
    a, b, dtype, c64 = f["a"], f["b"], int(f["dtype"]), f["c64"]
    K = a.shape[1]
    rms = np.sqrt(np.mean(c64 ** 2))
    for cfg in [None] + beamc.list_configs():
        got = bits_to_f64(run_gemm(beamc, a, b, dtype, cfg), dtype)
        err = np.abs(got - c64)
        if dtype == BF16:
            err = err - np.abs(c64) / 256.0
        assert err.max() <= 1e-2 * (K / 1024.0) ** 0.5 * rms, (path, cfg)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "ln_*.npz"))))
def test_ln_fixture(gpu, beamc, path):
    f = np.load(path)
    dtype = int(f["dtype"])
    got = bits_to_f64(run_ln(beamc, f["a"], f["b"], f["gamma"], f["beta"], dtype, float(f["eps"])), dtype)
    err = np.abs(got - f["y64"])
    if dtype == BF16:
        err = err - np.abs(f["y64"]) / 256.0
    assert err.max() <= 2e-3, path


def test_reference_named_operators_on_torch_tensors(gpu):
    """Scripts written against the reference call f(a=, b=, c=) on CUDA tensors
    (python/gemm_test.py:78-107); the same calls work here, on torch's current stream.  Runs in its own
    process because torch must be imported before beam (they then share torch's HIP runtime)."""
    import subprocess
    import sys
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "torch_dropin_check.py")
    r = subprocess.run([sys.executable, "-u", script], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "torch drop-in OK" in r.stdout


def test_tuner_end_to_end(gpu, beamc, tmp_path):
    import beam
    path = str(tmp_path / "tune.json")
    tuner = beam.OperatorTuner(cache_path=path, warmup=2, rep=5)
    small = [op for op in tuner.gemm_ops if "64x64" in str(op) or str(op) in ("gemmrc", "custom_gemmrc_128x128")]
    best, tflops = tuner.tune((256, 256, 8192), ops=small)
    assert best is not None and tflops > 0
    assert "splitk" in str(best), f"split-K should win at 256x256x8192, got {best}"
    assert tuner.tune((256, 256, 8192)) == (best, tflops)
    best_bf16, t_bf16 = tuner.tune((512, 512, 512), dtype="bf16", ops=small)
    assert best_bf16 is not None and not str(best_bf16).startswith("custom_")
    assert os.path.exists(path)
