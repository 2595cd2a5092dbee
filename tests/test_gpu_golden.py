"""The HIP path against the committed float64 fixtures (tests/golden), the reference-shaped
Python operators on torch tensors, and the tuner end to end."""
import glob
import os

import numpy as np
import pytest

from test_gpu_gemm import F16, BF16, run_gemm
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


def test_reference_named_operators_on_torch_tensors(gpu, beamc, oracle):
    """Scripts written against the reference call f(a=, b=, c=) on CUDA tensors
    (python/gemm_test.py:78-107); the same calls work here, on torch's current stream."""
    import torch
    import beam
    M, N, K = 512, 640, 1024
    a_bits = beamc.host_uniform((M, K), F16, 31, 0)
    b_bits = beamc.host_uniform((N, K), F16, 31, 1)
    ref = oracle.gemmrc(a_bits, b_bits, F16)
    a = torch.from_numpy(a_bits.view(np.float16)).cuda()
    b = torch.from_numpy(b_bits.view(np.float16)).cuda()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for fn, kw in [(beam.custom_gemmrc_128x128, {}), (beam.custom_gemmrc_128x256, {}),
                       (beam.cutlass_gemmrc, {}),
                       (beam.cutlass_gemmrc_spec, dict(shape_threadblock=[256, 128], shape_warp=[128, 32])),
                       (beam.cutlass_gemmrc_splitk, dict(split_k_slices=3)),
                       (beam.cutlass_gemmrc_splitk_spec, dict(shape_threadblock=[128, 64], shape_warp=[64, 32],
                                                              split_k_slices=5))]:
            c = torch.zeros(M, N, dtype=torch.float16, device="cuda")
            fn(a=a, b=b, c=c, **kw)
            stream.synchronize()
            r = oracle.compare(c.cpu().numpy().view(np.uint16), ref, F16)
            assert r["max_abs_err"] <= oracle.gemm_tolerance(K) * r["rms_ref"], fn.__name__
    # unsupported inputs raise instead of returning silently
    with pytest.raises(beam.BeamError):
        beam.cutlass_gemmrc(a=a.float(), b=b.float(), c=torch.zeros(M, N, device="cuda"))
    with pytest.raises(beam.BeamError):
        beam.cutlass_gemmrc(a=a.cpu(), b=b, c=torch.zeros(M, N, dtype=torch.float16, device="cuda"))
    with pytest.raises(beam.BeamError):
        beam.cutlass_gemmrc_spec(a=a, b=b, c=torch.zeros(M, N, dtype=torch.float16, device="cuda"),
                                 shape_threadblock=[48, 48])


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
