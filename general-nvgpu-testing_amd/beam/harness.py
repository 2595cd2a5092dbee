"""Correctness / performance harness for the gemmrc operators.

Counterpart of the reference's only test driver, python/gemm_test.py:
  check            :29-70    dtype + shape equality, then a tolerance check per output
  run_perf         :73-75    latency of one candidate
  universal_test   :78-107   inputs -> answer -> for each candidate: clear, time, check
  test_gemm        :160-192  the tiled kernels at one shape
  test_gemm_splitk :110-157  split_k_slices = 1..15 sweep (here: a CSV instead of splitk.pdf)
  test_tuner       :203-217  OperatorTuner on three shapes
  print_device_info:221-232  device banner

Differences, on purpose: inputs are seeded (the library's counter-based generator), a failed check
raises instead of printing in colour and carrying on, and the bound is the RMS-relative one used
everywhere in this repository (max|err| <= 1e-2*sqrt(K/1024)*RMS, with the |ref|/256 allowance for
bf16) instead of rtol=atol=2e-2.  The answer function is any callable f(a, b, c) writing c: by
default the library's own default-tile kernel (a self-consistency check); the test-suite passes
a CPU reference instead.
"""
from __future__ import annotations

import csv
import time
from functools import partial
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np

from . import _C
from .tuner import OperatorTuner

STR_DTYPE_MAPPING = {"fp16": _C.F16, "bf16": _C.BF16}


def _to_f32(bits: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == _C.BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


class CheckFailed(AssertionError):
    pass


def check(func, answers: Sequence[np.ndarray], outputs: Sequence[_C.DeviceArray], K: int) -> Dict[str, float]:
    """answers: fp32 host arrays; outputs: device arrays just written by `func`."""
    name = getattr(func, "__name__", None) or str(func)
    if len(outputs) != len(answers):
        raise CheckFailed(f"{name}: {len(outputs)} outputs, {len(answers)} answers")
    worst = 0.0
    for i, (ans, out) in enumerate(zip(answers, outputs)):
        if tuple(out.shape) != tuple(ans.shape):
            raise CheckFailed(f"{name} tensor({i}): shape {out.shape} != {ans.shape}")
        got = _to_f32(out.to_numpy(), out.dtype)
        err = np.abs(got - ans)
        if out.dtype == _C.BF16:
            err = err - np.abs(ans) / 256.0
        rms = float(np.sqrt(np.mean(ans.astype(np.float64) ** 2)))
        bound = 1e-2 * (K / 1024.0) ** 0.5 * max(rms, 1e-30)
        e = float(err.max())
        worst = max(worst, e / max(rms, 1e-30))
        if not np.isfinite(got).all() or e > bound:
            raise CheckFailed(f"{name} tensor({i}): max error {e:.4g} exceeds {bound:.4g} (RMS {rms:.4g})")
    return {"max_err_over_rms": worst}


def run_perf(func, inputs, outputs, warmup: int = 10, rep: int = 30) -> float:
    """Seconds per call."""
    time.sleep(0.05)
    return _C.do_bench(lambda: func(*(list(inputs) + list(outputs))), warmup=warmup, rep=rep) * 1e-3


def universal_test(ansfunc, funcs: List[Callable], input_shapes, output_shapes, dtype: int, metric, K: int,
                   seed: int = 0, verbose: bool = True) -> Dict:
    inputs = [_C.DeviceArray.from_numpy(_C.host_normal(s, dtype, seed, i, 0.0, K ** -0.5), dtype)
              for i, s in enumerate(input_shapes)]
    outputs = [_C.DeviceArray(s, dtype) for s in output_shapes]
    answers_dev = [_C.DeviceArray(s, dtype) for s in output_shapes]
    for d in answers_dev:
        d.fill_bytes(0)
    ansfunc(*(inputs + answers_dev))
    answers = [_to_f32(d.to_numpy(), dtype) for d in answers_dev]
    ret = {"custom": [], "names": [], "max_err_over_rms": []}
    for func in funcs:
        for d in outputs:
            d.fill_bytes(0)
        latency = run_perf(func, inputs, outputs)
        name = getattr(func, "__name__", None) or str(func)
        res = check(func, answers, outputs, K)
        if verbose:
            print(f"{name}: {latency * 1e3:.6f} ms, [{metric(latency=latency):.3f}] TFLOPS, "
                  f"max err {res['max_err_over_rms']:.2e} x RMS: success")
        ret["custom"].append(metric(latency=latency))
        ret["names"].append(name)
        ret["max_err_over_rms"].append(res["max_err_over_rms"])
    for d in inputs + outputs + answers_dev:
        d.free()
    return ret


def compute_flops(m, n, k, latency):
    return 2 * m * n * k / latency * 1e-12


def test_gemm(m: int, n: int, k: int, dtype: str = "fp16", ansfunc: Optional[Callable] = None, verbose=True):
    d = STR_DTYPE_MAPPING[dtype]
    if verbose:
        print(f"[TEST] GEMM: {(m, n, k)=}, {dtype=}")
    funcs = [_C.gemmrc,
             partial(_C.gemmrc_spec, shape_threadblock=[128, 256], shape_warp=[64, 64]),
             partial(_C.gemmrc_spec, shape_threadblock=[128, 128], shape_warp=[64, 64]),
             partial(_C.gemmrc_spec, shape_threadblock=[256, 128], shape_warp=[64, 64])]
    if d == _C.F16:
        funcs += [_C.custom_gemmrc_128x256, _C.custom_gemmrc_128x128]
    return universal_test(ansfunc or _C.gemmrc, funcs, [(m, k), (n, k)], [(m, n)], d,
                          partial(compute_flops, m, n, k), k, verbose=verbose)


def test_gemm_splitk(m: int, n: int, k: int, dtype: str = "fp16", csv_path: Optional[str] = None,
                     ansfunc: Optional[Callable] = None, verbose=True):
    d = STR_DTYPE_MAPPING[dtype]
    if verbose:
        print(f"[TEST] GEMM SPLITK: {m=}, {n=}, {k=}, {dtype=}")
    funcs = []
    for s in range(1, 16):
        f = partial(_C.gemmrc_splitk_spec, shape_threadblock=[128, 64], shape_warp=[64, 32], split_k_slices=s)
        f.__name__ = f"gemmrc_splitk_spec[128x64,s{s}]"  # type: ignore[attr-defined]
        funcs.append(f)
    rets = universal_test(ansfunc or _C.gemmrc, funcs, [(m, k), (n, k)], [(m, n)], d,
                          partial(compute_flops, m, n, k), k, verbose=verbose)
    if csv_path:
        with open(csv_path, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(["split_k_slices", "TFLOPS", "max_err_over_rms"])
            for s, (t, e) in enumerate(zip(rets["custom"], rets["max_err_over_rms"]), start=1):
                w.writerow([s, f"{t:.4f}", f"{e:.3e}"])
    return rets


def test_tuner(shapes=((2048, 2048, 4096), (4096, 4096, 4096), (8192, 8192, 4096)), cache_path=None, verbose=True):
    tuner = OperatorTuner(cache_path=cache_path)
    out = {}
    for shape in shapes:
        op, tflops = tuner.tune(shape)
        out[tuple(shape)] = (str(op), tflops)
        if verbose:
            print(shape, str(op), tflops)
    return out


def print_device_info() -> dict:
    info = _C.device_info()
    print("-" * 14 + " Device Info " + "-" * 13)
    print(f"name:   {info['name']}")
    print(f"CUs:    {info['compute_units']}  peak clock {info['clock_khz'] / 1e3:.0f} MHz")
    print(f"memory: {info['memory_bytes'] / 2 ** 30:.1f} GiB")
    if "gfx950" not in info["name"]:
        print("  [WARNING]: device is not an MI355X-class (gfx950) part")
    print("-" * 40)
    return info


def main():
    print_device_info()
    test_gemm(4096, 4096, 4096, "fp16")
    test_gemm_splitk(512, 512, 8192, "fp16")


if __name__ == "__main__":
    main()
