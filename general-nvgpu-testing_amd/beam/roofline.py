"""Roofline arithmetic for tiled GEMMs, with an MI355X row.

Counterpart of the reference's python/scripts/gemm_flops.py:1-90 (GPUSpec :4-13, spec list
:26-32, print_gemm_bound :37-76): the time a GEMM needs at the matrix-unit peak, the time its
tiles need at the memory bandwidth when every tile fetches its operands once, and their ratio.
Differences: a function that returns the numbers (the reference only prints), bytes counted with
one write of C per tile by default (the reference counts C twice, for an atomicAdd epilogue this
library does not have; `c_traffic=2` reproduces its figure), and dense peaks only (the
reference halves NVIDIA's sparsity-inflated H100 numbers by hand, :30-31).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict


@dataclass(frozen=True)
class GPUSpec:
    name: str
    bw: float        # memory bandwidth, GB/s
    fp32: float      # vector fp32, TFLOP/s
    tf32: float      # matrix units, dense, TFLOP/s (TOP/s for int8); 0 = not supported
    fp16: float
    int8: float
    fp8: float = 0.0
    lds_kib: int = 0      # shared memory / LDS per compute unit
    compute_units: int = 0


BITWIDTH_MAP = {"tf32": 32, "fp16": 16, "bf16": 16, "fp8": 8, "int8": 8, "int4": 4}

GPU_SPEC_LIST = [
    # one row of the reference's list, kept so that its worked example can be reproduced as a check
    GPUSpec("A100_{PCIe,SXM}_HBM2", 1555, 19.5, 156, 312, 624, 0, 164, 108),
    # MI355X (gfx950): 256 CUs x 4 SIMDs x 1024 fp16 FLOP/clk x 2.4 GHz; HBM3E 8 TB/s; no tf32 unit
    # (the fp32 matrix rate is 157.3 TFLOP/s).
    GPUSpec("MI355X", 8000, 157.3, 0, 2516.6, 5033.2, 5033.2, 160, 256),
]

GPU_NAME_SPEC_MAP: Dict[str, GPUSpec] = {spec.name: spec for spec in GPU_SPEC_LIST}


def gemm_bound(spec: GPUSpec, dtype: str, n: int, k: int, m: int, micro_n: int, micro_k: int, micro_m: int,
               c_traffic: int = 1) -> dict:
    """Bounds in milliseconds for an n x k x m GEMM cut into micro_n x micro_k x micro_m jobs
    (argument order of the reference's print_gemm_bound)."""
    if dtype not in BITWIDTH_MAP:
        raise ValueError(f"unknown dtype {dtype!r}")
    rate = getattr(spec, "fp16" if dtype == "bf16" else dtype if dtype != "int4" else "int8")
    if dtype == "int4":
        rate *= 2
    if rate <= 0:
        raise ValueError(f"{spec.name} has no {dtype} matrix rate")
    size = BITWIDTH_MAP[dtype] / 8
    flops = 2.0 * n * k * m
    jobs = (n / micro_n) * (k / micro_k) * (m / micro_m)
    job_bytes = (micro_n * micro_k + micro_k * micro_m + micro_n * micro_m * c_traffic) * size
    compute_ms = flops / (rate * 1e12) * 1e3
    memory_ms = jobs * job_bytes / (spec.bw * 1e9) * 1e3
    return {"gpu": spec.name, "dtype": dtype, "flops": flops, "jobs": jobs, "bytes": jobs * job_bytes,
            "compute_ms": compute_ms, "memory_ms": memory_ms, "ratio": compute_ms / memory_ms,
            "intensity": flops / (jobs * job_bytes), "ridge": rate * 1e12 / (spec.bw * 1e9)}


def print_gemm_bound(spec: GPUSpec, dtype: str, n: int, k: int, m: int, micro_n: int, micro_k: int, micro_m: int,
                     c_traffic: int = 2) -> dict:
    """The reference's report (its C-counted-twice convention by default)."""
    r = gemm_bound(spec, dtype, n, k, m, micro_n, micro_k, micro_m, c_traffic)
    print(spec.name)
    print(f"\t{dtype} n={n} k={k} m={m}")
    print(f"\tmicro_n={micro_n} micro_k={micro_k} micro_m={micro_m}")
    print(f"\tparallel degree={r['jobs']}")
    print(f"\tCompute bound: {r['compute_ms']:.2f} ms")
    print(f"\tMemory bound: {r['memory_ms']:.2f} ms")
    print(f"\tCompute to Memory ratio: {r['ratio']:.2f}")
    return r


if __name__ == "__main__":
    print_gemm_bound(GPU_NAME_SPEC_MAP["MI355X"], "fp16", 8192, 8192, 8192, 256, 8192, 256)
    print_gemm_bound(GPU_NAME_SPEC_MAP["MI355X"], "fp16", 256, 32768, 256, 64, 2048, 64)
