"""ctypes front end of the CPU oracle (oracle/beam_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
module; the shipped `beam` package never does.

16-bit tensors travel as numpy uint16 arrays holding the raw bit patterns (fp16 or bf16),
fp32 results as numpy float32 arrays.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

F16 = 0
BF16 = 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbeam_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/beam_oracle.c with gcc (plain make)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        f32p = ctypes.POINTER(ctypes.c_float)
        f64p = ctypes.POINTER(ctypes.c_double)
        i = ctypes.c_int
        L.oracle_gemmrc.argtypes = [u16p, u16p, i, i, i, i, f32p, u16p]
        L.oracle_gemmrc.restype = i
        L.oracle_gemmrc_naive_f64.argtypes = [u16p, u16p, i, i, i, i, f64p]
        L.oracle_gemmrc_naive_f64.restype = None
        L.oracle_gemmrc_splitk.argtypes = [u16p, u16p, i, i, i, i, i, i, f32p, u16p]
        L.oracle_gemmrc_splitk.restype = i
        L.oracle_gemmrc_ln.argtypes = [u16p, u16p, u16p, u16p, ctypes.c_float, i, i, i, i, f32p, u16p]
        L.oracle_gemmrc_ln.restype = i
        L.oracle_compare.argtypes = [u16p, f32p, ctypes.c_size_t, i, f64p, f64p, f64p, f64p]
        L.oracle_compare.restype = None
        L.oracle_to_f32.argtypes = [u16p, f32p, ctypes.c_size_t, i]
        L.oracle_from_f32.argtypes = [f32p, u16p, ctypes.c_size_t, i]
        L.oracle_slice_heuristic.argtypes = [i, ctypes.c_float]
        L.oracle_slice_heuristic.restype = i
        L.oracle_split_k_len.argtypes = [i, i, i]
        L.oracle_split_k_len.restype = i
        L.oracle_tflops.argtypes = [ctypes.c_double] * 4
        L.oracle_tflops.restype = ctypes.c_double
        L.oracle_num_threads.restype = i
        L.oracle_silu.argtypes = [u16p, u16p, f32p, ctypes.c_size_t, i]
        L.oracle_silu.restype = None
        _lib = L
    return _lib


def _u16(a: np.ndarray):
    assert a.dtype == np.uint16 and a.flags.c_contiguous
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16))


def _f32(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def to_f32(bits: np.ndarray, dtype: int) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().oracle_to_f32(_u16(bits), _f32(out), bits.size, dtype)
    return out


def from_f32(x: np.ndarray, dtype: int) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_from_f32(_f32(x), _u16(out), x.size, dtype)
    return out


def gemmrc(a_bits: np.ndarray, b_bits: np.ndarray, dtype: int = F16, want16: bool = False):
    """fp32-accumulate C = A . B^T.  Returns the fp32 result (and its 16-bit rounding)."""
    M, K = a_bits.shape
    N, K2 = b_bits.shape
    assert K == K2
    c32 = np.empty((M, N), dtype=np.float32)
    c16 = np.empty((M, N), dtype=np.uint16) if want16 else None
    rc = lib().oracle_gemmrc(_u16(a_bits), _u16(b_bits), M, N, K, dtype, _f32(c32),
                             _u16(c16) if want16 else None)
    if rc != 0:
        raise MemoryError("oracle_gemmrc failed")
    return (c32, c16) if want16 else c32


def gemmrc_naive_f64(a_bits: np.ndarray, b_bits: np.ndarray, dtype: int = F16) -> np.ndarray:
    M, K = a_bits.shape
    N, _ = b_bits.shape
    out = np.empty((M, N), dtype=np.float64)
    lib().oracle_gemmrc_naive_f64(_u16(a_bits), _u16(b_bits), M, N, K, dtype,
                                  out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)))
    return out


def gemmrc_splitk(a_bits, b_bits, splits: int, dtype: int = F16, ktile: int = 64) -> np.ndarray:
    M, K = a_bits.shape
    N, _ = b_bits.shape
    c32 = np.empty((M, N), dtype=np.float32)
    rc = lib().oracle_gemmrc_splitk(_u16(a_bits), _u16(b_bits), M, N, K, dtype, splits, ktile,
                                    _f32(c32), None)
    if rc != 0:
        raise RuntimeError(f"oracle_gemmrc_splitk failed ({rc})")
    return c32


def gemmrc_ln(a_bits, b_bits, gamma_bits, beta_bits, eps: float = 1e-5, dtype: int = F16) -> np.ndarray:
    M, K = a_bits.shape
    N, _ = b_bits.shape
    y32 = np.empty((M, N), dtype=np.float32)
    rc = lib().oracle_gemmrc_ln(_u16(a_bits), _u16(b_bits), _u16(gamma_bits), _u16(beta_bits),
                                eps, M, N, K, dtype, _f32(y32), None)
    if rc != 0:
        raise MemoryError("oracle_gemmrc_ln failed")
    return y32


def matmul_nn(a_bits: np.ndarray, b_kn_bits: np.ndarray, dtype: int = F16) -> np.ndarray:
    """fp32 C = A . B for B stored [K][N]: the same sum as gemmrc on the transposed copy of B
    (layout of python/beam/triton_kernels/gemm.py:78-99)."""
    return gemmrc(a_bits, np.ascontiguousarray(np.asarray(b_kn_bits).T), dtype)


def silu(x_bits: np.ndarray, dtype: int = F16):
    """(fp32 values, RN 16-bit bit patterns) of x / (1 + exp(-x)) on a flat 16-bit array."""
    x = np.ascontiguousarray(x_bits, dtype=np.uint16).ravel()
    y32 = np.empty(x.size, dtype=np.float32)
    y16 = np.empty(x.size, dtype=np.uint16)
    lib().oracle_silu(_u16(x), _u16(y16), _f32(y32), x.size, dtype)
    return y32.reshape(x_bits.shape), y16.reshape(x_bits.shape)


def compare(got_bits: np.ndarray, ref32: np.ndarray, dtype: int = F16) -> dict:
    """max |got-ref|, RMS(ref), max |ref| and the error in excess of bf16's half-ulp."""
    got_bits = np.ascontiguousarray(got_bits, dtype=np.uint16)
    ref32 = np.ascontiguousarray(ref32, dtype=np.float32)
    assert got_bits.size == ref32.size
    vals = [ctypes.c_double() for _ in range(4)]
    lib().oracle_compare(_u16(got_bits), _f32(ref32), got_bits.size, dtype,
                         *[ctypes.byref(v) for v in vals])
    return {"max_abs_err": vals[0].value, "rms_ref": vals[1].value, "max_abs_ref": vals[2].value,
            "max_bf16_excess": vals[3].value}


def gemm_tolerance(K: int) -> float:
    """Bound on max|err| / RMS(ref) for a gemmrc with reduction length K."""
    return 1e-2 * (K / 1024.0) ** 0.5


LN_ABS_TOL = 2e-3


def slice_heuristic(tiles: int, units: float) -> int:
    return lib().oracle_slice_heuristic(tiles, units)


def split_k_len(K: int, splits: int, ktile: int = 64) -> int:
    return lib().oracle_split_k_len(K, splits, ktile)


def tflops(m, n, k, ms) -> float:
    return lib().oracle_tflops(float(m), float(n), float(k), float(ms))


def num_threads() -> int:
    return lib().oracle_num_threads()
