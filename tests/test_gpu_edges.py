"""Problems outside what the tiled kernels take -- K not a multiple of 8, the [K][N] layout with N not a
multiple of 8, operands at addresses that are not 16-byte aligned -- are computed (by a plain kernel), never
refused: every entry point against the oracle, to the same tolerances as everywhere else.  The reference's
NN path masks any edge (python/beam/triton_kernels/gemm.py:62-63,75)."""

import pytest

from test_gpu_gemm import F16, BF16, assert_close
from test_gpu_ln import make_ln_inputs, check_ln

pytestmark = pytest.mark.gpu

EDGE_SHAPES = [(3, 5, 7), (130, 70, 50), (257, 129, 1001), (64, 64, 12), (1, 1, 1)]


def close_enough(oracle, got_bits, ref32, K, dtype, what):
    """The GEMM bound 1e-2 * sqrt(K / 1024) * RMS; below K = 64 that bound is smaller than the rounding of a
    16-bit output itself (half an ulp: |c| * 2^-11 in fp16), which is then allowed on top, explicitly."""
    if K >= 64 or dtype != F16:
        return assert_close(oracle, got_bits, ref32, K, dtype, what)
    r = oracle.compare(got_bits, ref32, dtype)
    tol = oracle.gemm_tolerance(K) * r["rms_ref"] + r["max_abs_ref"] * 2.0 ** -11
    assert r["max_abs_err"] <= tol, f"{what}: max err {r['max_abs_err']:.4g} > {tol:.4g}"


@pytest.mark.parametrize("shape", EDGE_SHAPES)
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemmrc_any_k(gpu, beamc, oracle, shape, dtype):
    M, N, K = shape
    a = beamc.host_uniform((M, K), dtype, 61, 0)
    b = beamc.host_uniform((N, K), dtype, 61, 1)
    ref = oracle.gemmrc(a, b, dtype)
    da, db = beamc.DeviceArray.from_numpy(a, dtype), beamc.DeviceArray.from_numpy(b, dtype)
    c = beamc.DeviceArray((M, N), dtype)
    for what, call in (("gemmrc", lambda: beamc.gemmrc(da, db, c)),
                       ("gemmrc_spec", lambda: beamc.gemmrc_spec(da, db, c, shape_threadblock=[128, 128], shape_warp=[64, 64])),
                       ("split-K", lambda: beamc.gemmrc_splitk(da, db, c, split_k_slices=4)),
                       ("split-K, library's choice", lambda: beamc.gemmrc_splitk(da, db, c))):
        c.fill_bytes(0xEE)
        call()
        close_enough(oracle, c.to_numpy(), ref, K, dtype, f"{what} {shape}")
    for t in (da, db, c):
        t.free()


@pytest.mark.parametrize("shape", [(64, 36, 64), (130, 70, 50), (5, 3, 9), (257, 1001, 129)])
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_matmul_nn_any_n(gpu, beamc, oracle, shape, dtype):
    M, N, K = shape
    a = beamc.host_uniform((M, K), dtype, 62, 0)
    b = beamc.host_uniform((K, N), dtype, 62, 1)
    ref = oracle.matmul_nn(a, b, dtype)
    da, db = beamc.DeviceArray.from_numpy(a, dtype), beamc.DeviceArray.from_numpy(b, dtype)
    c = beamc.DeviceArray((M, N), dtype)
    c.fill_bytes(0xEE)
    beamc.matmul(da, db, c)
    close_enough(oracle, c.to_numpy(), ref, K, dtype, f"matmul {shape}")
    for t in (da, db, c):
        t.free()


@pytest.mark.parametrize("shape", [(130, 70, 50), (33, 257, 1001), (3, 5, 7)])
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemmrc_ln_any_k(gpu, beamc, oracle, shape, dtype):
    M, N, K = shape
    a, b, g, bt = make_ln_inputs(beamc, M, N, K, dtype, 63)
    ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, dtype)
    da, db = beamc.DeviceArray.from_numpy(a, dtype), beamc.DeviceArray.from_numpy(b, dtype)
    dg, dbt = beamc.DeviceArray.from_numpy(g, dtype), beamc.DeviceArray.from_numpy(bt, dtype)
    y = beamc.DeviceArray((M, N), dtype)
    for mode in (beamc.LN_AUTO, beamc.LN_TWOPASS, beamc.LN_FUSED):  # whatever is named: the problem decides
        y.fill_bytes(0xEE)
        beamc.gemmrc_ln(da, db, y, dg, dbt, mode=mode)
        check_ln(oracle, y.to_numpy(), ref, dtype, f"LayerNorm {shape} mode {mode}")
    for t in (da, db, dg, dbt, y):
        t.free()


def test_unaligned_operands(gpu, beamc, oracle):
    """A, B and C two bytes past a 16-byte boundary (views into larger buffers), K a multiple of 8."""
    M, N, K = 96, 80, 128
    a = beamc.host_uniform((M, K), F16, 64, 0)
    b = beamc.host_uniform((N, K), F16, 64, 1)
    ref = oracle.gemmrc(a, b, F16)
    bufs = [beamc.DeviceArray((n + 8,), F16) for n in (M * K, N * K, M * N)]
    L = beamc.lib
    for buf, host in ((bufs[0], a), (bufs[1], b)):
        beamc._check(L.beam_memcpy_h2d(buf.ptr + 2, host.ctypes.data, host.nbytes))
    bufs[2].fill_bytes(0xEE)
    beamc._check(L.beam_gemmrc(bufs[0].ptr + 2, bufs[1].ptr + 2, bufs[2].ptr + 2, M, N, K, F16, None, None))
    beamc.sync()
    out = bufs[2].to_numpy()
    assert out[0] == 0xEEEE and (out[1 + M * N:] == 0xEEEE).all()  # nothing outside C was written
    assert_close(oracle, out[1:1 + M * N].reshape(M, N), ref, K, F16, "unaligned operands")
    for t in bufs:
        t.free()
