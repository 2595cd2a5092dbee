"""Pins the CPU oracle (oracle/beam_oracle.c) without any GPU:

* against the committed float64 fixtures (tests/golden, made by numpy from the definition);
* against closed forms (identity, all-ones, one-hot) whose answers are exact;
* against a brute-force double-precision triple loop on tiny and ragged shapes;
* its 16-bit converters against numpy's float16 and against every bf16 rounding case;
* its split-K restatement against linearity (slices sum to the whole) and S=1 identity;
* its LayerNorm against invariants (mean 0 / variance 1, constant rows give beta);
* its slice heuristic against the worked example of the reference's formula (4 tiles on 108
  units -> 41 slices) and an independent pure-Python restatement.

A dropped term, a transposed operand, a wrong sign or a truncating conversion fails one of these.
"""
import glob
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F16, BF16 = 0, 1


def bits_to_f64(bits, dtype):
    if dtype == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return bits.view(np.float16).astype(np.float64)


def test_fixtures_exist():
    assert len(glob.glob(os.path.join(GOLDEN, "gemm_*.npz"))) >= 6
    assert len(glob.glob(os.path.join(GOLDEN, "ln_*.npz"))) >= 4


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "gemm_*.npz"))))
def test_gemm_against_float64_fixture(oracle, path):
    f = np.load(path)
    a, b, dtype, c64 = f["a"], f["b"], int(f["dtype"]), f["c64"]
    K = a.shape[1]
    c32, c16 = oracle.gemmrc(a, b, dtype, want16=True)
    scale = np.sqrt(np.mean(c64 ** 2))
    # fp32 accumulation of K terms: error far below the parity bound, far above a wrong formula
    assert np.abs(c32 - c64).max() <= 2e-6 * np.sqrt(K) * max(scale, 1.0) + 1e-6
    # the rounded copy is the RN rounding of the fp32 result
    assert (c16 == oracle.from_f32(c32, dtype)).all()
    # a transposed B or swapped operands cannot pass: c64 is not symmetric for these shapes
    naive = oracle.gemmrc_naive_f64(a, b, dtype)
    assert np.abs(naive - c64).max() <= 1e-12 * max(scale, 1.0) * K


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "ln_*.npz"))))
def test_gemm_ln_against_float64_fixture(oracle, path):
    f = np.load(path)
    dtype = int(f["dtype"])
    y32 = oracle.gemmrc_ln(f["a"], f["b"], f["gamma"], f["beta"], float(f["eps"]), dtype)
    # x carries fp32 accumulation error ~1e-7 relative; it is amplified by 1/sigma ~ 1
    assert np.abs(y32 - f["y64"]).max() <= 2e-5


def test_closed_forms(oracle):
    n = 96
    eye = np.eye(n, dtype=np.float16).view(np.uint16)
    rng = np.random.default_rng(1)
    b = rng.uniform(-1, 1, (70, n)).astype(np.float16).view(np.uint16)
    c32, c16 = oracle.gemmrc(eye, b, F16, want16=True)
    assert (c16 == b.T).all()                               # I . B^T = B^T exactly
    K = 2048
    ones_a = np.ones((7, K), np.float16).view(np.uint16)
    ones_b = np.ones((9, K), np.float16).view(np.uint16)
    assert (oracle.gemmrc(ones_a, ones_b, F16) == K).all()  # exact in fp32 and in fp16
    idx = (np.arange(20) * 7) % 64
    a = np.zeros((20, 64), np.float16)
    a[np.arange(20), idx] = -2.0                            # one-hot rows, scaled by a power of two
    bb = rng.uniform(-1, 1, (30, 64)).astype(np.float16)
    got = oracle.gemmrc(a.view(np.uint16), bb.view(np.uint16), F16)
    assert (got == -2.0 * bb[:, idx].T.astype(np.float32)).all()


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 16), (7, 2, 9), (130, 70, 48), (6, 16, 512), (5, 17, 513), (13, 33, 1025)])
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_against_brute_force(oracle, shape, dtype):
    M, N, K = shape
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    a32 = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b32 = rng.uniform(-1, 1, (N, K)).astype(np.float32)
    a, b = oracle.from_f32(a32, dtype), oracle.from_f32(b32, dtype)
    ref = bits_to_f64(a, dtype) @ bits_to_f64(b, dtype).T
    got = oracle.gemmrc(a, b, dtype)
    assert np.abs(got - ref).max() <= 1e-6 * K ** 0.5 + 1e-6
    assert np.abs(oracle.gemmrc_naive_f64(a, b, dtype) - ref).max() <= 1e-12 * K


def test_f16_converters_match_numpy(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    f = oracle.to_f32(allbits, F16)
    want = allbits.view(np.float16).astype(np.float32)
    assert (f.view(np.uint32) == want.view(np.uint32)).all()
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(2_000_00) * 10.0 ** rng.integers(-9, 6, 2_000_00)).astype(np.float32)
    # ties, subnormals, overflow boundary, signed zeros, infinities
    special = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -24,
                        2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 1.0 + 2.0 ** -11,
                        1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20], np.float32)
    x = np.concatenate([x, special, -special])
    with np.errstate(over="ignore"):
        want16 = x.astype(np.float16).view(np.uint16)
    assert (oracle.from_f32(x, F16) == want16).all()
    assert oracle.from_f32(np.array([np.nan], np.float32), F16)[0] & 0x7C00 == 0x7C00


def test_bf16_converters(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    f = oracle.to_f32(allbits, BF16)
    assert (f.view(np.uint32) == (allbits.astype(np.uint32) << 16)).all()
    # round to nearest even on the 16 dropped bits, checked against integer arithmetic
    rng = np.random.default_rng(3)
    u = rng.integers(0, 0x7F800000, 300000, dtype=np.uint32)
    u = np.concatenate([u, np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF], np.uint32)])
    x = u.view(np.float32)
    got = oracle.from_f32(x, BF16).astype(np.uint32)
    lo = u & 0xFFFF
    up = (lo > 0x8000) | ((lo == 0x8000) & (((u >> 16) & 1) == 1))
    assert (got == (u >> 16) + up).all()


def test_splitk_restatement(oracle):
    rng = np.random.default_rng(4)
    M, N, K = 37, 29, 1000
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16).view(np.uint16)
    b = rng.uniform(-1, 1, (N, K)).astype(np.float16).view(np.uint16)
    whole = oracle.gemmrc(a, b, F16)
    assert (oracle.gemmrc_splitk(a, b, 1, F16) == whole).all()          # one slice = the plain GEMM
    ref = bits_to_f64(a, F16) @ bits_to_f64(b, F16).T
    for s in (2, 3, 7, 16, 64):
        got = oracle.gemmrc_splitk(a, b, s, F16)
        assert np.abs(got - ref).max() <= 1e-4
        # slices partition K: the sum of per-slice float64 products is the whole product
        L = oracle.split_k_len(K, s)
        assert L % 64 == 0 and L * s >= K
        parts = sum(bits_to_f64(a[:, i * L:(i + 1) * L], F16) @ bits_to_f64(b[:, i * L:(i + 1) * L], F16).T
                    for i in range(s))
        assert np.abs(parts - ref).max() <= 1e-9


def test_ln_invariants(oracle):
    rng = np.random.default_rng(5)
    M, N, K = 19, 300, 64
    a = rng.standard_normal((M, K)).astype(np.float16).view(np.uint16)
    b = rng.standard_normal((N, K)).astype(np.float16).view(np.uint16)
    ones = np.ones(N, np.float16).view(np.uint16)
    zeros = np.zeros(N, np.uint16)
    y = oracle.gemmrc_ln(a, b, ones, zeros, 0.0, F16).astype(np.float64)
    assert np.abs(y.mean(axis=1)).max() < 1e-5
    assert np.abs(y.var(axis=1) - 1.0).max() < 1e-4
    beta = rng.standard_normal(N).astype(np.float16)
    y0 = oracle.gemmrc_ln(np.zeros_like(a), b, ones, beta.view(np.uint16), 1e-5, F16)
    assert (y0 == beta.astype(np.float32)[None, :]).all()      # constant rows: y = beta
    # scaling x by 4 leaves y unchanged when eps = 0 (variance over N, not N-1, either way)
    a4 = (a.view(np.float16) * np.float16(4)).view(np.uint16)
    y4 = oracle.gemmrc_ln(a4, b, ones, zeros, 0.0, F16)
    assert np.abs(y4 - y).max() < 1e-4
    # biased variance: for a row with values (+1, -1) repeated, var = 1 exactly -> y = x
    K2 = 8
    a2 = np.zeros((1, K2), np.float16)
    a2[0, 0] = 1
    b2 = np.zeros((4, K2), np.float16)
    b2[:, 0] = [1, -1, 1, -1]
    y2 = oracle.gemmrc_ln(a2.view(np.uint16), b2.view(np.uint16), np.ones(4, np.float16).view(np.uint16),
                          np.zeros(4, np.uint16), 0.0, F16)
    assert np.allclose(y2, [[1, -1, 1, -1]], atol=1e-6)


def _heuristic_py(tiles, units):
    f = np.float32
    s = 1
    if f(tiles) < f(units):
        s = int((f(units) - f(1)) / f(tiles) + f(1))
        while True:
            waves = f(s) * f(tiles) / f(units)
            if waves - f(int(waves)) >= f(0.5):
                break
            s += 1
    return s


def test_slice_heuristic(oracle):
    assert oracle.slice_heuristic(4, 108.0) == 41       # worked example of the reference's rule
    assert oracle.slice_heuristic(108, 108.0) == 1
    assert oracle.slice_heuristic(500, 108.0) == 1
    for units in (108, 256):
        for tiles in range(1, units + 3):
            assert oracle.slice_heuristic(tiles, float(units)) == _heuristic_py(tiles, units)


def test_metric_and_compare(oracle):
    assert oracle.tflops(4096, 4096, 4096, 1.0) == pytest.approx(2 * 4096 ** 3 / 1e9)
    ref = np.array([1.0, -2.0, 3.0, 0.5], np.float32)
    got = np.array([1.0, -2.0, 3.5, 0.5], np.float16).view(np.uint16)
    r = oracle.compare(got, ref, F16)
    assert r["max_abs_err"] == pytest.approx(0.5)
    assert r["rms_ref"] == pytest.approx(np.sqrt((1 + 4 + 9 + 0.25) / 4))
    assert r["max_abs_ref"] == 3.0
    assert oracle.gemm_tolerance(1024) == pytest.approx(1e-2)
    assert oracle.gemm_tolerance(4096) == pytest.approx(2e-2)


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_silu_exhaustive_against_library_sigmoid(oracle):
    """Every fp16 and every bf16 input: the fp32 oracle against x * expit(x) evaluated in float64 by
    scipy, and its 16-bit rounding against numpy's / the bit-level RN rounding of the float64 value."""
    from scipy.special import expit
    allbits = np.arange(65536, dtype=np.uint16)
    for dtype in (oracle.F16, oracle.BF16):
        with np.errstate(invalid="ignore"):  # (widening a signalling NaN)
            x = allbits.view(np.float16).astype(np.float64) if dtype == oracle.F16 else _bf16_to_f32(allbits).astype(np.float64)
        y32, y16 = oracle.silu(allbits, dtype)
        fin = np.isfinite(x)
        with np.errstate(over="ignore", invalid="ignore"):
            want = x * expit(x)
        # Below x = -88.7 exp(-x) overflows in fp32 and the formula returns -0 where the exact value
        # is a denormal of magnitude up to 1.2e-36: that flush belongs to the reference's formula.
        assert np.allclose(y32[fin], want[fin], rtol=4e-7, atol=2e-36)
        assert np.isnan(y32[np.isnan(x)]).all()
        assert y32[x == np.inf][0] == np.inf
        got = y16.view(np.float16).astype(np.float64) if dtype == oracle.F16 else _bf16_to_f32(y16).astype(np.float64)
        ulp = 2.0 ** -10 if dtype == oracle.F16 else 2.0 ** -7
        tiny = 2.0 ** -24 if dtype == oracle.F16 else 4e-36
        assert (np.abs(got[fin] - want[fin]) <= 0.5001 * ulp * np.abs(want[fin]) + 0.5001 * tiny).all()


def test_silu_identities(oracle):
    """silu(x) - silu(-x) = x; silu(0) = 0; silu(x) -> x for large x; the global minimum
    -0.27846454 at x = -1.27846454 (root of 1 + e^x + x = 0 ... i.e. x = -(1 + e^x))."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(4096) * 4).astype(np.float16)
    pos, _ = oracle.silu(x.view(np.uint16), oracle.F16)
    neg, _ = oracle.silu((-x).view(np.uint16), oracle.F16)
    assert np.allclose(pos - neg, x.astype(np.float32), rtol=0, atol=3e-6)
    z32, z16 = oracle.silu(np.array([0x0000, 0x8000], dtype=np.uint16), oracle.F16)
    assert (z32 == 0).all() and (z16 & 0x7FFF == 0).all()
    big = np.array([20.0, 100.0, 60000.0], dtype=np.float16)
    b32, b16 = oracle.silu(big.view(np.uint16), oracle.F16)
    assert (b16 == big.view(np.uint16)).all()
    grid = np.arange(-2.0, 0.0, 2.0 ** -10, dtype=np.float16)  # exactly representable steps
    g32, _ = oracle.silu(grid.view(np.uint16), oracle.F16)
    k = int(np.argmin(g32))
    assert abs(float(grid[k]) + 1.27846454) < 2.0 ** -10 and abs(float(g32[k]) + 0.27846454) < 1e-6
