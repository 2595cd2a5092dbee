"""Fused GEMM + LayerNorm through the C ABI against the oracle: |Y_gpu - Y_ref| <= 2e-3 absolute,
Y_ref being the oracle's un-rounded fp32 result."""
import numpy as np
import pytest

from test_gpu_gemm import F16, BF16

pytestmark = pytest.mark.gpu

LN_TOL = 2e-3


def make_ln_inputs(beamc, M, N, K, dtype, seed):
    a = beamc.host_normal((M, K), dtype, seed, 0, 0.0, K ** -0.5)
    b = beamc.host_normal((N, K), dtype, seed, 1, 0.0, K ** -0.5)
    gamma = beamc.host_normal((N,), dtype, seed, 2, 1.0, 0.1)
    beta = beamc.host_normal((N,), dtype, seed, 3, 0.0, 0.1)
    return a, b, gamma, beta


def run_ln(beamc, a, b, gamma, beta, dtype, eps=1e-5, config=None, mode=0):
    M, N = a.shape[0], b.shape[0]
    da, db = beamc.DeviceArray.from_numpy(a, dtype), beamc.DeviceArray.from_numpy(b, dtype)
    dg, dbt = beamc.DeviceArray.from_numpy(gamma, dtype), beamc.DeviceArray.from_numpy(beta, dtype)
    y = beamc.DeviceArray((M, N), dtype)
    y.fill_bytes(0xEE)
    beamc.gemmrc_ln(da, db, y, dg, dbt, eps=eps, config=config, mode=mode)
    out = y.to_numpy()
    assert not beamc.gemmrc_ln_timed_out()
    for x in (da, db, dg, dbt, y):
        x.free()
    return out


def check_ln(oracle, got_bits, ref32, dtype, what):
    r = oracle.compare(got_bits, ref32, dtype)
    if dtype == F16:
        # fp16 rounding alone is within 2e-3 only below 8.0; the inputs are chosen so that holds
        assert r["max_abs_ref"] < 8.0, f"{what}: |y| reaches {r['max_abs_ref']}"
        assert r["max_abs_err"] <= LN_TOL, f"{what}: {r['max_abs_err']:.4g} > {LN_TOL}"
    else:
        assert r["max_bf16_excess"] <= LN_TOL, f"{what}: {r['max_bf16_excess']:.4g} > {LN_TOL}"


@pytest.mark.parametrize("shape", [(256, 512, 256), (1024, 1024, 512), (300, 1000, 200), (64, 4096, 128),
                                   (17, 40, 64), (16384, 2048, 128), (4200, 1000, 72)])
def test_ln_small(gpu, beamc, oracle, shape):
    M, N, K = shape
    for dtype in (F16, BF16):
        a, b, g, bt = make_ln_inputs(beamc, M, N, K, dtype, 21)
        ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, dtype)
        for cfg in [None, beamc.TileConfig(128, 128, 64, 64), beamc.TileConfig(64, 64, 32, 32),
                    beamc.TileConfig(256, 256, 128, 64)]:
            for mode in (beamc.LN_TWOPASS, beamc.LN_FUSED):
                got = run_ln(beamc, a, b, g, bt, dtype, config=cfg, mode=mode)
                check_ln(oracle, got, ref, dtype, f"{shape} dtype {dtype} {cfg.name if cfg else 'default'} mode {mode}")


def test_ln_every_config(gpu, beamc, oracle):
    """Ragged 300 x 1000 x 200, every compiled tile with every LDS slot count, both modes.  With two
    slots per operand the 256-row tiles stage their output through LDS in two passes."""
    M, N, K = 300, 1000, 200
    a, b, g, bt = make_ln_inputs(beamc, M, N, K, F16, 23)
    ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, F16)
    for cfg in beamc.list_configs():
        for pipe in (0, 1, 2):
            c = beamc.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, pipe, 0)
            for mode in (beamc.LN_TWOPASS, beamc.LN_FUSED):
                got = run_ln(beamc, a, b, g, bt, F16, config=c, mode=mode)
                check_ln(oracle, got, ref, F16, f"{c.name} mode {mode}")


def test_ln_4096_cube(gpu, beamc, oracle):
    """X[4096x4096] . W[4096x4096]^T, LayerNorm over N = 4096, eps = 1e-5."""
    M = N = K = 4096
    a, b, g, bt = make_ln_inputs(beamc, M, N, K, F16, 22)
    ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, F16)
    for mode in (beamc.LN_TWOPASS, beamc.LN_FUSED):
        got = run_ln(beamc, a, b, g, bt, F16, mode=mode)
        check_ln(oracle, got, ref, F16, f"4096^3 mode {mode}")


def test_ln_many_column_tiles(gpu, beamc, oracle):
    """N = 11008 (43 column tiles of 256: one band spans two XCDs) and a 64-wide tile with 64 column
    tiles (the most the fused path takes); beyond that AUTO falls back to two passes."""
    for (M, N, K, cfg) in [(512, 11008, 256, None), (128, 4096, 128, beamc.TileConfig(64, 64, 32, 32)),
                           (130, 4100, 136, beamc.TileConfig(64, 64, 32, 32))]:
        a, b, g, bt = make_ln_inputs(beamc, M, N, K, F16, 24)
        ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, F16)
        got = run_ln(beamc, a, b, g, bt, F16, config=cfg, mode=beamc.LN_AUTO)
        check_ln(oracle, got, ref, F16, f"{(M, N, K)} auto")
    with pytest.raises(beamc.BeamError):
        a, b, g, bt = make_ln_inputs(beamc, 64, 8192, 64, F16, 25)
        run_ln(beamc, a, b, g, bt, F16, config=beamc.TileConfig(64, 64, 32, 32), mode=beamc.LN_FUSED)


def test_ln_invariants(gpu, beamc, oracle):
    """gamma = 1, beta = 0: every row has mean 0 and variance 1; a constant row gives beta."""
    M, N, K = 128, 2048, 256
    a, b, _, _ = make_ln_inputs(beamc, M, N, K, F16, 23)
    ones = np.ones((N,), np.float16).view(np.uint16)
    zeros = np.zeros((N,), np.uint16)
    y = run_ln(beamc, a, b, ones, zeros, F16).view(np.float16).astype(np.float64)
    assert np.abs(y.mean(axis=1)).max() < 2e-3
    assert np.abs(y.var(axis=1) - 1.0).max() < 5e-3
    # A = 0 gives x = 0 on every row: y = beta exactly (eps keeps rstd finite)
    beta = beamc.host_normal((N,), F16, 23, 3, 0.0, 0.1)
    y0 = run_ln(beamc, np.zeros_like(a), b, ones, beta, F16)
    assert (y0 == beta[None, :]).all()
    # large common offset: statistics must not lose the variance to cancellation
    K2 = 64
    a2 = np.full((64, K2), 1.0, np.float16).view(np.uint16)
    b2 = (np.float16(8.0) + beamc.host_uniform((N, K2), F16, 23, 5).view(np.float16) * np.float16(0.01)).astype(np.float16).view(np.uint16)
    ref = oracle.gemmrc_ln(a2, b2, ones, zeros, 1e-5, F16)
    got = run_ln(beamc, a2, b2, ones, zeros, F16)
    r = oracle.compare(got, ref, F16)
    assert r["max_abs_err"] <= 4e-3, r


def test_ln_fused_timeout_is_reported_not_hung(gpu, beamc):
    """With a zero poll budget every workgroup gives up waiting at once: the kernel still ends normally,
    the flag is raised, and the next call with the normal budget is correct again."""
    M, N, K = 512, 4096, 256
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 26)
    good = run_ln(beamc, a, b, g_, bt, F16, mode=beamc.LN_FUSED)
    try:
        assert beamc.lib.beam_set_ln_spin_limit(0) == 0
        da, db = beamc.DeviceArray.from_numpy(a), beamc.DeviceArray.from_numpy(b)
        dg, dbt = beamc.DeviceArray.from_numpy(g_), beamc.DeviceArray.from_numpy(bt)
        y = beamc.DeviceArray((M, N))
        beamc.gemmrc_ln(da, db, y, dg, dbt, mode=beamc.LN_FUSED)
        beamc.sync()
        assert beamc.gemmrc_ln_timed_out()
    finally:
        beamc.lib.beam_set_ln_spin_limit(4 << 20)
    beamc.lib.beam_gemmrc_ln_workspace_reset(beamc._ln_workspace.ptr)
    again = run_ln(beamc, a, b, g_, bt, F16, mode=beamc.LN_FUSED)
    assert (again == good).all()
