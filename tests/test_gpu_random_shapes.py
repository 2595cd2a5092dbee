"""Seeded sweep over odd shapes: every entry point that multiplies, a random tile, against the CPU oracle.

Shapes are drawn so that M and N straddle tile edges in every way (1 .. 700, not multiples of anything),
K covers short loops, tails of every multiple of 8 and several tiles; the [K][N] layout gets N rounded
to its multiple of 8.  Bounds: the GEMM bound of the other tests; LayerNorm 2e-3 absolute; split-K also
bit-identical between two runs.  Below K = 64 the GEMM bound (which shrinks with sqrt(K)) is smaller than
the rounding of an fp16 output by itself, so there the error in excess of half an fp16 ulp, |ref| * 2^-11,
is held to it -- the same kind of allowance bf16 needs at every K.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F16, BF16 = 0, 1


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        M = int(rng.integers(1, 700))
        N = int(rng.integers(1, 700))
        K = int(rng.choice([8, 16, 24, 56, 64, 72, 120, 128, 200, 256, 264, 520, 1000, 2048]))
        out.append((M, N, K, int(rng.integers(0, 2)), int(rng.integers(0, 1 << 30))))
    return out


def _tile(beamc, rng, pipelines):
    cfgs = beamc.list_configs()
    c = cfgs[int(rng.integers(0, len(cfgs)))]
    return beamc.TileConfig(c.block_m, c.block_n, c.wave_m, c.wave_n, int(rng.choice(pipelines)), int(rng.choice([0, 1, 3, 8])))


def _close(oracle, got, ref, K, dtype, what):
    r = oracle.compare(got, ref, dtype)
    err = r["max_abs_err"] if dtype == F16 else r["max_bf16_excess"]
    if dtype == F16 and K < 64:
        g32 = got.view(np.float16).astype(np.float32)
        err = float((np.abs(g32 - ref) - np.abs(ref) * 2.0 ** -11).max())
    assert err <= oracle.gemm_tolerance(K) * max(r["rms_ref"], 1e-30), f"{what}: {err:.4g} (rms {r['rms_ref']:.4g})"


def test_random_shapes(gpu, beamc, oracle):
    for M, N, K, dtype, seed in _cases(160, 2024):
        rng = np.random.default_rng(seed)
        a = beamc.host_uniform((M, K), dtype, seed, 0)
        b = beamc.host_uniform((N, K), dtype, seed, 1)
        ref = oracle.gemmrc(a, b, dtype)
        da, db = beamc.DeviceArray.from_numpy(a, dtype), beamc.DeviceArray.from_numpy(b, dtype)
        dc = beamc.DeviceArray((M, N), dtype)
        what = f"M={M} N={N} K={K} dtype={dtype}"
        # plain
        cfg = _tile(beamc, rng, [0, 1, 2])
        dc.fill_bytes(0xEE)
        beamc.gemmrc(da, db, dc, config=cfg)
        _close(oracle, dc.to_numpy(), ref, K, dtype, f"gemmrc {cfg.name} {what}")
        # split-K, twice
        cfg = _tile(beamc, rng, [0, 2])
        s = int(rng.choice([2, 3, 4, 8, 16]))
        outs = []
        for _ in range(2):
            dc.fill_bytes(0xEE)
            beamc.gemmrc_splitk_spec(da, db, dc, shape_threadblock=[cfg.block_m, cfg.block_n],
                                     shape_warp=[cfg.wave_m, cfg.wave_n], split_k_slices=s, pipeline=cfg.pipeline)
            outs.append(dc.to_numpy())
        _close(oracle, outs[0], ref, K, dtype, f"split-K {cfg.name} S={s} {what}")
        assert (outs[0] == outs[1]).all(), f"split-K not reproducible: {cfg.name} S={s} {what}"
        # GEMM carrying a SiLU array
        cfg = _tile(beamc, rng, [0, 1])
        n = int(rng.integers(0, 50000))
        x = beamc.host_normal((max(n, 1),), dtype, seed, 2, 0.0, 3.0)[:n]
        dx = beamc.DeviceArray.from_numpy(np.concatenate([x, np.zeros(8, np.uint16)]), dtype)
        dy = beamc.DeviceArray((n + 8,), dtype)
        dy.fill_bytes(0xEE)
        xv, yv = beamc.DeviceArray.__new__(beamc.DeviceArray), beamc.DeviceArray.__new__(beamc.DeviceArray)
        for v, src in ((xv, dx), (yv, dy)):
            v.shape, v.dtype, v.itemsize, v.nbytes, v.ptr = (n,), dtype, 2, n * 2, src.ptr
        dc.fill_bytes(0xEE)
        beamc.parallel_gemmrc_silu(da, db, dc, xv, yv, config=cfg)
        _close(oracle, dc.to_numpy(), ref, K, dtype, f"gemm+silu {cfg.name} {what}")
        y = dy.to_numpy()
        assert (y[n:] == 0xEEEE).all(), f"side job wrote past its array: {cfg.name} n={n} {what}"
        if n:
            _, want = oracle.silu(x, dtype)
            o = lambda t: np.where(t.astype(np.int32) & 0x8000, -(t.astype(np.int32) & 0x7FFF), t.astype(np.int32) & 0x7FFF)
            assert np.abs(o(y[:n]) - o(want)).max() <= 1, f"side job: {cfg.name} n={n} {what}"
        xv.ptr = yv.ptr = 0
        # B stored [K][N]
        N8 = max(8, N // 8 * 8)
        bkn = beamc.host_uniform((K, N8), dtype, seed, 3)
        dbk = beamc.DeviceArray.from_numpy(bkn, dtype)
        dc8 = beamc.DeviceArray((M, N8), dtype)
        cfg = _tile(beamc, rng, [0, 1, 2])
        dc8.fill_bytes(0xEE)
        beamc.matmul(da, dbk, dc8, config=cfg)
        _close(oracle, dc8.to_numpy(), oracle.matmul_nn(a, bkn, dtype), K, dtype, f"matmul_nn {cfg.name} M={M} N={N8} K={K}")
        # GEMM + LayerNorm, both modes where the fused one applies
        g = beamc.host_normal((N,), dtype, seed, 4, 1.0, 0.1)
        bt = beamc.host_normal((N,), dtype, seed, 5, 0.0, 0.1)
        an = beamc.host_normal((M, K), dtype, seed, 6, 0.0, K ** -0.5)
        bn = beamc.host_normal((N, K), dtype, seed, 7, 0.0, K ** -0.5)
        yref = oracle.gemmrc_ln(an, bn, g, bt, 1e-5, dtype)
        dan, dbn = beamc.DeviceArray.from_numpy(an, dtype), beamc.DeviceArray.from_numpy(bn, dtype)
        dg, dbt = beamc.DeviceArray.from_numpy(g, dtype), beamc.DeviceArray.from_numpy(bt, dtype)
        cfg = _tile(beamc, rng, [0, 1])
        for mode in (beamc.LN_TWOPASS, beamc.LN_AUTO):
            dc.fill_bytes(0xEE)
            beamc.gemmrc_ln(dan, dbn, dc, dg, dbt, eps=1e-5, config=cfg, mode=mode)
            r = oracle.compare(dc.to_numpy(), yref, dtype)
            err = r["max_abs_err"] if dtype == F16 else r["max_bf16_excess"]
            assert err <= oracle.LN_ABS_TOL, f"LN mode {mode} {cfg.name} {what}: {err:.4g}"
        assert not beamc.gemmrc_ln_timed_out()
        for t in (da, db, dc, dx, dy, dbk, dc8, dan, dbn, dg, dbt):
            t.free()
