"""Parity of the tiled gemmrc kernels (through the C ABI) with the CPU oracle.

Bound for fp16: max|C_gpu - C_ref| <= 1e-2 * sqrt(K/1024) * RMS(C_ref), C_ref being the oracle's
un-rounded fp32 result.  bf16 output carries a half-ulp of 2^-9 relative by itself (more than
the bound at small K), so for bf16 the error in excess of |ref|/256 is held to the same bound.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F16, BF16 = 0, 1


def run_gemm(beamc, a_bits, b_bits, dtype, config=None, guard_rows=4):
    M, K = a_bits.shape
    N = b_bits.shape[0]
    a = beamc.DeviceArray.from_numpy(a_bits, dtype)
    b = beamc.DeviceArray.from_numpy(b_bits, dtype)
    # Output with guard rows behind it: a kernel writing past C is caught, not just wrong.
    full = beamc.DeviceArray((M + guard_rows, N), dtype)
    full.fill_bytes(0xEE)
    c = beamc.DeviceArray.__new__(beamc.DeviceArray)
    c.shape, c.dtype, c.itemsize, c.nbytes, c.ptr = (M, N), dtype, 2, M * N * 2, full.ptr
    try:
        beamc.gemmrc(a, b, c, config=config)
        out = full.to_numpy()
    finally:
        c.ptr = 0
        for x in (a, b, full):
            x.free()
    assert (out[M:] == 0xEEEE).all(), "kernel wrote past the end of C"
    return out[:M]


def assert_close(oracle, got_bits, ref32, K, dtype, what=""):
    r = oracle.compare(got_bits, ref32, dtype)
    tol = oracle.gemm_tolerance(K) * r["rms_ref"]
    err = r["max_abs_err"] if dtype == F16 else r["max_bf16_excess"]
    assert err <= tol, f"{what}: max err {err:.4g} > {tol:.4g} (rms {r['rms_ref']:.4g})"
    return r


def all_configs(beamc):
    out = []
    for cfg in beamc.list_configs():
        out.append(cfg)
        out.append(beamc.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, 1, 0))
        out.append(beamc.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, 2, 0))
    return out


def test_1024_cube_every_config(gpu, beamc, oracle):
    """fp16 1024^3, uniform[-1,1): every compiled tile, both pipeline depths."""
    M = N = K = 1024
    a = beamc.host_uniform((M, K), F16, 1, 0)
    b = beamc.host_uniform((N, K), F16, 1, 1)
    ref = oracle.gemmrc(a, b, F16)
    for cfg in all_configs(beamc):
        got = run_gemm(beamc, a, b, F16, cfg)
        assert_close(oracle, got, ref, K, F16, cfg.name)


@pytest.mark.parametrize("shape", [(3, 5, 16), (1, 1, 8), (130, 70, 48), (257, 129, 1000), (64, 64, 64),
                                   (300, 500, 200), (33, 1000, 72), (1000, 31, 136)])
def test_ragged_small_every_config(gpu, beamc, oracle, shape):
    M, N, K = shape
    a = beamc.host_uniform((M, K), F16, 2, 0)
    b = beamc.host_uniform((N, K), F16, 2, 1)
    ref = oracle.gemmrc(a, b, F16)
    naive = oracle.gemmrc_naive_f64(a, b, F16)
    assert np.abs(ref - naive).max() <= 1e-5 * max(1.0, np.abs(naive).max())
    for cfg in all_configs(beamc):
        got = run_gemm(beamc, a, b, F16, cfg)
        assert_close(oracle, got, ref, K, F16, f"{shape} {cfg.name}")


@pytest.mark.parametrize("shape", [(300, 264, 136), (257, 132, 72), (130, 70, 48)])
def test_output_8_byte_aligned(gpu, beamc, shape):
    """C needs 8-byte alignment only.  The epilogue writes 16-byte pieces of rows where it can
    (C 16-byte aligned and N % 8 == 0) and falls back to 8-byte or single-element stores otherwise:
    all three must give the same bits, and none may write outside C."""
    M, N, K = shape
    a_bits = beamc.host_uniform((M, K), F16, 5, 0)
    b_bits = beamc.host_uniform((N, K), F16, 5, 1)
    a = beamc.DeviceArray.from_numpy(a_bits, F16)
    b = beamc.DeviceArray.from_numpy(b_bits, F16)
    full = beamc.DeviceArray((M * N + 64,), F16)
    c = beamc.DeviceArray.__new__(beamc.DeviceArray)
    c.shape, c.dtype, c.itemsize, c.nbytes = (M, N), F16, 2, M * N * 2
    try:
        for cfg in all_configs(beamc):
            outs = []
            for shift in (0, 4, 8, 12):  # elements: 0, 8, 16 and 24 bytes past a 256-byte boundary
                full.fill_bytes(0xEE)
                c.ptr = full.ptr + 2 * shift
                beamc.gemmrc(a, b, c, config=cfg)
                out = full.to_numpy()
                assert (out[:shift] == 0xEEEE).all() and (out[shift + M * N:] == 0xEEEE).all(), (cfg.name, shift)
                outs.append(out[shift:shift + M * N])
            for o in outs[1:]:
                assert (o == outs[0]).all(), cfg.name
    finally:
        c.ptr = 0
        for x in (a, b, full):
            x.free()


def test_ragged_3000x5000x2000(gpu, beamc, oracle):
    """Edge tiles in M and N and a short last K tile (K = 31*64 + 16), fp16 and bf16."""
    M, N, K = 3000, 5000, 2000
    for dtype in (F16, BF16):
        a = beamc.host_uniform((M, K), dtype, 3, 0)
        b = beamc.host_uniform((N, K), dtype, 3, 1)
        ref = oracle.gemmrc(a, b, dtype)
        for cfg in [None] + [c for c in beamc.list_configs() if (c.block_m, c.block_n) in ((256, 256), (128, 128), (256, 128))]:
            got = run_gemm(beamc, a, b, dtype, cfg)
            assert_close(oracle, got, ref, K, dtype, f"dtype {dtype} {cfg.name if cfg else 'default'}")


def test_closed_forms(gpu, beamc, oracle):
    """Identity, all-ones and one-hot operands have exact answers."""
    n = 256
    eye = np.eye(n, dtype=np.float16).view(np.uint16)
    b = beamc.host_uniform((384, n), F16, 4, 1)
    got = run_gemm(beamc, eye, b, F16)            # C = I . B^T = B^T exactly
    assert (got == b.T).all()
    K = 2048
    ones_a = np.ones((100, K), np.float16).view(np.uint16)
    ones_b = np.ones((36, K), np.float16).view(np.uint16)
    got = run_gemm(beamc, ones_a, ones_b, F16)    # every element = K, exact in fp16
    assert (got.view(np.float16) == np.float16(K)).all()
    # one-hot rows of A pick single columns of B: C[m][n] = B[n][k_m]
    K = 512
    idx = (np.arange(200) * 37) % K
    a = np.zeros((200, K), np.float16)
    a[np.arange(200), idx] = 1
    b = beamc.host_uniform((300, K), F16, 4, 2)
    got = run_gemm(beamc, a.view(np.uint16), b, F16)
    assert (got == b[:, idx].T).all()


def test_bf16_sweep(gpu, beamc, oracle):
    for (M, N, K) in [(512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048)]:
        a = beamc.host_uniform((M, K), BF16, 5, 0)
        b = beamc.host_uniform((N, K), BF16, 5, 1)
        ref = oracle.gemmrc(a, b, BF16)
        for cfg in [None, beamc.TileConfig(128, 128, 64, 64), beamc.TileConfig(64, 64, 32, 32)]:
            got = run_gemm(beamc, a, b, BF16, cfg)
            assert_close(oracle, got, ref, K, BF16, f"{(M, N, K)}")
    for (M, N, K) in [(4096, 4096, 4096), (4096, 11008, 4096), (4096, 4096, 11008)]:
        a = beamc.host_uniform((M, K), BF16, 5, 0)
        b = beamc.host_uniform((N, K), BF16, 5, 1)
        assert_close(oracle, run_gemm(beamc, a, b, BF16), oracle.gemmrc(a, b, BF16), K, BF16, f"{(M, N, K)}")


@pytest.mark.parametrize("shape", [(512, 512, 512), (2048, 2048, 2048), (4096, 4096, 4096),
                                   (4096, 11008, 4096), (4096, 4096, 11008)])
def test_fp16_sweep(gpu, beamc, oracle, shape):
    M, N, K = shape
    a = beamc.host_uniform((M, K), F16, 6, 0)
    b = beamc.host_uniform((N, K), F16, 6, 1)
    ref = oracle.gemmrc(a, b, F16)
    got = run_gemm(beamc, a, b, F16)
    assert_close(oracle, got, ref, K, F16, f"{shape}")


@pytest.mark.parametrize("shape", [(4200, 4296, 128), (8192, 8200, 64), (2600, 9000, 192), (4096, 4104, 256), (5000, 5000, 320)])
def test_more_tiles_than_compute_units(gpu, beamc, oracle, shape):
    """More tiles than CUs: with 3 A + 2 B slots the large tiles run as one workgroup per CU that walks
    its tiles and prefetches the next one's operands during the store.  Ragged M and N (rows and
    columns dropped by the store's buffer descriptor), against the oracle and, bit for bit, against the
    same tile with 2 + 2 slots, which runs one workgroup per tile."""
    M, N, K = shape
    for dtype in (F16, BF16):
        a = beamc.host_uniform((M, K), dtype, 12, 0)
        b = beamc.host_uniform((N, K), dtype, 12, 1)
        ref = oracle.gemmrc(a, b, dtype)
        for tile in ((256, 256, 128, 64), (224, 256, 112, 64), (192, 256, 96, 64)):
            walk = run_gemm(beamc, a, b, dtype, beamc.TileConfig(*tile, 0, 0))
            once = run_gemm(beamc, a, b, dtype, beamc.TileConfig(*tile, 1, 0))
            assert_close(oracle, walk, ref, K, dtype, f"{shape} {tile}")
            assert (walk == once).all(), (shape, tile)
        # The default tile: the 4-wavefront kernel where K >= 192 (one workgroup per CU, load streams that
        # run ahead across tile boundaries: at K = 192 the A stream changes tile in a tile's first K tile).
        assert_close(oracle, run_gemm(beamc, a, b, dtype), ref, K, dtype, f"{shape} default")


def _decode(bits, dtype):
    if dtype == F16:
        return bits.view(np.float16).astype(np.float64)
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_16384_cube_sampled_rows_and_column_sums(gpu, beamc, oracle, dtype):
    """The largest square of the sweep, 4096 tiles of 256 x 256.  The oracle computes one row out of every
    256-row band (every tile contributes columns to the comparison), and every element enters the
    column sums 1^T C, which must equal (1^T A) B^T (float64) up to the rounding of the 16-bit outputs."""
    M = N = K = 16384
    a = beamc.host_uniform((M, K), dtype, 8, 0)
    b = beamc.host_uniform((N, K), dtype, 8, 1)
    got = run_gemm(beamc, a, b, dtype)
    rows = np.array([t * 256 + (37 * t) % 256 for t in range(M // 256)])
    ref = oracle.gemmrc(np.ascontiguousarray(a[rows]), b, dtype)
    r = assert_close(oracle, np.ascontiguousarray(got[rows]), ref, K, dtype, "sampled rows")
    assert abs(r["rms_ref"] / (K ** 0.5 / 3) - 1) < 0.05      # RMS(C) = sqrt(K)/3 for uniform inputs
    bf = _decode(b, dtype)
    want = bf @ _decode(a, dtype).sum(axis=0)                  # [N]
    have = _decode(got, dtype).sum(axis=0)
    half_ulp = 2.0 ** -11 if dtype == F16 else 2.0 ** -8
    bound = 8 * np.sqrt(M) * half_ulp * 4 * r["rms_ref"]       # 8 sigma of M roundings of values up to ~4 RMS
    assert np.abs(have - want).max() <= bound, (np.abs(have - want).max(), bound)


def test_headline_8192_cube(gpu, beamc, oracle):
    """fp16 8192^3, N(0,1)/sqrt(K): default tile and the three named tiles, full oracle."""
    M = N = K = 8192
    a = beamc.host_normal((M, K), F16, 7, 0, 0.0, K ** -0.5)
    b = beamc.host_normal((N, K), F16, 7, 1, 0.0, K ** -0.5)
    ref = oracle.gemmrc(a, b, F16)
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    assert abs(rms * K ** 0.5 - 1.0) < 0.05          # RMS(C) = 1/sqrt(K) for these inputs
    for cfg in [None, beamc.TileConfig(128, 128, 64, 64), beamc.TileConfig(128, 256, 64, 64),
                beamc.TileConfig(256, 128, 64, 64)]:
        got = run_gemm(beamc, a, b, F16, cfg)
        assert_close(oracle, got, ref, K, F16, cfg.name if cfg else "default")


def test_fixed_tile_entry_points(gpu, beamc, oracle):
    """The three reference-named launchers (fp16 only)."""
    M, N, K = 512, 768, 1024
    a_bits = beamc.host_uniform((M, K), F16, 8, 0)
    b_bits = beamc.host_uniform((N, K), F16, 8, 1)
    ref = oracle.gemmrc(a_bits, b_bits, F16)
    a = beamc.DeviceArray.from_numpy(a_bits)
    b = beamc.DeviceArray.from_numpy(b_bits)
    c = beamc.DeviceArray((M, N))
    for fn in (beamc.custom_gemmrc_128x128, beamc.custom_gemmrc_128x256, beamc.custom_gemmrc_256x128):
        c.fill_bytes(0)
        fn(a=a, b=b, c=c)
        assert_close(oracle, c.to_numpy(), ref, K, F16, fn.__name__)


def test_error_codes(gpu, beamc):
    a = beamc.DeviceArray((64, 64))
    b = beamc.DeviceArray((64, 64))
    c = beamc.DeviceArray((64, 64))
    with pytest.raises(beamc.BeamError) as e:
        beamc.gemmrc_spec(a, b, c, shape_threadblock=[96, 96], shape_warp=[48, 48])
    assert e.value.status == 2
    with pytest.raises(beamc.BeamError) as e:
        beamc.gemmrc(a, b, beamc.DeviceArray((64, 32)))
    assert e.value.status == 1
    with pytest.raises(beamc.BeamError) as e:
        beamc.gemmrc_spec(a, b, c, shape_threadblock=[64, 64], shape_warp=[32, 32], pipeline=3)
    assert e.value.status == 2
    # empty problems are no-ops, K == 0 clears C
    beamc.gemmrc(beamc.DeviceArray((0, 64)), b, beamc.DeviceArray((0, 64)))
    c.fill_bytes(0x55)
    beamc.gemmrc(beamc.DeviceArray((64, 0)), beamc.DeviceArray((64, 0)), c)
    assert (c.to_numpy() == 0).all()
