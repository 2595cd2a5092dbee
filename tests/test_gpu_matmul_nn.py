"""C = A . B with B stored [K][N] (beam_matmul_nn) against the CPU oracle, and against beam_gemmrc on
the transposed copy of B: both kernels add the same products in the same order, so their outputs
must be bit-identical.  Bound against the oracle: the GEMM bound used everywhere,
max|C_gpu - C_ref| <= 1e-2 * sqrt(K/1024) * RMS(C_ref) (bf16: error in excess of |ref|/256).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F16, BF16 = 0, 1


def run_nn(beamc, a_bits, b_kn_bits, dtype, config=None):
    M, K = a_bits.shape
    N = b_kn_bits.shape[1]
    a = beamc.DeviceArray.from_numpy(a_bits, dtype)
    b = beamc.DeviceArray.from_numpy(b_kn_bits, dtype)
    full = beamc.DeviceArray((M + 4, N), dtype)
    full.fill_bytes(0xEE)
    c = beamc.DeviceArray.__new__(beamc.DeviceArray)
    c.shape, c.dtype, c.itemsize, c.nbytes, c.ptr = (M, N), dtype, 2, M * N * 2, full.ptr
    try:
        beamc.matmul(a, b, c, config=config)
        out = full.to_numpy()
    finally:
        c.ptr = 0
        for x in (a, b, full):
            x.free()
    assert (out[M:] == 0xEEEE).all(), "kernel wrote past the end of C"
    return out[:M]


def run_rc(beamc, a_bits, b_nk_bits, dtype, config=None):
    a = beamc.DeviceArray.from_numpy(a_bits, dtype)
    b = beamc.DeviceArray.from_numpy(b_nk_bits, dtype)
    c = beamc.DeviceArray((a_bits.shape[0], b_nk_bits.shape[0]), dtype)
    try:
        beamc.gemmrc(a, b, c, config=config)
        return c.to_numpy()
    finally:
        for x in (a, b, c):
            x.free()


def check(oracle, got, ref, K, dtype, what):
    r = oracle.compare(got, ref, dtype)
    err = r["max_abs_err"] if dtype == F16 else r["max_bf16_excess"]
    tol = oracle.gemm_tolerance(K) * r["rms_ref"]
    assert err <= tol, f"{what}: max err {err:.4g} > {tol:.4g}"


def test_every_config_1024_cube(gpu, beamc, oracle):
    M = N = K = 1024
    a = beamc.host_uniform((M, K), F16, 1, 0)
    b = beamc.host_uniform((K, N), F16, 1, 1)
    ref = oracle.matmul_nn(a, b, F16)
    bt = np.ascontiguousarray(b.T)
    for cfg in beamc.list_configs():
        for pipe in (0, 1, 2):
            c = beamc.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, pipe, 0)
            got = run_nn(beamc, a, b, F16, c)
            check(oracle, got, ref, K, F16, c.name)
            assert (got == run_rc(beamc, a, bt, F16, c)).all(), f"{c.name}: differs from gemmrc on B^T"


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("shape", [(300, 200, 136), (1, 8, 8), (257, 264, 72), (130, 72, 48), (64, 4096, 64), (513, 520, 1000)])
def test_ragged_shapes_every_config(gpu, beamc, oracle, shape, dtype):
    """Edge tiles in M and N (N a multiple of 8), K tails of 8 .. 56, K shorter than one tile."""
    M, N, K = shape
    a = beamc.host_uniform((M, K), dtype, 3, 0)
    b = beamc.host_uniform((K, N), dtype, 3, 1)
    ref = oracle.matmul_nn(a, b, dtype)
    for cfg in beamc.list_configs():
        check(oracle, run_nn(beamc, a, b, dtype, cfg), ref, K, dtype, f"{cfg.name} {shape}")
        deep = beamc.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, 2, 0)
        check(oracle, run_nn(beamc, a, b, dtype, deep), ref, K, dtype, f"{deep.name} {shape}")


@pytest.mark.parametrize("shape", [(768, 3072, 768), (256, 8192, 1024), (64, 4096, 512), (1280, 1280, 1280), (2048, 2048, 512)])
def test_library_chosen_tile(gpu, beamc, oracle, shape):
    """No tile named: the library takes the tile it would for gemmrc, except that tiles with 64-column wavefronts
    give way to their 32-column relatives in this layout (and not where that would make more tiles)."""
    M, N, K = shape
    a = beamc.host_uniform((M, K), F16, 5, 0)
    b = beamc.host_uniform((K, N), F16, 5, 1)
    check(oracle, run_nn(beamc, a, b, F16), oracle.matmul_nn(a, b, F16), K, F16, f"default {shape}")


def test_closed_forms(gpu, beamc):
    """A = I gives C = B exactly; B = ones gives row sums of A (exact in fp16 for small integers)."""
    n = 512
    eye = np.zeros((n, n), np.float16)
    np.fill_diagonal(eye, 1.0)
    b = beamc.host_uniform((n, n), F16, 4, 1)
    assert (run_nn(beamc, eye.view(np.uint16), b, F16) == b).all()
    a = (np.arange(n * n, dtype=np.int64).reshape(n, n) % 5 - 2).astype(np.float16)
    ones = np.ones((n, 264), np.float16)
    got = run_nn(beamc, a.view(np.uint16), ones.view(np.uint16), F16).view(np.float16).astype(np.float64)
    assert (got == a.astype(np.float64).sum(axis=1, keepdims=True)).all()


def test_full_size_equals_gemmrc_on_transpose(gpu, beamc, oracle):
    """8192 x 8192 x 4096: bit-identical to gemmrc on B^T, and a sampled check against the oracle."""
    M, N, K = 8192, 8192, 4096
    a = beamc.host_normal((M, K), F16, 7, 0, 0.0, K ** -0.5)
    b = beamc.host_normal((K, N), F16, 7, 1, 0.0, K ** -0.5)
    got = run_nn(beamc, a, b, F16)
    assert (got == run_rc(beamc, a, np.ascontiguousarray(b.T), F16)).all()
    rows = np.arange(0, M, 61)[:96]
    ref = oracle.matmul_nn(a[rows], b, F16)
    check(oracle, got[rows], ref, K, F16, "sampled rows")


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("shape", [(4352, 4360, 192), (3000, 5000, 2048), (257, 264, 448), (8192, 520, 1024), (512, 256, 4096)])
def test_four_wavefront_kernel(gpu, beamc, oracle, shape, dtype):
    """The 256 x 256 tile of four 128 x 128 wavefronts with B as [K][N]: more tiles than CUs (a workgroup walks
    several, its operand ring running through the tile boundaries), edge tiles in M and N, the shortest K the
    kernel takes and a long one.  Bit-identical to gemmrc on B^T with the same tile, and sampled rows against the
    oracle."""
    M, N, K = shape
    cfg = beamc.TileConfig(256, 256, 128, 128, 0, 0)
    a = beamc.host_uniform((M, K), dtype, 11, 0)
    b = beamc.host_uniform((K, N), dtype, 11, 1)
    got = run_nn(beamc, a, b, dtype, cfg)
    assert (got == run_rc(beamc, a, np.ascontiguousarray(b.T), dtype, cfg)).all()
    rows = np.unique(np.concatenate([np.arange(0, M, 37), np.arange(max(0, M - 3), M)]))[:160]
    check(oracle, got[rows], oracle.matmul_nn(a[rows], b, dtype), K, dtype, f"{cfg.name} {shape}")


def test_four_wavefront_kernel_random_shapes(gpu, beamc, oracle):
    """Seeded odd shapes on the 4-wavefront kernel: any M, N a multiple of 8, K a multiple of 64 from 192 up,
    every raster group; one to a few dozen tiles, so single-tile workgroups, edge tiles and empty columns of
    tiles all occur."""
    rng = np.random.default_rng(77)
    for _ in range(24):
        M = int(rng.integers(1, 1500))
        N = 8 * int(rng.integers(1, 190))
        K = int(rng.choice([192, 256, 320, 448, 1024]))
        dtype = int(rng.integers(0, 2))
        cfg = beamc.TileConfig(256, 256, 128, 128, 0, int(rng.choice([0, 1, 3, 4, 8])))
        seed = int(rng.integers(0, 1 << 30))
        a = beamc.host_uniform((M, K), dtype, seed, 0)
        b = beamc.host_uniform((K, N), dtype, seed, 1)
        got = run_nn(beamc, a, b, dtype, cfg)
        what = f"M={M} N={N} K={K} dtype={dtype} group={cfg.group_m}"
        assert (got == run_rc(beamc, a, np.ascontiguousarray(b.T), dtype, cfg)).all(), what
        rows = np.unique(rng.integers(0, M, 48))
        check(oracle, got[rows], oracle.matmul_nn(a[rows], b, dtype), K, dtype, what)


def test_four_wavefront_kernel_streaming_stores(gpu, beamc, oracle):
    """An output beyond the last-level cache (12288 x 12288: 302 MB) takes the form with non-temporal stores."""
    M, N, K = 12288, 12288, 1024
    a = beamc.host_normal((M, K), F16, 13, 0, 0.0, K ** -0.5)
    b = beamc.host_normal((K, N), F16, 13, 1, 0.0, K ** -0.5)
    got = run_nn(beamc, a, b, F16)
    assert (got == run_rc(beamc, a, np.ascontiguousarray(b.T), F16)).all()
    rows = np.arange(0, M, 131)[:96]
    check(oracle, got[rows], oracle.matmul_nn(a[rows], b, F16), K, F16, "sampled rows")


def test_error_paths(gpu, beamc):
    a = beamc.DeviceArray((64, 64), F16)
    b = beamc.DeviceArray((64, 36), F16)
    b2 = beamc.DeviceArray((32, 64), F16)
    with pytest.raises(beamc.BeamError):
        beamc.matmul(a, b2)  # inner dimensions differ
    b3 = beamc.DeviceArray((64, 64), F16)
    with pytest.raises(beamc.BeamError) as e:
        beamc.matmul(a, b3, config=beamc.TileConfig(128, 128, 64, 64, 3, 0))  # no such LDS depth
    assert e.value.status == 2
    for t in (a, b, b2, b3):
        t.free()
