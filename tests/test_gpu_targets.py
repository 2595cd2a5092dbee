"""Timing guards on the measured claims: a regression that leaves results correct (registers
spilled to scratch memory, a lost fast path) shows up here.  Thresholds are the stated targets or sit
well below the values measured on the slowest machine seen; every figure is the best of three rounds,
the first of which also absorbs the clock transient after idle."""
import pytest

pytestmark = pytest.mark.gpu

F16 = 0


def _best(fn, rounds=3):
    return min(fn() for _ in range(rounds))


def test_headline_throughput(gpu, beamc):
    """fp16 8192^3 on N(0,1)/sqrt(K) data: 1468-1570 TFLOP/s measured across machines (the 8-wavefront kernel this
    one replaced: 1445 on its best machine)."""
    M = N = K = 8192
    a = beamc.DeviceArray.from_numpy(beamc.host_normal((M, K), F16, 7, 0, 0.0, K ** -0.5))
    b = beamc.DeviceArray.from_numpy(beamc.host_normal((N, K), F16, 7, 1, 0.0, K ** -0.5))
    c = beamc.DeviceArray((M, N))
    try:
        ms = _best(lambda: beamc.bench(beamc.OP_GEMM, a, b, c, warmup=100, iters=100))
    finally:
        for t in (a, b, c):
            t.free()
    tflops = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    # The part is power limited on this data and machines differ by +-4%: a machine that misses the absolute figure
    # must at least keep the ratio to what its own matrix cores sustain from registers (0.77-0.79 measured).
    ceiling = max(beamc.probe_mfma(F16, warmup=50, iters=100)[1] for _ in range(2))
    assert tflops >= 1400.0 or tflops >= 0.75 * ceiling, (ms, tflops, ceiling)


def test_splitk_three_times_faster_than_no_split(gpu, beamc):
    """256 x 256 x 32768: the library's split-K choice against its best tile without a split (13x measured;
    the target is 3x)."""
    M, N, K = 256, 256, 32768
    a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), F16, 11, 0))
    b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), F16, 11, 1))
    c = beamc.DeviceArray((M, N))
    try:
        split = _best(lambda: beamc.bench(beamc.OP_SPLITK, a, b, c, config=None, split_k=0, warmup=20, iters=100))
        plain = min(_best(lambda cfg=cfg: beamc.bench(beamc.OP_GEMM, a, b, c, config=cfg, warmup=5, iters=20), 2)
                    for cfg in beamc.list_configs())
    finally:
        for t in (a, b, c):
            t.free()
    assert plain >= 3.0 * split, (plain, split)
    assert split <= 0.016, split  # ms; 12.5-14 us measured


def test_fused_layernorm_within_ten_percent_of_plain_gemm(gpu, beamc):
    """4096^3: GEMM+LayerNorm in one kernel against the plain GEMM of the same tile (+5.6-7.3% measured)."""
    M = N = K = 4096
    a = beamc.DeviceArray.from_numpy(beamc.host_normal((M, K), F16, 22, 0, 0.0, K ** -0.5))
    b = beamc.DeviceArray.from_numpy(beamc.host_normal((N, K), F16, 22, 1, 0.0, K ** -0.5))
    g = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, 22, 2, 1.0, 0.1))
    bt = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, 22, 3, 0.0, 0.1))
    c = beamc.DeviceArray((M, N))
    try:
        # both as the library runs them when left the choice (the 256 x 256 tile of four 128 x 128 wavefronts)
        # (the two in turn, best of five rounds each: +6-7% leaves little room for a lucky round of one against
        # an unlucky round of the other)
        plain, fused = 1e9, 1e9
        for _ in range(5):
            plain = min(plain, beamc.bench(beamc.OP_GEMM, a, b, c, warmup=50, iters=100))
            fused = min(fused, beamc.bench(beamc.OP_GEMM_LN, a, b, c, gamma=g, beta=bt, warmup=50, iters=100))
    finally:
        for t in (a, b, g, bt, c):
            t.free()
    assert fused <= 1.10 * plain, (plain, fused)


def test_kmajor_layout_keeps_up_with_gemmrc(gpu, beamc):
    """4096 x 8192 x 4096: matmul with B as [K][N] runs on the same 4-wavefront kernel as gemmrc (1-3% behind when
    healthy; 8-10% if the call falls back to the 8-wavefront tile).  The two in turn, best of four rounds each."""
    M, N, K = 4096, 8192, 4096
    a = beamc.DeviceArray.from_numpy(beamc.host_normal((M, K), F16, 9, 0, 0.0, K ** -0.5))
    bnk = beamc.DeviceArray.from_numpy(beamc.host_normal((N, K), F16, 9, 1, 0.0, K ** -0.5))
    bkn = beamc.DeviceArray.from_numpy(beamc.host_normal((K, N), F16, 9, 1, 0.0, K ** -0.5))
    c = beamc.DeviceArray((M, N))
    try:
        rc, nn = 1e9, 1e9
        for _ in range(4):
            rc = min(rc, beamc.bench(beamc.OP_GEMM, a, bnk, c, warmup=50, iters=100))
            nn = min(nn, beamc.bench(beamc.OP_MATMUL_NN, a, bkn, c, warmup=50, iters=100))
    finally:
        for t in (a, bnk, bkn, c):
            t.free()
    assert nn <= 1.06 * rc, (rc, nn)
