"""Fused GEMM + LayerNorm through the C ABI against the oracle: |Y_gpu - Y_ref| <= 2e-3 absolute,
Y_ref being the oracle's un-rounded fp32 result."""
import numpy as np
import pytest

from test_gpu_gemm import F16, BF16

pytestmark = pytest.mark.gpu

LN_TOL = 2e-3
# fp16: what is left of the error once the rounding of the output itself (half an ulp: at most |y| * 2^-11)
# is taken off, i.e. the error of the statistics and the normalisation
LN_OWN_TOL = 2e-4


def f16_error_beyond_rounding(got_bits, ref32):
    got = np.ascontiguousarray(got_bits, dtype=np.uint16).view(np.float16).astype(np.float64).ravel()
    ref = np.asarray(ref32, dtype=np.float64).ravel()
    return float((np.abs(got - ref) - np.abs(ref) * 2.0 ** -11).max())


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
        own = f16_error_beyond_rounding(got_bits, ref32)
        assert own <= LN_OWN_TOL, f"{what}: error beyond the output's rounding {own:.4g} > {LN_OWN_TOL}"
    else:
        assert r["max_bf16_excess"] <= LN_TOL, f"{what}: {r['max_bf16_excess']:.4g} > {LN_TOL}"


@pytest.mark.parametrize("shape", [(256, 512, 256), (1024, 1024, 512), (300, 1000, 200), (64, 4096, 128),
                                   (17, 40, 64), (16384, 2048, 128), (4200, 1000, 72), (300, 1000, 256), (700, 1304, 192)])
def test_ln_small(gpu, beamc, oracle, shape):
    M, N, K = shape
    for dtype in (F16, BF16):
        a, b, g, bt = make_ln_inputs(beamc, M, N, K, dtype, 21)
        ref = oracle.gemmrc_ln(a, b, g, bt, 1e-5, dtype)
        # (256 x 256 / 128 x 128 is the 4-wavefront kernel where K is a multiple of 64 from 192 on, the
        # 8-wavefront family's tile of that shape elsewhere)
        for cfg in [None, beamc.TileConfig(128, 128, 64, 64), beamc.TileConfig(64, 64, 32, 32),
                    beamc.TileConfig(256, 256, 128, 64), beamc.TileConfig(256, 256, 128, 128)]:
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
    """Spin limit -1 makes every wait of the fused kernel give up at once, whatever has been published: the
    kernel still ends normally, the flag is raised, the rows come out as NaN (not as plausible numbers), the
    checking form of the call raises -- and the next call with the normal budget is correct again with no
    reset in between."""
    M, N, K = 512, 4096, 256
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 26)
    good = run_ln(beamc, a, b, g_, bt, F16, mode=beamc.LN_FUSED)
    da, db = beamc.DeviceArray.from_numpy(a), beamc.DeviceArray.from_numpy(b)
    dg, dbt = beamc.DeviceArray.from_numpy(g_), beamc.DeviceArray.from_numpy(bt)
    y = beamc.DeviceArray((M, N))
    try:
        assert beamc.lib.beam_set_ln_spin_limit(-1) == 0
        beamc.gemmrc_ln(da, db, y, dg, dbt, mode=beamc.LN_FUSED, check=False)
        beamc.sync()
        assert beamc.gemmrc_ln_timed_out()
        assert np.isnan(y.to_numpy().view(np.float16)).all()
        with pytest.raises(beamc.BeamError):
            beamc.gemmrc_ln(da, db, y, dg, dbt, mode=beamc.LN_FUSED, check=True)
    finally:
        beamc.lib.beam_set_ln_spin_limit(beamc.DEFAULT_SPIN_LIMIT)
    beamc.gemmrc_ln(da, db, y, dg, dbt, mode=beamc.LN_FUSED, check=True)  # the flag was cleared by this call
    assert (y.to_numpy() == good).all()
    for x in (da, db, dg, dbt, y):
        x.free()


def test_default_call_recovers_from_a_forced_timeout(gpu, beamc, oracle):
    """The default Python call (LN_AUTO, checking) gives the right result even when the one-kernel form cannot
    finish its exchange: with the spin limit at -1 every wait gives up at once (every kernel still ends normally),
    the call notices, runs again as two passes and says so.  The C entry behind it (beam_gemmrc_ln_checked) reports
    the same through its flag; without the forced time-out neither falls back."""
    import ctypes
    M, N, K = 512, 4096, 256
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 27)
    ref = oracle.gemmrc_ln(a, b, g_, bt, 1e-5, F16)
    two_pass = run_ln(beamc, a, b, g_, bt, F16, mode=beamc.LN_TWOPASS)
    da, db = beamc.DeviceArray.from_numpy(a), beamc.DeviceArray.from_numpy(b)
    dg, dbt = beamc.DeviceArray.from_numpy(g_), beamc.DeviceArray.from_numpy(bt)
    y = beamc.DeviceArray((M, N))
    L = beamc.lib
    assert L.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, beamc.LN_AUTO) >= \
        max(L.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, m) for m in (beamc.LN_FUSED, beamc.LN_TWOPASS))
    ws = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, beamc.LN_AUTO),), itemsize=1)
    try:
        y.fill_bytes(0xEE)
        assert beamc.gemmrc_ln(da, db, y, dg, dbt) is False       # a quiet device: one kernel, no retry
        check_ln(oracle, y.to_numpy(), ref, F16, "default call")
        assert L.beam_set_ln_spin_limit(-1) == 0
        y.fill_bytes(0xEE)
        assert beamc.gemmrc_ln(da, db, y, dg, dbt) is True        # gave up, ran again as two passes
        got = y.to_numpy()
        check_ln(oracle, got, ref, F16, "default call with every wait forced to give up")
        assert (got == two_pass).all()
        y.fill_bytes(0xEE)
        fell_back = ctypes.c_int(0)
        rc = L.beam_gemmrc_ln_checked(da.ptr, db.ptr, dg.ptr, dbt.ptr, ctypes.c_float(1e-5), y.ptr, M, N, K, F16, None,
                                      ws.ptr, ws.nbytes, None, ctypes.byref(fell_back))
        assert rc == 0 and fell_back.value == 1, L.beam_last_error().decode()
        assert (y.to_numpy() == two_pass).all()
    finally:
        L.beam_set_ln_spin_limit(beamc.DEFAULT_SPIN_LIMIT)
    fell_back = ctypes.c_int(1)
    rc = L.beam_gemmrc_ln_checked(da.ptr, db.ptr, dg.ptr, dbt.ptr, ctypes.c_float(1e-5), y.ptr, M, N, K, F16, None,
                                  ws.ptr, ws.nbytes, None, ctypes.byref(fell_back))
    assert rc == 0 and fell_back.value == 0
    check_ln(oracle, y.to_numpy(), ref, F16, "checked call, normal budget")
    for x in (da, db, dg, dbt, y, ws):
        x.free()


def _ln_ex(beamc, da, db, dg, dbt, y, M, N, K, dtype, ws, mode):
    import ctypes
    rc = beamc.lib.beam_gemmrc_ln_ex(da.ptr, db.ptr, dg.ptr, dbt.ptr, ctypes.c_float(1e-5), y.ptr, M, N, K, dtype, None, mode,
                                     ws.ptr, ws.nbytes, None)
    assert rc == 0, beamc.lib.beam_last_error().decode()


def test_ln_fused_workspace_describes_itself(gpu, beamc, oracle):
    """The fused kernel's workspace needs no preparation and no reset: statistics words count only if they carry
    the tag of the launch that reads them.  A fresh buffer, one freed and handed out again, one overwritten
    with bytes that look like plausible statistics (0x3f...), one that holds the statistics of the previous
    launch on other data of the same shape, one used for another shape in between: all give the oracle's result."""
    M, N, K = 768, 2048, 256
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 31)
    ref = oracle.gemmrc_ln(a, b, g_, bt, 1e-5, F16)
    da, db = beamc.DeviceArray.from_numpy(a), beamc.DeviceArray.from_numpy(b)
    dg, dbt = beamc.DeviceArray.from_numpy(g_), beamc.DeviceArray.from_numpy(bt)
    y = beamc.DeviceArray((M, N))
    M2, N2 = 512, 1024  # the other shape that shares the buffer below
    need = max(beamc.lib.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, beamc.LN_FUSED),
               beamc.lib.beam_gemmrc_ln_workspace_bytes_for(M2, N2, K, None, beamc.LN_FUSED))
    assert need > 0

    def launch_and_check(ws, what):
        y.fill_bytes(0xEE)
        _ln_ex(beamc, da, db, dg, dbt, y, M, N, K, F16, ws, beamc.LN_FUSED)
        beamc.sync()
        check_ln(oracle, y.to_numpy(), ref, F16, what)

    ws = beamc.DeviceArray((need,), itemsize=1)
    launch_and_check(ws, "fresh workspace")
    launch_and_check(ws, "second launch on it")
    ws.free()
    ws = beamc.DeviceArray((need,), itemsize=1)  # usually the same address again
    ws.fill_bytes(0x3F)
    launch_and_check(ws, "re-allocated workspace full of 0x3f")
    launch_and_check(ws, "launch after that")
    # the same shape with other data: what the previous launch published must not pass for this launch's
    a3, b3, g3, bt3 = make_ln_inputs(beamc, M, N, K, F16, 33)
    ref3 = oracle.gemmrc_ln(a3, b3, g3, bt3, 1e-5, F16)
    da3, db3 = beamc.DeviceArray.from_numpy(a3), beamc.DeviceArray.from_numpy(b3)
    dg3, dbt3 = beamc.DeviceArray.from_numpy(g3), beamc.DeviceArray.from_numpy(bt3)
    for rep in range(3):
        y.fill_bytes(0xEE)
        _ln_ex(beamc, da3, db3, dg3, dbt3, y, M, N, K, F16, ws, beamc.LN_FUSED)
        beamc.sync()
        check_ln(oracle, y.to_numpy(), ref3, F16, f"other data, same shape, same workspace ({rep})")
        launch_and_check(ws, f"and the first data again ({rep})")
    for x in (da3, db3, dg3, dbt3):
        x.free()
    # another shape on the same buffer in between, then the first one again
    a2, b2, g2, bt2 = make_ln_inputs(beamc, M2, N2, K, F16, 32)
    ref2 = oracle.gemmrc_ln(a2, b2, g2, bt2, 1e-5, F16)
    da2, db2 = beamc.DeviceArray.from_numpy(a2), beamc.DeviceArray.from_numpy(b2)
    dg2, dbt2 = beamc.DeviceArray.from_numpy(g2), beamc.DeviceArray.from_numpy(bt2)
    y2 = beamc.DeviceArray((M2, N2))
    _ln_ex(beamc, da2, db2, dg2, dbt2, y2, M2, N2, K, F16, ws, beamc.LN_FUSED)
    beamc.sync()
    check_ln(oracle, y2.to_numpy(), ref2, F16, "other shape on the same workspace")
    launch_and_check(ws, "first shape again")
    for x in (da, db, dg, dbt, y, da2, db2, dg2, dbt2, y2, ws):
        x.free()


def test_two_fused_launches_share_the_device(gpu, beamc):
    """Two streams, each with fused launches that fill the device on their own (256 tiles each), issued in turn so
    that the two are in flight together: a band's workgroups have consecutive ids and are placed in id order, so a
    launch that holds only part of the device finishes band by band and nobody waits for a workgroup that cannot be
    placed.  Every result equals the one from a quiet device, and no launch gives up waiting.  (The wait is
    bounded in any case; the budget is lowered here so that a regression fails in seconds.)"""
    import ctypes
    L = beamc.lib
    M, N, K = 4096, 4096, 256
    streams = []
    for _ in range(2):
        s = ctypes.c_void_p()
        beamc._check(L.beam_stream_create(ctypes.byref(s)))
        streams.append(s)
    sets = []
    for i in range(2):
        a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 71 + i)
        d = [beamc.DeviceArray.from_numpy(x) for x in (a, b, g_, bt)]
        y = beamc.DeviceArray((M, N))
        ws = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, beamc.LN_FUSED),), itemsize=1)
        sets.append((d, y, ws))

    def launch(i, stream):
        (da, db, dg, dbt), y, ws = sets[i]
        rc = L.beam_gemmrc_ln_ex(da.ptr, db.ptr, dg.ptr, dbt.ptr, ctypes.c_float(1e-5), y.ptr, M, N, K, F16, None, beamc.LN_FUSED,
                                 ws.ptr, ws.nbytes, stream)
        assert rc == 0, L.beam_last_error().decode()

    want = []
    for i in range(2):
        launch(i, None)
        beamc.sync()
        want.append(sets[i][1].to_numpy().copy())
    beamc._check(L.beam_set_ln_spin_limit(500000))
    try:
        for rep in range(30):
            for i in range(2):
                sets[i][1].fill_bytes(0xEE)
            beamc.sync()
            for _ in range(4):
                for i in range(2):
                    launch(i, streams[i])
            for i in range(2):
                flag = ctypes.c_int(1)
                beamc._check(L.beam_gemmrc_ln_timed_out(sets[i][2].ptr, streams[i], ctypes.byref(flag)))
                assert flag.value == 0, f"stream {i} gave up waiting (repetition {rep})"
                assert (sets[i][1].to_numpy() == want[i]).all(), f"stream {i}, repetition {rep}"
    finally:
        beamc._check(L.beam_set_ln_spin_limit(beamc.DEFAULT_SPIN_LIMIT))
        for s in streams:
            beamc._check(L.beam_stream_destroy(s))
        for d, y, ws in sets:
            for t in d + [y, ws]:
                t.free()


@pytest.mark.parametrize("shape,dtype", [((8192, 8192, 256), F16), ((6144, 6144, 192), F16), ((5000, 7000, 320), F16),
                                         ((16500, 2048, 256), BF16), ((4100, 8192, 448), BF16), ((9000, 4352, 192), F16)])
def test_ln_walking_tiles_matches_one_tile_per_workgroup(gpu, beamc, oracle, shape, dtype):
    """More 256 x 256 tiles than CUs: one workgroup per CU walks its tiles (the next tile's operands arrive while the
    band's statistics are exchanged) and gives, bit for bit, what one workgroup per tile gives; the oracle agrees.
    The shapes cover the three workgroup orders (band blocks over all XCDs, whole bands per XCD, band after band),
    bands of 32 column tiles (the most the walking form takes), ragged edges in M and N, K of 3 to 7 tiles (the
    operand streams change tile inside a tile's first K tiles), and workgroups with 2, 3 and 5 tiles."""
    M, N, K = shape
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, dtype, 51)
    ref = oracle.gemmrc_ln(a, b, g_, bt, 1e-5, dtype)
    cfg = beamc.TileConfig(256, 256, 128, 128)
    L = beamc.lib
    try:
        assert L.beam_set_ln_walk(0) == 0
        one_each = run_ln(beamc, a, b, g_, bt, dtype, config=cfg, mode=beamc.LN_FUSED)
        assert L.beam_set_ln_walk(1) == 0
        for rep in range(3):
            walked = run_ln(beamc, a, b, g_, bt, dtype, config=cfg, mode=beamc.LN_FUSED)
            assert (walked == one_each).all(), f"{shape}: walking differs from one workgroup per tile (repetition {rep})"
    finally:
        L.beam_set_ln_walk(1)
    check_ln(oracle, walked, ref, dtype, f"{shape} dtype {dtype} walking")
    # and the call that names nothing (whatever tile and form the library takes for it)
    check_ln(oracle, run_ln(beamc, a, b, g_, bt, dtype), ref, dtype, f"{shape} dtype {dtype} default call")


def test_ln_default_call_never_lacks_workspace(gpu, beamc, oracle):
    """M=1024, N=8192, K=2048 without a tile: the library's tile for that K takes the two-pass path (32 column
    tiles of 256 fit the fused kernel, but the tile chosen is another); the Python wrapper sizes its buffer for
    exactly that call."""
    M, N, K = 1024, 8192, 2048
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 33)
    ref = oracle.gemmrc_ln(a, b, g_, bt, 1e-5, F16)
    got = run_ln(beamc, a, b, g_, bt, F16)
    check_ln(oracle, got, ref, F16, "default call 1024 x 8192 x 2048")


def test_walking_kernel_ends_when_every_wait_gives_up(gpu, beamc):
    """The walking form of the 4-wavefront kernel (1024 tiles on 256 workgroups) with the spin limit at -1: every
    wait of every tile gives up at once, the workgroups still walk all their tiles and end normally, every row is
    NaN and the record says so; the next call with the normal budget is right again, with no reset in between."""
    M, N, K = 8192, 8192, 256
    w4 = beamc.TileConfig(256, 256, 128, 128)
    a, b, g_, bt = make_ln_inputs(beamc, M, N, K, F16, 33)
    good = run_ln(beamc, a, b, g_, bt, F16, config=w4, mode=beamc.LN_FUSED)
    da, db = beamc.DeviceArray.from_numpy(a), beamc.DeviceArray.from_numpy(b)
    dg, dbt = beamc.DeviceArray.from_numpy(g_), beamc.DeviceArray.from_numpy(bt)
    y = beamc.DeviceArray((M, N))
    try:
        assert beamc.lib.beam_set_ln_spin_limit(-1) == 0
        beamc.gemmrc_ln(da, db, y, dg, dbt, config=w4, mode=beamc.LN_FUSED, check=False)
        beamc.sync()
        assert beamc.gemmrc_ln_timed_out()
        assert np.isnan(y.to_numpy().view(np.float16)).all()
    finally:
        beamc.lib.beam_set_ln_spin_limit(beamc.DEFAULT_SPIN_LIMIT)
    beamc.gemmrc_ln(da, db, y, dg, dbt, config=w4, mode=beamc.LN_FUSED, check=True)
    assert (y.to_numpy() == good).all()
    for x in (da, db, dg, dbt, y):
        x.free()
