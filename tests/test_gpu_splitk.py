"""Split-K gemmrc through the C ABI: parity with the oracle, determinism, S=1 identity."""
import numpy as np
import pytest

from test_gpu_gemm import F16, BF16, assert_close

pytestmark = pytest.mark.gpu


def run_splitk(beamc, a_bits, b_bits, dtype, tb, wp, s, pipeline=0):
    M, K = a_bits.shape
    N = b_bits.shape[0]
    a = beamc.DeviceArray.from_numpy(a_bits, dtype)
    b = beamc.DeviceArray.from_numpy(b_bits, dtype)
    c = beamc.DeviceArray((M, N), dtype)
    c.fill_bytes(0xEE)
    beamc.gemmrc_splitk_spec(a, b, c, shape_threadblock=tb, shape_warp=wp, split_k_slices=s, pipeline=pipeline)
    out = c.to_numpy()
    for x in (a, b, c):
        x.free()
    return out


# The tile list of the reference's split-K entry (cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:189-193), largest first.
# (256 x 128 is above what the one-launch form is built for: it runs as partial kernel + reduce kernel.)
TILES = [((256, 128), (64, 64)), ((128, 128), (64, 64)), ((128, 64), (64, 32)), ((64, 128), (32, 64)), ((64, 64), (32, 32))]


@pytest.mark.parametrize("shape", [(256, 256, 32768), (64, 128, 65536)])
def test_splitk_configs(gpu, beamc, oracle, shape):
    M, N, K = shape
    a = beamc.host_uniform((M, K), F16, 11, 0)
    b = beamc.host_uniform((N, K), F16, 11, 1)
    ref = oracle.gemmrc(a, b, F16)
    r = oracle.compare(oracle.from_f32(ref, F16), ref, F16)
    assert abs(r["rms_ref"] / (K ** 0.5 / 3.0) - 1.0) < 0.05      # RMS(C) = sqrt(K)/3 for uniform inputs
    assert r["max_abs_ref"] < 65504                                # inside fp16 range
    for tb, wp in TILES:
        for s in (4, 8, 16, 32, 64):
            for pipe in (0, 2):
                got = run_splitk(beamc, a, b, F16, tb, wp, s, pipe)
                assert_close(oracle, got, ref, K, F16, f"{tb} s={s} pipeline {pipe}")
    # the oracle's own slice-ordered sum agrees with its single-pass sum to fp32 reorder noise
    ref_s = oracle.gemmrc_splitk(a, b, 16, F16)
    assert np.abs(ref_s - ref).max() <= 1e-4 * r["rms_ref"]


def test_splitk_deterministic_and_s1_identity(gpu, beamc, oracle):
    M, N, K = 256, 256, 8192
    a = beamc.host_uniform((M, K), F16, 12, 0)
    b = beamc.host_uniform((N, K), F16, 12, 1)
    first = run_splitk(beamc, a, b, F16, (64, 64), (32, 32), 16)
    for _ in range(3):
        again = run_splitk(beamc, a, b, F16, (64, 64), (32, 32), 16)
        assert (again == first).all(), "split-K result changed from run to run"
    # one slice is the plain kernel, bit for bit
    s1 = run_splitk(beamc, a, b, F16, (64, 64), (32, 32), 1)
    da = beamc.DeviceArray.from_numpy(a)
    db = beamc.DeviceArray.from_numpy(b)
    dc = beamc.DeviceArray((M, N))
    beamc.gemmrc_spec(da, db, dc, shape_threadblock=[64, 64], shape_warp=[32, 32])
    assert (dc.to_numpy() == s1).all()


@pytest.mark.parametrize("shape,s", [((100, 72, 1000), 3), ((256, 256, 200), 64), ((33, 65, 4104), 7),
                                      ((512, 512, 8192), 0), ((512, 512, 8192), 15)])
def test_splitk_ragged_and_clamped(gpu, beamc, oracle, shape, s):
    """Ragged M, N, K tail inside a slice, more slices than K tiles (clamped), heuristic (0)."""
    M, N, K = shape
    for dtype in (F16, BF16):
        a = beamc.host_uniform((M, K), dtype, 13, 0)
        b = beamc.host_uniform((N, K), dtype, 13, 1)
        ref = oracle.gemmrc(a, b, dtype)
        for pipe in (0, 1, 2):
            got = run_splitk(beamc, a, b, dtype, (64, 64), (32, 32), s, pipe)
            assert_close(oracle, got, ref, K, dtype, f"{shape} s={s} pipeline {pipe}")


def test_splitk_workspace_errors(gpu, beamc):
    import ctypes
    a = beamc.DeviceArray((256, 4096))
    b = beamc.DeviceArray((256, 4096))
    c = beamc.DeviceArray((256, 256))
    cfg = beamc.TileConfig(64, 64, 32, 32).to_c()
    rc = beamc.lib.beam_gemmrc_splitk(a.ptr, b.ptr, c.ptr, 256, 256, 4096, 0, ctypes.byref(cfg), 8, None, 0, None)
    assert rc == 3
    assert b"workspace" in beamc.lib.beam_last_error()
    assert beamc.lib.beam_splitk_workspace_bytes(256, 256, 8) >= 8 * 256 * 256 * 4


def test_splitk_choice_is_logged_once_per_shape(gpu, beamc, capfd):
    """With the library choosing the slice count, a verbose library reports its choice once per shape
    (the reference's once-per-shape "[INFO] ... split_k(..), CTAs(..), waves(..)" line,
    cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:12-24,87-93), and a quiet one (the default) never."""
    M, N, K = 128, 192, 16384
    a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), F16, 3, 0), F16)
    b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), F16, 3, 1), F16)
    c = beamc.DeviceArray((M, N), F16)
    capfd.readouterr()
    beamc.gemmrc_splitk(a, b, c)
    assert "[beam]" not in capfd.readouterr().err
    assert beamc.lib.beam_set_verbose(1) == 0
    try:
        for _ in range(3):
            beamc.gemmrc_splitk(a, b, c)
        beamc.gemmrc_splitk(a, b, c, split_k_slices=4)   # a slice count the caller gave is not a decision
        err = capfd.readouterr().err
    finally:
        beamc.lib.beam_set_verbose(0)
    lines = [l for l in err.splitlines() if l.startswith("[beam] split-K")]
    assert len(lines) == 1, err
    s = beamc.lib.beam_splitk_effective(M, N, K, None, 0)
    assert f"[{M},{N},{K}]" in lines[0] and f"{s} slices" in lines[0] and "workgroups" in lines[0] and "rounds" in lines[0]
    for x in (a, b, c):
        x.free()
