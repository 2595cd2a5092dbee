"""The split-K entry point that allocates nothing (its workspace is device memory built into the library)
against beam_gemmrc_splitk with a caller-owned workspace: same bits, on two calls in a row, the second on a
smaller problem (the built-in array keeps the first call's contents), and a clear error beyond its size."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu

F16, BF16 = 0, 1


def _both(beamc, M, N, K, dtype, cfg, split, seed):
    L = beamc.lib
    a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), dtype, seed, 0), dtype)
    b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), dtype, seed, 1), dtype)
    want, got = beamc.DeviceArray((M, N), dtype), beamc.DeviceArray((M, N), dtype)
    want.fill_bytes(0xEE)
    got.fill_bytes(0xDD)
    cfgp = ctypes.byref(cfg) if cfg is not None else None
    s = L.beam_splitk_effective(M, N, K, cfgp, split)
    assert s >= 1
    ws = beamc.DeviceArray((max(L.beam_splitk_workspace_bytes(M, N, s), 256),), itemsize=1)
    rc = L.beam_gemmrc_splitk(a.ptr, b.ptr, want.ptr, M, N, K, dtype, cfgp, split, ws.ptr, ws.nbytes, None)
    assert rc == 0, L.beam_last_error().decode()
    rc = L.beam_gemmrc_splitk_noalloc(a.ptr, b.ptr, got.ptr, M, N, K, dtype, cfgp, split, None)
    assert rc == 0, L.beam_last_error().decode()
    beamc.sync()
    w, g = want.to_numpy(), got.to_numpy()
    for t in (a, b, want, got, ws):
        t.free()
    return w, g, s


def test_no_alloc_splitk_matches_workspace_entry_point(gpu, beamc):
    L = beamc.lib
    assert L.beam_splitk_noalloc_max_bytes() == 16 << 20
    cfg = beamc.TileConfig(64, 64, 32, 32, 2, 0).to_c()
    # the headline split-K shape, then a smaller one straight after it (stale partial sums of the first call
    # lie in the array), then the library's own choice of tile and slices, then bf16 and a ragged shape
    for (M, N, K, dtype, c, split, seed) in ((256, 256, 32768, F16, cfg, 16, 41), (64, 128, 8192, F16, cfg, 8, 42),
                                              (256, 256, 32768, F16, None, 0, 43), (200, 136, 4096, BF16, cfg, 7, 44)):
        want, got, s = _both(beamc, M, N, K, dtype, c, split, seed)
        assert s > 1
        assert (want == got).all(), (M, N, K, dtype, split)
        assert not (got == 0xDDDD).any()


def test_no_alloc_splitk_rejects_what_does_not_fit(gpu, beamc):
    L = beamc.lib
    M = N = 2048  # 64 slices x 2048 x 2048 x 4 bytes = 1 GiB
    cfg = beamc.TileConfig(64, 64, 32, 32, 2, 0).to_c()
    a, b, c = beamc.DeviceArray((M, 8192)), beamc.DeviceArray((N, 8192)), beamc.DeviceArray((M, N))
    c.fill_bytes(0xAB)
    rc = L.beam_gemmrc_splitk_noalloc(a.ptr, b.ptr, c.ptr, M, N, 8192, F16, ctypes.byref(cfg), 64, None)
    assert rc == 3 and b"built-in workspace" in L.beam_last_error()
    beamc.sync()
    assert (c.to_numpy() == 0xABAB).all()  # nothing was launched
    for t in (a, b, c):
        t.free()
