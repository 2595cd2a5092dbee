"""Split-K in one launch (reducing workgroups in the same grid as the multiplying ones) against the two-launch
form (partial kernel, reduce kernel): same bits on every tile the form is built for, on one workspace that is
never cleared between shapes; the fallbacks; the bounded wait forced to give up from the host."""
import ctypes

import numpy as np
import pytest

from test_gpu_gemm import F16, BF16, assert_close

pytestmark = pytest.mark.gpu

SMALL_TILES = [(128, 128, 64, 64), (128, 128, 64, 32), (128, 64, 64, 32), (64, 128, 32, 64), (64, 64, 32, 32)]


def _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, two_launches):
    L = beamc.lib
    assert L.beam_set_splitk_two_launches(1 if two_launches else 0) == 0
    try:
        c.fill_bytes(0xEE)
        cfgp = ctypes.byref(cfg) if cfg is not None else None
        rc = L.beam_gemmrc_splitk(a.ptr, b.ptr, c.ptr, M, N, K, dtype, cfgp, split, ws.ptr, ws.nbytes, None)
        assert rc == 0, L.beam_last_error().decode()
        beamc.sync()
        return c.to_numpy().copy()
    finally:
        L.beam_set_splitk_two_launches(0)


def test_one_launch_equals_two_launches(gpu, beamc):
    """Every small tile x LDS depth on shapes with one and with several rounds of workgroups, ragged M and N,
    a K tail, both dtypes; the workspace starts as 0x3F bytes and is shared by all cases without clearing."""
    L = beamc.lib
    ws = beamc.DeviceArray((64 << 20,), itemsize=1)
    ws.fill_bytes(0x3F)
    cases = [(256, 256, 32768, F16, 32), (256, 256, 32768, F16, 16), (64, 128, 65536, F16, 64), (512, 512, 8192, F16, 16),
             (200, 136, 4104, BF16, 7), (100, 260, 2048, F16, 5), (33, 68, 4096, BF16, 3), (1024, 256, 4096, F16, 4),
             (65, 64, 4096, F16, 8)]  # (a sliver of a second 128-row tile: as many flags as a whole one)
    seed = 50
    for (M, N, K, dtype, split) in cases:
        seed += 1
        a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), dtype, seed, 0), dtype)
        b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), dtype, seed, 1), dtype)
        c = beamc.DeviceArray((M, N), dtype)
        for (bm, bn, tm, tn) in SMALL_TILES:
            for pipe in (0, 2):
                cfg = beamc.TileConfig(bm, bn, tm, tn, pipe, 0).to_c()
                s = L.beam_splitk_effective(M, N, K, ctypes.byref(cfg), split)
                assert s > 1 and L.beam_splitk_workspace_bytes(M, N, s) <= ws.nbytes
                two = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, True)
                for _ in range(2):  # twice: the second call finds the first one's flags cleared
                    one = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, False)
                    assert (one == two).all(), (M, N, K, dtype, split, bm, bn, tm, tn, pipe)
                assert not (one == 0xEEEE).any()
                flag = ctypes.c_int(1)
                assert L.beam_gemmrc_splitk_timed_out(ws.ptr, ws.nbytes, M, N, s, None, ctypes.byref(flag)) == 0 and flag.value == 0
        for t in (a, b, c):
            t.free()
    ws.free()


def test_self_reducing_workgroups_give_the_same_bits(gpu, beamc):
    """The measurement form without reducing workgroups (every multiplying workgroup adds its share of its tile):
    the same bits as two launches, where the slices outnumber the parts of a tile, equal them and are fewer; twice in
    a row on one never-cleared workspace; no time-out."""
    L = beamc.lib
    ws = beamc.DeviceArray((64 << 20,), itemsize=1)
    ws.fill_bytes(0x5C)
    cases = [(256, 256, 32768, F16, 32, (64, 128, 32, 64), 2), (256, 256, 32768, F16, 16, (64, 64, 32, 32), 2),
             (64, 128, 65536, F16, 64, (64, 64, 32, 32), 0), (128, 128, 8192, BF16, 4, (64, 64, 32, 32), 0),
             (200, 136, 4104, BF16, 7, (64, 128, 32, 64), 2), (256, 256, 8192, F16, 3, (128, 128, 64, 64), 0)]
    assert L.beam_dbg_set_splitk_self_reduce(1) == 0
    try:
        for seed, (M, N, K, dtype, split, tile, pipe) in enumerate(cases):
            a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), dtype, 90 + seed, 0), dtype)
            b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), dtype, 90 + seed, 1), dtype)
            c = beamc.DeviceArray((M, N), dtype)
            cfg = beamc.TileConfig(*tile, pipe, 0).to_c()
            s = L.beam_splitk_effective(M, N, K, ctypes.byref(cfg), split)
            assert s > 1
            two = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, True)
            for _ in range(2):
                one = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, False)
                assert (one == two).all(), (M, N, K, dtype, split, tile, pipe)
            flag = ctypes.c_int(1)
            assert L.beam_gemmrc_splitk_timed_out(ws.ptr, ws.nbytes, M, N, s, None, ctypes.byref(flag)) == 0 and flag.value == 0
            for t in (a, b, c):
                t.free()
    finally:
        L.beam_dbg_set_splitk_self_reduce(0)
        ws.free()


def test_random_shapes_tiles_and_slice_counts(gpu, beamc):
    """80 seeded random problems (ragged M, N a multiple of 4, K a multiple of 8 with tails inside slices), random
    small tile, LDS depth and slice count, both dtypes, one never-cleared workspace: the two forms agree bit for bit."""
    L = beamc.lib
    rng = np.random.default_rng(20240607)
    ws = beamc.DeviceArray((96 << 20,), itemsize=1)
    ws.fill_bytes(0xA5)
    done = 0
    while done < 80:
        M = int(rng.integers(1, 700))
        N = 4 * int(rng.integers(1, 176))
        K = 8 * int(rng.integers(16, 1200))
        dtype = F16 if rng.random() < 0.6 else BF16
        bm, bn, tm, tn = SMALL_TILES[int(rng.integers(0, len(SMALL_TILES)))]
        pipe = int(rng.choice([0, 1, 2]))
        split = int(rng.choice([0, 2, 3, 5, 8, 13, 16, 32, 64]))
        cfg = beamc.TileConfig(bm, bn, tm, tn, pipe, 0).to_c()
        s = L.beam_splitk_effective(M, N, K, ctypes.byref(cfg), split)
        if s <= 1 or L.beam_splitk_workspace_bytes(M, N, s) > ws.nbytes:
            continue
        a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), dtype, 900 + done, 0), dtype)
        b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), dtype, 900 + done, 1), dtype)
        c = beamc.DeviceArray((M, N), dtype)
        two = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, True)
        one = _call(beamc, a, b, c, M, N, K, dtype, cfg, split, ws, False)
        assert (one == two).all(), (M, N, K, dtype, (bm, bn, tm, tn), pipe, split, s)
        for t in (a, b, c):
            t.free()
        done += 1
    ws.free()


def test_new_data_on_a_used_workspace(gpu, beamc):
    """Call after call on one workspace with different operands: nothing a reducing workgroup reads (partial sums
    of the previous call at the same addresses, in whatever cache) may be the previous call's."""
    L = beamc.lib
    M, N, K = 256, 256, 32768
    a, b, c = beamc.DeviceArray((M, K)), beamc.DeviceArray((N, K)), beamc.DeviceArray((M, N))
    s = L.beam_splitk_effective(M, N, K, None, 0)
    ws = beamc.DeviceArray((L.beam_splitk_workspace_bytes(M, N, s),), itemsize=1)
    ws2 = beamc.DeviceArray((L.beam_splitk_workspace_bytes(M, N, s),), itemsize=1)
    for seed in range(80, 86):
        ha, hb = beamc.host_uniform((M, K), F16, seed, 0), beamc.host_uniform((N, K), F16, seed, 1)
        beamc._check(L.beam_memcpy_h2d(a.ptr, ha.ctypes.data, ha.nbytes))
        beamc._check(L.beam_memcpy_h2d(b.ptr, hb.ctypes.data, hb.nbytes))
        one = _call(beamc, a, b, c, M, N, K, F16, None, 0, ws, False)
        two = _call(beamc, a, b, c, M, N, K, F16, None, 0, ws2, True)
        assert (one == two).all(), seed
    for t in (a, b, c, ws, ws2):
        t.free()


def test_fallbacks_to_two_launches(gpu, beamc, oracle):
    """A workspace that holds the partial sums only, N that is not a multiple of 4, a tile above 128 x 128:
    two launches, same contract."""
    L = beamc.lib
    cfg = beamc.TileConfig(64, 64, 32, 32, 2, 0).to_c()
    for (M, N, K, tile) in ((256, 256, 8192, cfg), (96, 70, 4096, cfg), (512, 512, 4096, beamc.TileConfig(256, 128, 64, 64, 0, 0).to_c())):
        a_bits = beamc.host_uniform((M, K), F16, 61, 0)
        b_bits = beamc.host_uniform((N, K), F16, 61, 1)
        a, b = beamc.DeviceArray.from_numpy(a_bits), beamc.DeviceArray.from_numpy(b_bits)
        c = beamc.DeviceArray((M, N))
        s = L.beam_splitk_effective(M, N, K, ctypes.byref(tile), 8)
        ws = beamc.DeviceArray((s * M * N * 4,), itemsize=1)  # no room for synchronisation words
        ws.fill_bytes(0x3F)
        got = _call(beamc, a, b, c, M, N, K, F16, tile, 8, ws, False)
        assert_close(oracle, got, oracle.gemmrc(a_bits, b_bits, F16), K, F16, f"{M}x{N}x{K}")
        for t in (a, b, c, ws):
            t.free()


def test_bounded_wait_gives_up_visibly(gpu, beamc):
    """The reducing workgroups' wait forced to give up from the host (spin limit -1: no poll is ever made):
    every kernel still ends, the outputs are NaN, the query says so and the checking Python call raises; the
    next call on the same workspace is clean."""
    L = beamc.lib
    M, N, K = 256, 256, 8192
    a = beamc.DeviceArray.from_numpy(beamc.host_uniform((M, K), F16, 71, 0))
    b = beamc.DeviceArray.from_numpy(beamc.host_uniform((N, K), F16, 71, 1))
    c = beamc.DeviceArray((M, N))
    cfg = beamc.TileConfig(64, 64, 32, 32, 2, 0).to_c()
    s = L.beam_splitk_effective(M, N, K, ctypes.byref(cfg), 16)
    ws = beamc.DeviceArray((L.beam_splitk_workspace_bytes(M, N, s),), itemsize=1)
    good = _call(beamc, a, b, c, M, N, K, F16, cfg, 16, ws, False)
    assert L.beam_set_ln_spin_limit(-1) == 0
    try:
        bad = _call(beamc, a, b, c, M, N, K, F16, cfg, 16, ws, False)
        flag = ctypes.c_int(0)
        assert L.beam_gemmrc_splitk_timed_out(ws.ptr, ws.nbytes, M, N, s, None, ctypes.byref(flag)) == 0 and flag.value == 1
        assert np.isnan(bad.view(np.float16)).all()
        with pytest.raises(beamc.BeamError):
            beamc.gemmrc_splitk_spec(a, b, c, shape_threadblock=(64, 64), shape_warp=(32, 32), split_k_slices=16,
                                     pipeline=2, check=True)
    finally:
        assert L.beam_set_ln_spin_limit(4 << 20) == 0
    again = _call(beamc, a, b, c, M, N, K, F16, cfg, 16, ws, False)
    assert (again == good).all()
    flag = ctypes.c_int(1)
    assert L.beam_gemmrc_splitk_timed_out(ws.ptr, ws.nbytes, M, N, s, None, ctypes.byref(flag)) == 0 and flag.value == 0
    beamc.gemmrc_splitk_spec(a, b, c, shape_threadblock=(64, 64), shape_warp=(32, 32), split_k_slices=16, pipeline=2, check=True)
    for t in (a, b, c, ws):
        t.free()
