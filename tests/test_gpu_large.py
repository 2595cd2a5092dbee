"""Outputs and workspaces beyond 4 GiB: every byte offset the kernels form has to be 64-bit, or inside a buffer
descriptor whose base is.  The operands are chosen so that the exact result at (m, n) is known in closed form and
differs from its neighbours: an offset that wrapped at 2^32 would put a value where another belongs."""
import ctypes

import numpy as np
import pytest

from test_gpu_gemm import F16

pytestmark = pytest.mark.gpu


def _rows_to_check(M, N, itemsize):
    """Row ranges: the first and the last rows, the rows around every multiple of 4 GiB, every 97th row between."""
    rows = set(range(0, 300)) | set(range(M - 300, M)) | set(range(0, M, 97))
    step = (1 << 32) // (N * itemsize)
    for k in range(1, M * N * itemsize // (1 << 32) + 1):
        rows |= set(range(max(0, k * step - 150), min(M, k * step + 150)))
    return sorted(rows)


def _download_rows(beamc, dev, rows, N):
    out = np.empty((len(rows), N), np.uint16)
    beamc.sync()
    # runs of consecutive rows, one copy each
    start = 0
    while start < len(rows):
        end = start
        while end + 1 < len(rows) and rows[end + 1] == rows[end] + 1:
            end += 1
        n = end - start + 1
        beamc._check(beamc.lib.beam_memcpy_d2h(out[start:].ctypes.data, dev.ptr + rows[start] * N * 2, n * N * 2))
        start = end + 1
    return out


def test_output_beyond_4_gib(gpu, beamc):
    """C = 49152 x 49152 fp16 (4.5 GiB), K = 256.  Row m of A is the unit vector e_(m % 256) and
    B[n][k] = ((7 n + 13 k) % 2048) - 1024, so C[m][n] = ((7 n + 13 (m % 256)) % 2048) - 1024 exactly.  The default
    call (the 4-wavefront kernel walking 144 tiles per CU) and two 8-wavefront tiles (one walking its tiles, one
    with a workgroup per tile)."""
    M = N = 49152
    K = 256
    a = np.zeros((M, K), np.float16)
    a[np.arange(M), np.arange(M) % K] = 1.0
    n_idx, k_idx = np.arange(N, dtype=np.int64)[:, None], np.arange(K, dtype=np.int64)[None, :]
    b = (((7 * n_idx + 13 * k_idx) % 2048) - 1024).astype(np.float16)
    da, db = beamc.DeviceArray.from_numpy(a.view(np.uint16)), beamc.DeviceArray.from_numpy(b.view(np.uint16))
    dc = beamc.DeviceArray((M, N))
    assert dc.nbytes > (1 << 32)
    rows = _rows_to_check(M, N, 2)
    m_idx = np.asarray(rows, dtype=np.int64)[:, None]
    want = (((7 * np.arange(N, dtype=np.int64)[None, :] + 13 * (m_idx % K)) % 2048) - 1024).astype(np.float16).view(np.uint16)
    try:
        for cfg in (None, beamc.TileConfig(256, 256, 128, 64), beamc.TileConfig(128, 128, 64, 64)):
            dc.fill_bytes(0xEE)
            print("49152 x 49152 x 256 with", cfg.name if cfg else "the default tile", flush=True)
            beamc.gemmrc(da, db, dc, config=cfg)
            got = _download_rows(beamc, dc, rows, N)
            bad = np.argwhere(got != want)
            assert bad.size == 0, (cfg.name if cfg else "default", rows[bad[0][0]], int(bad[0][1]), len(bad))
    finally:
        for t in (da, db, dc):
            t.free()


def test_two_pass_layernorm_workspace_beyond_4_gib(gpu, beamc):
    """Two-pass GEMM+LayerNorm with an fp32 X of 32768 x 36864 (4.5 GiB) in the workspace.  A[m][:] = (m % 512) / 64
    and B = 1 with K = 64 make row m of X the constant m % 512 (exact in fp32), so every row's variance is 0 and
    Y = beta exactly -- unless a part of some row of X was read from, or written to, another row's place."""
    M, N, K = 32768, 36864, 64
    a = np.repeat(((np.arange(M) % 512) / 64.0).astype(np.float16)[:, None], K, axis=1)
    b = np.ones((N, K), np.float16)
    gamma = beamc.host_normal((N,), F16, 41, 2, 1.0, 0.1)
    beta = beamc.host_normal((N,), F16, 41, 3, 0.0, 0.1)
    L = beamc.lib
    need = L.beam_gemmrc_ln_workspace_bytes_for(M, N, K, None, beamc.LN_TWOPASS)
    assert need > (1 << 32)
    da, db = beamc.DeviceArray.from_numpy(a.view(np.uint16)), beamc.DeviceArray.from_numpy(b.view(np.uint16))
    dg, dbt = beamc.DeviceArray.from_numpy(gamma), beamc.DeviceArray.from_numpy(beta)
    y = beamc.DeviceArray((M, N))
    ws = beamc.DeviceArray((need,), itemsize=1)
    try:
        y.fill_bytes(0xEE)
        ws.fill_bytes(0x3F)
        rc = L.beam_gemmrc_ln_ex(da.ptr, db.ptr, dg.ptr, dbt.ptr, ctypes.c_float(1e-5), y.ptr, M, N, K, F16, None,
                                 beamc.LN_TWOPASS, ws.ptr, ws.nbytes, None)
        assert rc == 0, L.beam_last_error().decode()
        rows = _rows_to_check(M, N, 4)  # multiples of 4 GiB in X (fp32) ...
        rows = sorted(set(rows) | set(_rows_to_check(M, N, 2)))  # ... and in Y
        got = _download_rows(beamc, y, rows, N)
        bad = np.argwhere(got != beta[None, :])
        assert bad.size == 0, (rows[bad[0][0]], int(bad[0][1]), len(bad))
        # the fp32 X itself: row m holds m % 512
        x_rows = [0, 1, 511, 512, 29127, 29128, 29129, M - 1]   # 29127.1 rows of X are 4 GiB
        for m in x_rows:
            row = np.empty((N,), np.float32)
            beamc._check(L.beam_memcpy_d2h(row.ctypes.data, ws.ptr + m * N * 4, N * 4))
            assert (row == float(m % 512)).all(), m
    finally:
        for t in (da, db, dg, dbt, y, ws):
            t.free()
