"""Re-entrancy: host threads on their own streams call the operators at the same time.

Four threads, each with its own stream, inputs, outputs and workspaces, loop over gemmrc, split-K, the
[K][N] matmul, GEMM+SiLU and the two-pass GEMM+LayerNorm (the fused one keeps per-workspace state and is
exercised with a private workspace per thread as well).  Every result must equal what the same call
gives on a quiet device, bit for bit.
"""
import ctypes
import threading

import pytest

pytestmark = pytest.mark.gpu

F16 = 0


def test_threads_on_private_streams(gpu, beamc):
    L, chk = beamc.lib, beamc._check
    M, N, K, n = 320, 384, 512, 30011
    nthreads, loops = 4, 12

    class Ctx:
        pass

    def make(seed):
        c = Ctx()
        c.a = beamc.DeviceArray.from_numpy(beamc.host_normal((M, K), F16, seed, 0, 0.0, K ** -0.5))
        c.b = beamc.DeviceArray.from_numpy(beamc.host_normal((N, K), F16, seed, 1, 0.0, K ** -0.5))
        c.bkn = beamc.DeviceArray.from_numpy(beamc.host_normal((K, N), F16, seed, 2, 0.0, K ** -0.5))
        c.x = beamc.DeviceArray.from_numpy(beamc.host_normal((n,), F16, seed, 3, 0.0, 2.0))
        c.g = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, seed, 4, 1.0, 0.1))
        c.bt = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, seed, 5, 0.0, 0.1))
        c.out = {k: beamc.DeviceArray((M, N), F16) for k in ("gemm", "splitk", "nn", "pair", "ln2", "lnf")}
        c.y = beamc.DeviceArray((n,), F16)
        c.cfg = beamc.TileConfig(64, 64, 32, 32, 0, 0).to_c()
        s = L.beam_splitk_effective(M, N, K, ctypes.byref(c.cfg), 4)
        c.ws_sk = beamc.DeviceArray((max(L.beam_splitk_workspace_bytes(M, N, s), 256),), F16, 1)
        c.ws_ln2 = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_ex(M, N, None, beamc.LN_TWOPASS),), F16, 1)
        c.ws_lnf = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_ex(M, N, None, beamc.LN_FUSED),), F16, 1)
        return c

    def calls(c, stream):
        chk(L.beam_gemmrc(c.a.ptr, c.b.ptr, c.out["gemm"].ptr, M, N, K, F16, None, stream))
        chk(L.beam_gemmrc_splitk(c.a.ptr, c.b.ptr, c.out["splitk"].ptr, M, N, K, F16, ctypes.byref(c.cfg), 4, c.ws_sk.ptr, c.ws_sk.nbytes, stream))
        chk(L.beam_matmul_nn(c.a.ptr, c.bkn.ptr, c.out["nn"].ptr, M, N, K, F16, None, stream))
        chk(L.beam_parallel_gemmrc_silu(c.a.ptr, c.b.ptr, c.out["pair"].ptr, M, N, K, c.x.ptr, c.y.ptr, n, F16, None, stream))
        chk(L.beam_gemmrc_ln_ex(c.a.ptr, c.b.ptr, c.g.ptr, c.bt.ptr, 1e-5, c.out["ln2"].ptr, M, N, K, F16, None, beamc.LN_TWOPASS,
                                c.ws_ln2.ptr, c.ws_ln2.nbytes, stream))
        chk(L.beam_gemmrc_ln_ex(c.a.ptr, c.b.ptr, c.g.ptr, c.bt.ptr, 1e-5, c.out["lnf"].ptr, M, N, K, F16, None, beamc.LN_FUSED,
                                c.ws_lnf.ptr, c.ws_lnf.nbytes, stream))

    def snapshot(c):
        return {k: v.to_numpy().copy() for k, v in list(c.out.items()) + [("y", c.y)]}

    ctxs = [make(100 + t) for t in range(nthreads)]
    want = []
    for c in ctxs:  # quiet device, default stream
        calls(c, None)
        want.append(snapshot(c))
        for v in list(c.out.values()) + [c.y]:
            v.fill_bytes(0xEE)
    errors = []

    def worker(t):
        try:
            stream = ctypes.c_void_p()
            chk(L.beam_stream_create(ctypes.byref(stream)))
            for _ in range(loops):
                calls(ctxs[t], stream)
            chk(L.beam_sync(stream))
            flag = ctypes.c_int(0)
            chk(L.beam_gemmrc_ln_timed_out(ctxs[t].ws_lnf.ptr, stream, ctypes.byref(flag)))
            if flag.value:
                errors.append(f"thread {t}: fused LayerNorm timed out")
            chk(L.beam_stream_destroy(stream))
        except Exception as e:  # noqa: BLE001
            errors.append(f"thread {t}: {e}")

    # The fused LayerNorm waits (bounded) for the other tiles of its band; these problems are far too
    # small to fill the device even four at a time, but keep the bound short so that a surprise shows
    # up as a reported time-out rather than as seconds of spinning.
    chk(L.beam_set_ln_spin_limit(1 << 16))
    try:
        threads = [threading.Thread(target=worker, args=(t,)) for t in range(nthreads)]
        for th in threads:
            th.start()
        for th in threads:
            th.join()
    finally:
        chk(L.beam_set_ln_spin_limit(4 << 20))
    assert not errors, errors
    for t, c in enumerate(ctxs):
        got = snapshot(c)
        for k in want[t]:
            assert (got[k] == want[t][k]).all(), f"thread {t}: {k} differs from the quiet-device result"
        for v in [c.a, c.b, c.bkn, c.x, c.g, c.bt, c.y, c.ws_sk, c.ws_ln2, c.ws_lnf] + list(c.out.values()):
            v.free()
