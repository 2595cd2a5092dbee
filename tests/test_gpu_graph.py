"""A captured sequence of operators replays as a HIP graph with the eager results.

The graph holds gemmrc, split-K (one launch: multiplying and reducing workgroups in one grid; with a caller's
workspace and with the library's built-in one), GEMM+SiLU, the [K][N] matmul, a K = 0 call (its clear is a
kernel, not a memset node), a two-pass GEMM+LayerNorm (what BEAM_LN_AUTO turns into under capture) and an
explicitly fused one (its workspace keeps its launch count on the device, so replays and the eager calls in
between simply take turns on it).
It is replayed several times with the inputs changed and eager work of the library in between; every
replay must reproduce, bit for bit, what the same calls give eagerly on the same inputs.
"""
import ctypes

import pytest

pytestmark = pytest.mark.gpu

F16 = 0


def test_graph_replay_matches_eager(gpu, beamc):
    L, chk = beamc.lib, beamc._check
    M, N, K, n = 384, 320, 512, 70001
    rng_seed = [0]

    def fresh(shape, scale):
        rng_seed[0] += 1
        return beamc.host_normal(shape, F16, 99, rng_seed[0], 0.0, scale)

    a, b, bkn, x = (beamc.DeviceArray(s, F16) for s in ((M, K), (N, K), (K, N), (n,)))
    g = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, 99, 1000, 1.0, 0.1), F16)
    bt = beamc.DeviceArray.from_numpy(beamc.host_normal((N,), F16, 99, 1001, 0.0, 0.1), F16)
    outs = {k: beamc.DeviceArray((M, N), F16) for k in ("gemm", "splitk", "splitk_na", "pair", "nn", "k0", "ln", "lnf")}
    y = beamc.DeviceArray((n,), F16)
    cfg = beamc.TileConfig(64, 64, 32, 32, 0, 0).to_c()
    s_eff = L.beam_splitk_effective(M, N, K, ctypes.byref(cfg), 4)
    ws_sk = beamc.DeviceArray((max(L.beam_splitk_workspace_bytes(M, N, s_eff), 256),), F16, 1)
    ws_ln = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_ex(M, N, None, beamc.LN_TWOPASS),), F16, 1)
    ws_lnf = beamc.DeviceArray((L.beam_gemmrc_ln_workspace_bytes_ex(M, N, None, beamc.LN_FUSED),), F16, 1)

    def upload():
        for d, shape, scale in ((a, (M, K), K ** -0.5), (b, (N, K), K ** -0.5), (bkn, (K, N), K ** -0.5), (x, (n,), 2.0)):
            h = fresh(shape, scale)
            chk(L.beam_memcpy_h2d(d.ptr, h.ctypes.data, h.nbytes))

    def sequence(stream):
        chk(L.beam_gemmrc(a.ptr, b.ptr, outs["gemm"].ptr, M, N, K, F16, None, stream))
        chk(L.beam_gemmrc_splitk(a.ptr, b.ptr, outs["splitk"].ptr, M, N, K, F16, ctypes.byref(cfg), 4, ws_sk.ptr, ws_sk.nbytes, stream))
        # (the entry point made for code under capture: its workspace is the library's own device array)
        chk(L.beam_gemmrc_splitk_noalloc(a.ptr, b.ptr, outs["splitk_na"].ptr, M, N, K, F16, ctypes.byref(cfg), 8, stream))
        chk(L.beam_parallel_gemmrc_silu(a.ptr, b.ptr, outs["pair"].ptr, M, N, K, x.ptr, y.ptr, n, F16, None, stream))
        chk(L.beam_matmul_nn(a.ptr, bkn.ptr, outs["nn"].ptr, M, N, K, F16, None, stream))
        chk(L.beam_gemmrc(a.ptr, b.ptr, outs["k0"].ptr, M, N, 0, F16, None, stream))
        chk(L.beam_gemmrc_ln_ex(a.ptr, b.ptr, g.ptr, bt.ptr, 1e-5, outs["ln"].ptr, M, N, K, F16, None, beamc.LN_AUTO if stream else beamc.LN_TWOPASS,
                                ws_ln.ptr, ws_ln.nbytes, stream))
        chk(L.beam_gemmrc_ln_ex(a.ptr, b.ptr, g.ptr, bt.ptr, 1e-5, outs["lnf"].ptr, M, N, K, F16, None, beamc.LN_FUSED,
                                ws_lnf.ptr, ws_lnf.nbytes, stream))

    def snapshot():
        return {k: v.to_numpy().copy() for k, v in list(outs.items()) + [("y", y)]}

    def poison():
        for v in list(outs.values()) + [y]:
            v.fill_bytes(0xEE)

    stream = ctypes.c_void_p()
    chk(L.beam_stream_create(ctypes.byref(stream)))
    upload()
    sequence(None)  # eager warm-up: configures every kernel before anything is captured
    chk(L.beam_sync(None))
    chk(L.beam_graph_begin_capture(stream))
    sequence(stream)
    graph = ctypes.c_void_p()
    chk(L.beam_graph_end_capture(stream, ctypes.byref(graph)))
    try:
        for replay in range(4):
            upload()
            poison()
            sequence(None)
            want = snapshot()
            assert (want["k0"] == 0).all()
            poison()
            chk(L.beam_graph_launch(graph, stream))
            chk(L.beam_sync(stream))
            got = snapshot()
            for k in want:
                assert (got[k] == want[k]).all(), f"replay {replay}: {k} differs from the eager result"
            timed_out = ctypes.c_int(1)
            chk(L.beam_gemmrc_ln_timed_out(ws_lnf.ptr, stream, ctypes.byref(timed_out)))
            assert timed_out.value == 0
            # a second replay right behind the first, on new data: what the first replay left in the workspaces
            # (the fused LayerNorm's statistics among it) must not pass for the second one's
            upload()
            poison()
            chk(L.beam_graph_launch(graph, stream))
            chk(L.beam_sync(stream))
            got = snapshot()
            poison()
            sequence(None)
            want = snapshot()
            for k in want:
                assert (got[k] == want[k]).all(), f"replay {replay}, second in a row: {k} differs from the eager result"
        # A reset of the fused LayerNorm's workspace between two replays (what a caller does after a time-out) forgets
        # the recorded launch but not the replay counter: the replay behind it still gets a tag of its own, and the
        # statistics the replay before it left in the workspace do not pass for its own.
        chk(L.beam_gemmrc_ln_workspace_reset(ws_lnf.ptr))
        upload()
        poison()
        chk(L.beam_graph_launch(graph, stream))
        chk(L.beam_sync(stream))
        got = snapshot()
        poison()
        sequence(None)
        want = snapshot()
        for k in want:
            assert (got[k] == want[k]).all(), f"replay after a workspace reset: {k} differs from the eager result"
    finally:
        chk(L.beam_graph_destroy(graph))
        chk(L.beam_stream_destroy(stream))
        for t in [a, b, bkn, x, g, bt, y, ws_sk, ws_ln, ws_lnf] + list(outs.values()):
            t.free()
