"""The harness that mirrors python/gemm_test.py (check / universal_test / test_gemm / split-K sweep),
with the CPU oracle as the answer function."""
import csv

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def oracle_answer(oracle, dtype):
    def ans(a, b, c):
        ref16 = oracle.gemmrc(a.to_numpy(), b.to_numpy(), dtype, want16=True)[1]
        tmp = type(c).from_numpy(ref16, dtype)
        from beam import _C
        _C._check(_C.lib.beam_memcpy_d2d(c.ptr, tmp.ptr, c.nbytes))
        tmp.free()
    return ans


def test_gemm_harness(gpu, beamc, oracle):
    from beam import harness
    info = harness.print_device_info()
    assert "gfx950" in info["name"]
    r = harness.test_gemm(1024, 768, 512, "fp16", ansfunc=oracle_answer(oracle, 0), verbose=False)
    assert len(r["custom"]) == 6 and all(t > 0 for t in r["custom"])
    r = harness.test_gemm(512, 512, 1024, "bf16", ansfunc=oracle_answer(oracle, 1), verbose=False)
    assert len(r["custom"]) == 4


def test_splitk_sweep_harness(gpu, beamc, oracle, tmp_path):
    from beam import harness
    path = tmp_path / "splitk.csv"
    r = harness.test_gemm_splitk(512, 512, 8192, "fp16", csv_path=str(path), ansfunc=oracle_answer(oracle, 0),
                                 verbose=False)
    assert len(r["custom"]) == 15          # split_k_slices = 1..15 as in python/gemm_test.py:121-136
    rows = list(csv.reader(open(path)))
    assert rows[0] == ["split_k_slices", "TFLOPS", "max_err_over_rms"] and len(rows) == 16
    assert max(r["custom"][3:]) > r["custom"][0]    # splitting pays at 512x512x8192


def test_check_rejects_wrong_output(gpu, beamc):
    from beam import harness
    out = beamc.DeviceArray.from_numpy(np.ones((8, 8), np.float16).view(np.uint16))
    with pytest.raises(harness.CheckFailed):
        harness.check(lambda: None, [np.full((8, 8), 2.0, np.float32)], [out], K=64)
    with pytest.raises(harness.CheckFailed):
        harness.check(lambda: None, [np.ones((8, 4), np.float32)], [out], K=64)
    harness.check(lambda: None, [np.ones((8, 8), np.float32)], [out], K=64)
