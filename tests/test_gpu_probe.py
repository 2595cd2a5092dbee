"""The register-only matrix-core loop (beam_probe_mfma): the ceiling the GEMM's throughput is read against."""
import pytest

pytestmark = pytest.mark.gpu


def test_mfma_ceiling_probe(gpu, beamc):
    """All-zero operands run at (nearly) the full clock: within a few percent of 256 CUs x 4 SIMDs x 1024 flop per
    cycle x 2.4 GHz, which also checks the probe's flop count.  Operands of the headline workload's distribution draw
    more power per cycle and run slower under the cap, the 32x32x16 shape slower still (which is why the kernels use
    16x16x32).  Short runs: these are sanity bounds, not the figures of the profiles."""
    rate = {}
    for name, dtype, shape, data in (("zeros", beamc.F16, beamc.MFMA_16X16X32, beamc.PROBE_ZEROS),
                                     ("normal", beamc.F16, beamc.MFMA_16X16X32, beamc.PROBE_NORMAL),
                                     ("normal32", beamc.F16, beamc.MFMA_32X32X16, beamc.PROBE_NORMAL),
                                     ("normal_bf16", beamc.BF16, beamc.MFMA_16X16X32, beamc.PROBE_NORMAL)):
        ms, tflops = beamc.probe_mfma(dtype, shape, data, passes=1600, warmup=100, iters=100)
        print(name, round(ms, 4), "ms", round(tflops, 1), "TFLOP/s", flush=True)
        rate[name] = tflops
    assert 2100.0 <= rate["zeros"] <= 2560.0, rate
    assert 1500.0 <= rate["normal"] <= rate["zeros"], rate
    assert 1200.0 <= rate["normal32"] <= rate["zeros"], rate
    assert 1500.0 <= rate["normal_bf16"] <= rate["zeros"], rate
