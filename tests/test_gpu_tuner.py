"""The autotuner on the GPU with its whole candidate space: the winner is at least as good as the library's
default (within timing noise), and a candidate that does not produce the answer cannot win."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (4096, 4096, 1024), (256, 256, 8192)])
def test_tuned_pick_is_not_slower_than_default(gpu, beamc, shape):
    from beam import tuner
    t = tuner.OperatorTuner(warmup=3, rep=10)
    assert len(t.gemm_ops) > 150  # tiles x pipeline depths x raster groups + split-K tiles x depths x factors
    op, tf = t.tune(shape)
    assert op is not None and tf > 0
    M, N, K = shape
    a, b, c = t._make_inputs(M, N, K, beamc.F16)
    default = t.gemm_ops[0]
    assert str(default) == "gemmrc"
    best_default = max(default.get_performance(a, b, c, warmup=20, rep=50) for _ in range(3))
    best_tuned = max(op.get_performance(a, b, c, warmup=20, rep=50) for _ in range(3))
    for x in (a, b, c):
        x.free()
    assert best_tuned >= 0.97 * best_default, (str(op), best_tuned, best_default)


def test_a_candidate_that_writes_nothing_is_discarded(gpu, beamc):
    """It takes as long as a real kernel (it runs one, into a buffer of its own) and is the fastest candidate
    offered, but the output it was asked for keeps its fill pattern: the tuner must not pick it."""
    from beam import tuner
    M, N, K = 4096, 4096, 2048  # large enough for the kernels, not the Python calls, to set the times
    elsewhere = beamc.DeviceArray((M, N))

    def writes_nothing(a, b, c):
        beamc.gemmrc_spec(a, b, elsewhere, shape_threadblock=[128, 128], shape_warp=[64, 64])

    t = tuner.OperatorTuner(warmup=2, rep=5)
    honest = tuner.Operator(lambda a, b, c: beamc.gemmrc_spec(a, b, c, shape_threadblock=[64, 64], shape_warp=[32, 32]),
                            name="honest_but_slow")
    cheat = tuner.Operator(writes_nothing, name="writes_nothing")
    a, b, c = t._make_inputs(M, N, K, beamc.F16)
    assert cheat.get_performance(a, b, c) > honest.get_performance(a, b, c) > 0  # it would win on speed alone
    for x in (a, b, c):
        x.free()
    op, tf = t.tune((M, N, K), ops=[cheat, honest])
    assert str(op) == "honest_but_slow" and tf > 0
    elsewhere.free()
