"""Operator / OperatorTuner contract (reference: python/beam/tuner.py:19-137) with fake operators:
no GPU, no kernels."""
import json

import pytest


class FakeArray:
    def __init__(self, shape):
        self.shape = shape


@pytest.fixture()
def tuner_mod(beamc, monkeypatch):
    from beam import tuner
    monkeypatch.setattr(tuner._C, "sync", lambda: None)
    monkeypatch.setattr(tuner._C, "_describe", lambda x: (0, x.shape, 0, None))
    return tuner


def named(name, fn):
    fn.__name__ = name
    return fn


def test_operator_name_and_failure(tuner_mod):
    Operator = tuner_mod.Operator
    ok = Operator(named("fine", lambda a, b, c: None))
    assert str(ok) == "fine"
    assert str(Operator(lambda a, b, c: None)) == "<lambda>"

    def boom(a, b, c):
        raise RuntimeError("unsupported tile")
    bad = Operator(named("boom", boom))
    a, b, c = FakeArray((64, 32)), FakeArray((16, 32)), FakeArray((64, 16))
    assert ok.check_callable(a, b, c) is True
    assert bad.check_callable(a, b, c) is False
    assert bad.get_performance(a, b, c) == -1            # a failing call is -1, never an exception


def test_operator_performance_formula(tuner_mod, monkeypatch):
    Operator = tuner_mod.Operator
    a, b, c = FakeArray((4096, 2048)), FakeArray((1024, 2048)), FakeArray((4096, 1024))
    op = Operator(named("k", lambda a, b, c: None))
    monkeypatch.setattr(tuner_mod._C, "do_bench", lambda fn, warmup, rep, stream=None: 0.5)   # ms
    assert op.get_performance(a, b, c) == pytest.approx(2 * 4096 * 1024 * 2048 / 0.5e-3 * 1e-12)
    monkeypatch.setattr(tuner_mod._C, "do_bench", lambda fn, warmup, rep, stream=None: 1e-9)
    assert op.get_performance(a, b, c) == -1             # implausible throughput is discarded


def test_tuner_picks_max_and_memoises(tuner_mod, monkeypatch, tmp_path):
    speeds = {"slow": 10.0, "fast": 99.0, "broken": -1}
    calls = []

    class FakeOp(tuner_mod.Operator):
        def get_performance(self, a, b, c, warmup=5, rep=20, min_ms=0.0):
            calls.append(str(self))
            return speeds[str(self)]

    monkeypatch.setattr(tuner_mod.OperatorTuner, "_get_gemm_specs", lambda self: [])
    monkeypatch.setattr(tuner_mod.OperatorTuner, "_get_gemm_splitk_specs", lambda self: [])

    class Buf(FakeArray):
        def fill_bytes(self, b): pass
        def free(self): pass
    monkeypatch.setattr(tuner_mod.OperatorTuner, "_make_inputs",
                        lambda self, M, N, K, d: (Buf((M, K)), Buf((N, K)), Buf((M, N))))
    path = str(tmp_path / "cache.json")
    t = tuner_mod.OperatorTuner(cache_path=path, verify=False)
    t.gemm_ops = [FakeOp(named(n, lambda a, b, c: None)) for n in speeds]
    t._by_name = {str(o): o for o in t.gemm_ops}
    best, tf = t.tune((512, 256, 1024))
    assert str(best) == "fast" and tf == 99.0
    n = len(calls)
    assert t.tune((512, 256, 1024)) == (best, tf) and len(calls) == n        # memoised
    assert t.get_hash("gemm", [512, 256, 1024]) == "gemm(512,256,1024,)"     # reference key format
    t.tune((512, 256, 1024), dtype="bf16")
    assert len(calls) == 2 * n                                               # dtype is part of the key
    blob = json.load(open(path))
    assert blob["arch"] == "gfx950" and blob["entries"]["gemm(512,256,1024,fp16,gfx950,)"][0] == "fast"
    # a second tuner loads the persisted result and does not re-measure
    t2 = tuner_mod.OperatorTuner(cache_path=path, verify=False)
    t2.gemm_ops = t.gemm_ops
    t2._by_name = t._by_name
    t2._load(path)
    calls.clear()
    assert str(t2.tune((512, 256, 1024))[0]) == "fast" and not calls
    # ... but not a file written on another architecture, or for another CU count
    for change in ({"arch": "gfx942"}, {"compute_units": 12345}):
        other = dict(blob)
        other.update(change)
        monkeypatch.setattr(tuner_mod, "_compute_units", lambda: 256)
        json.dump(other, open(path, "w"))
        t3 = tuner_mod.OperatorTuner(cache_path=path, verify=False)
        assert not t3.cache
    # a problem on which nothing runs is reported, not remembered
    t4 = tuner_mod.OperatorTuner(verify=False)
    t4.gemm_ops = [FakeOp(named("broken", lambda a, b, c: None))]
    assert t4.tune((8, 8, 8)) == (None, -1) and not t4.cache


def test_candidate_space(beamc):
    from beam import tuner
    t = tuner.OperatorTuner(verify=False)
    names = [str(o) for o in t.gemm_ops]
    assert len(names) == len(set(names))
    assert "gemmrc" in names and "custom_gemmrc_128x128" in names and "custom_gemmrc_128x256" in names
    assert sum(n.startswith("gemmrc_splitk_spec") for n in names) >= 5 * len(tuner.SPLIT_FACTORS)
    assert any("256x256" in n for n in names)
    assert tuner.SPLIT_FACTORS == (4, 8, 16, 32, 64)
    # the LDS pipeline depth is an axis of the search: every tile appears with all three depths
    plain = [o for o in t.gemm_ops if str(o).startswith("gemmrc_spec[")]
    depths = {}
    for o in plain:
        c = o.native["config"]
        depths.setdefault((c.block_m, c.block_n, c.wave_m, c.wave_n), set()).add(c.pipeline)
    assert len(depths) == len(beamc.list_configs()) and all(d == {0, 1, 2} for d in depths.values())
