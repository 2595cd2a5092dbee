"""The C++ host (beam_host: test registry + CLI over the C ABI) runs its self-checks on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "general-nvgpu-testing_amd", "beam_host")


def run(*args, timeout=240):
    return subprocess.run([HOST, *args], capture_output=True, text=True, timeout=timeout)


def test_registry_runs_green(gpu):
    assert os.path.exists(HOST), "beam_host is not built (make -C general-nvgpu-testing_amd/csrc)"
    listed = run("--list").stdout.split()
    assert {"identity_every_tile", "all_ones_ragged", "one_hot_k_tail", "splitk_consistency",
            "layernorm_invariants", "gemm_silu_side_job", "matmul_nn_every_tile", "error_paths"} <= set(listed)
    r = run("--run", "all")
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("[ OK ]") == len(listed) and "FAIL" not in r.stdout


def test_cli_bench_and_info(gpu):
    r = run("--info")
    assert r.returncode == 0 and "gfx950" in r.stdout
    r = run("--bench", "--m", "1024", "--n", "1024", "--k", "1024", "--tile", "128x128", "--wave", "64x64", "--iters", "5")
    assert r.returncode == 0 and "TFLOP/s" in r.stdout, r.stdout + r.stderr
    r = run("--bench", "--op", "splitk", "--m", "256", "--n", "256", "--k", "8192", "--tile", "64x64", "--wave", "32x32",
            "--splitk", "16", "--iters", "5")
    assert r.returncode == 0 and "split 16" in r.stdout, r.stdout + r.stderr
    r = run("--bench", "--op", "silu", "--m", "1024", "--n", "1024", "--k", "1024", "--count", "1048579", "--iters", "5",
            "--warmup", "2")
    assert r.returncode == 0 and "gemm+silu in one launch" in r.stdout, r.stdout + r.stderr
    r = run("--bench", "--op", "nn", "--m", "512", "--n", "1024", "--k", "768", "--iters", "5")
    assert r.returncode == 0 and r.stdout.startswith("nn 512x1024x768"), r.stdout + r.stderr
    r = run("--bench", "--tile", "100x100")
    assert r.returncode != 0


def _ms(stdout):
    return float(stdout.split(":")[-1].split("ms")[0])


def test_cli_launch_floor_probes(gpu):
    """The launches that measure what the machine allows for split-K at 256 x 256 x 32768: an empty kernel, two
    of them, and the library's partial kernel with nothing but its loads.  They run, leave C alone, and are
    ordered as they must be: one empty launch <= two, loads only <= the whole split-K call."""
    shape = ["--m", "256", "--n", "256", "--k", "32768", "--data", "uniform", "--iters", "200", "--warmup", "50"]
    t = {}
    for op in ("probe-empty", "probe-empty-pair", "probe-splitk-loads", "splitk"):
        r = run("--bench", "--op", op, *shape)
        assert r.returncode == 0 and r.stdout.startswith(op), r.stdout + r.stderr
        t[op] = _ms(r.stdout)
    assert 0 < t["probe-empty"] <= t["probe-empty-pair"] * 1.05
    assert t["probe-empty"] < t["probe-splitk-loads"] <= t["splitk"] * 1.05, t
    # a tile the probe is not built for is refused, not run as something else
    r = run("--bench", "--op", "probe-splitk-loads", "--tile", "128x128", "--wave", "64x64", *shape)
    assert r.returncode != 0 and "probe" in r.stderr
