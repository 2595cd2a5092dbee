"""Run by tests/test_gpu_golden.py in a fresh process: the reference-named operators on torch CUDA
tensors, checked against the CPU oracle."""
import os
import sys

import numpy as np
import torch  # before beam: both then use the HIP runtime bundled with torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "general-nvgpu-testing_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

import beam  # noqa: E402
import oracle  # noqa: E402
from beam import _C  # noqa: E402

F16 = 0
M, N, K = 512, 640, 1024
a_bits = _C.host_uniform((M, K), F16, 31, 0)
b_bits = _C.host_uniform((N, K), F16, 31, 1)
ref = oracle.gemmrc(a_bits, b_bits, F16)
a = torch.from_numpy(a_bits.view(np.float16)).cuda()
b = torch.from_numpy(b_bits.view(np.float16)).cuda()
stream = torch.cuda.Stream()
with torch.cuda.stream(stream):
    for fn, kw in [(beam.custom_gemmrc_128x128, {}), (beam.custom_gemmrc_128x256, {}), (beam.cutlass_gemmrc, {}),
                   (beam.cutlass_gemmrc_spec, dict(shape_threadblock=[256, 128], shape_warp=[128, 32])),
                   (beam.cutlass_gemmrc_splitk, dict(split_k_slices=3)),
                   (beam.cutlass_gemmrc_splitk_spec, dict(shape_threadblock=[128, 64], shape_warp=[64, 32],
                                                          split_k_slices=5))]:
        c = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        fn(a=a, b=b, c=c, **kw)
        stream.synchronize()
        r = oracle.compare(c.cpu().numpy().view(np.uint16), ref, F16)
        assert r["max_abs_err"] <= oracle.gemm_tolerance(K) * r["rms_ref"], (fn.__name__, r)
        print(fn.__name__, "ok", r["max_abs_err"], flush=True)

# bf16 through the generic entry
ab = _C.host_uniform((M, K), 1, 32, 0)
bb = _C.host_uniform((N, K), 1, 32, 1)
refb = oracle.gemmrc(ab, bb, 1)
ta = torch.from_numpy(ab.view(np.int16)).cuda().view(torch.bfloat16)
tb = torch.from_numpy(bb.view(np.int16)).cuda().view(torch.bfloat16)
tc = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
beam.cutlass_gemmrc(a=ta, b=tb, c=tc)
torch.cuda.synchronize()
r = oracle.compare(tc.view(torch.int16).cpu().numpy().view(np.uint16), refb, 1)
assert r["max_bf16_excess"] <= oracle.gemm_tolerance(K) * r["rms_ref"], r


def raises(fn):
    try:
        fn()
    except beam.BeamError:
        return True
    return False


# unsupported inputs raise instead of returning silently (the reference prints and returns,
# cuda/cutlass_kernels/main.cc:43-45)
assert raises(lambda: beam.cutlass_gemmrc(a=a.float(), b=b.float(), c=torch.zeros(M, N, device="cuda")))
assert raises(lambda: beam.cutlass_gemmrc(a=a.cpu(), b=b, c=torch.zeros(M, N, dtype=torch.float16, device="cuda")))
assert raises(lambda: beam.cutlass_gemmrc_spec(a=a, b=b, c=torch.zeros(M, N, dtype=torch.float16, device="cuda"),
                                               shape_threadblock=[48, 48]))
assert raises(lambda: beam.cutlass_gemmrc(a=a, b=b[:, : K // 2], c=torch.zeros(M, N, dtype=torch.float16, device="cuda")))
print("torch drop-in OK", flush=True)
