"""Writes the committed golden fixtures (tests/golden/*.npz).

The reference repository holds no golden vectors, fixtures or seeds for this path (its only check
is a live comparison with a GPU torch.matmul, python/gemm_test.py:29-70), so these are computed
here from the mathematical definition in numpy float64 -- independently of oracle/ and of the
GPU code -- and pin both of them:

  gemm_*.npz : a (uint16 bits), b (uint16 bits), dtype (0 fp16 / 1 bf16),
               c64 = float64(a) @ float64(b).T
  ln_*.npz   : a, b, gamma, beta (bits), eps, y64 = LayerNorm over N (biased variance) of c64,
               times gamma plus beta, all in float64

Inputs come from numpy's PCG64 and are stored in the files, so nothing depends on regenerating
them.  Run:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def to_bf16_bits(x32: np.ndarray) -> np.ndarray:
    u = x32.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bits_to_f64(bits: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == 1:
        return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return bits.view(np.float16).astype(np.float64)


def make_bits(rng, shape, dtype, kind, scale=1.0, mean=0.0):
    x = rng.uniform(-1.0, 1.0, shape) if kind == "uniform" else mean + scale * rng.standard_normal(shape)
    x = x.astype(np.float32)
    return to_bf16_bits(x) if dtype == 1 else x.astype(np.float16).view(np.uint16)


def main():
    rng = np.random.Generator(np.random.PCG64(20240607))
    gemm_cases = [("tiny", 3, 5, 16, 0, "uniform"), ("ragged", 130, 70, 48, 0, "uniform"),
                  ("edge", 257, 129, 200, 0, "uniform"), ("square", 192, 192, 320, 0, "normal"),
                  ("bf16", 96, 160, 136, 1, "uniform"), ("bf16_ragged", 33, 47, 72, 1, "normal")]
    for name, M, N, K, dtype, kind in gemm_cases:
        scale = K ** -0.5 if kind == "normal" else 1.0
        a = make_bits(rng, (M, K), dtype, kind, scale)
        b = make_bits(rng, (N, K), dtype, kind, scale)
        c64 = bits_to_f64(a, dtype) @ bits_to_f64(b, dtype).T
        np.savez_compressed(os.path.join(HERE, f"gemm_{name}.npz"), a=a, b=b, dtype=np.int32(dtype), c64=c64)
    ln_cases = [("small", 24, 96, 64, 0), ("ragged", 50, 200, 72, 0), ("wide", 16, 1024, 128, 0),
                ("bf16", 40, 256, 64, 1)]
    for name, M, N, K, dtype in ln_cases:
        a = make_bits(rng, (M, K), dtype, "normal", K ** -0.5)
        b = make_bits(rng, (N, K), dtype, "normal", K ** -0.5)
        gamma = make_bits(rng, (N,), dtype, "normal", 0.1, 1.0)
        beta = make_bits(rng, (N,), dtype, "normal", 0.1, 0.0)
        eps = 1e-5
        x = bits_to_f64(a, dtype) @ bits_to_f64(b, dtype).T
        mu = x.mean(axis=1, keepdims=True)
        var = ((x - mu) ** 2).mean(axis=1, keepdims=True)
        y64 = (x - mu) / np.sqrt(var + eps) * bits_to_f64(gamma, dtype) + bits_to_f64(beta, dtype)
        np.savez_compressed(os.path.join(HERE, f"ln_{name}.npz"), a=a, b=b, gamma=gamma, beta=beta,
                            dtype=np.int32(dtype), eps=np.float64(eps), y64=y64)


if __name__ == "__main__":
    main()
