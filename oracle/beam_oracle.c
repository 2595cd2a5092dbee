/*
 * CPU oracle for the gemmrc hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing that ships (the HIP library, the Python `beam` package, the C++ host CLI) may link,
 * load or call this file.  It is used by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py, only as the checker / the reported CPU baseline.
 *
 * The reference repository holds no CPU GEMM (its only answer function is a GPU
 * torch.matmul, python/gemm_test.py:114-115,164-165), no golden vectors and no LayerNorm,
 * so this file restates the arithmetic the reference's kernels fix:
 *
 *   oracle_gemmrc        C[m][n] = sum_k float(A[m][k]) * float(B[n][k])   (fp32 accumulate)
 *                        layouts      cuda/cute_kernels/main.cc:29-40  (A[m,k], B[n,k], C[m,n])
 *                        fp32 acc     cuda/cute_kernels/cute_gemm_128x128.cu:89-92
 *                        RN 16-bit C  cuda/cute_kernels/cute_gemm_128x128.cu:176-188
 *                        alpha=1,beta=0  cuda/cutlass_kernels/cutlass_gemmrc.cu:26-27
 *   oracle_gemmrc_splitk per-slice fp32 partial sums added in slice order
 *                        cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:59-105 (contract only:
 *                        the arithmetic lives in CUTLASS ~3.5.1, which the reference does not
 *                        vendor; partitioning = equal whole K tiles per slice)
 *   oracle_slice_heuristic  cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:44-57
 *   oracle_tflops        cuda/include/gemm_utils.h:3-5
 *   oracle_gemmrc_ln     NOT in the reference (its cute_gemm_ln.cu is a GEMM plus an unrelated
 *                        SiLU).  Textbook LayerNorm over N on the fp32 GEMM result:
 *                        y = (x - mean) / sqrt(var + eps) * gamma + beta, biased variance.
 *
 *   oracle_silu          y = x / (1 + exp(-x)) in fp32 on the widened 16-bit input, RN 16-bit out:
 *                        the side job of cuda/cute_kernels/cute_gemm_ln.cu:186-197 (formula :191-192)
 *
 * Pinning (see tests/test_oracle.py): float64 numpy fixtures under tests/golden, closed forms
 * (identity, all-ones, one-hot), brute-force triple loops on tiny and ragged shapes, numpy's
 * own float16 conversion for the software converters, the worked example tiles=4 -> 41 slices
 * for the heuristic; oracle_silu over all 65536 fp16 inputs against x * scipy.special.expit(x) in
 * float64, the identity silu(x) - silu(-x) = x and the known minimum.  oracle_gemmrc_ln and oracle_gemmrc_splitk have no counterpart the
 * reference's own tests hold: they are pinned by the mathematics only.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_F16 0
#define ORACLE_BF16 1

/* ---------------------------------------------------------------- 16-bit converters */

static inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

float oracle_f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_to_float(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * (1.0f / 16777216.0f);
    return (sign ? -v : v);
  }
  if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
  return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even, overflow to infinity, gradual underflow */
uint16_t oracle_f32_to_f16_bits(float f) {
  const uint32_t x = float_to_bits(f);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (ax < 0x38800000u) {                                   /* below 2^-14: subnormal half */
    if (ax < 0x33000000u) return sign;                      /* < 2^-25 rounds to zero */
    const int e = (int)(ax >> 23);                          /* biased float exponent */
    const uint32_t m = (ax & 0x7fffffu) | 0x800000u;        /* 24-bit significand */
    const int shift = 126 - e;                              /* result = m >> shift, 14..24 */
    uint32_t r = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
  }
  uint32_t r = (ax - 0x38000000u) >> 13; /* rebias 127 -> 15, keep 10 mantissa bits */
  const uint32_t rem = ax & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
  return (uint16_t)(sign | r);
}

float oracle_bf16_bits_to_f32(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

uint16_t oracle_f32_to_bf16_bits(float f) {
  const uint32_t x = float_to_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet NaN */
  const uint32_t lsb = (x >> 16) & 1u;
  return (uint16_t)((x + 0x7fffu + lsb) >> 16);
}

void oracle_to_f32(const uint16_t* src, float* dst, size_t n, int dtype) {
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i)
    dst[i] = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(src[i]) : oracle_f16_bits_to_f32(src[i]);
}

void oracle_from_f32(const float* src, uint16_t* dst, size_t n, int dtype) {
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i)
    dst[i] = dtype == ORACLE_BF16 ? oracle_f32_to_bf16_bits(src[i]) : oracle_f32_to_f16_bits(src[i]);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------- fp32 GEMM core
 *
 * C[m][n] (+)= sum_{k in [k0,k1)} Af[m][k] * Bp(k, n), k ascending, one fp32 FMA chain per
 * output element.  Bp is B converted to fp32 and packed in panels of 16 columns:
 * Bp[(n/16)][k][n%16].  The micro-kernel keeps a 6 x 16 block of C in vector registers.
 */
typedef float v8f __attribute__((vector_size(32), aligned(4)));

#define MR 6
#define NR 16
#define KC 512

static void micro_6x16(const float* a, size_t lda, const float* bp, int kc, float* c, size_t ldc,
                       int mr, int nr, int first) {
  v8f acc[MR][2];
  float tmp[MR][NR];
  if (first) {
    for (int i = 0; i < MR; ++i) acc[i][0] = acc[i][1] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
  } else if (mr == MR && nr == NR) {
    for (int i = 0; i < MR; ++i) {
      acc[i][0] = *(const v8f*)(c + i * ldc);
      acc[i][1] = *(const v8f*)(c + i * ldc + 8);
    }
  } else {
    memset(tmp, 0, sizeof tmp);
    for (int i = 0; i < mr; ++i)
      for (int j = 0; j < nr; ++j) tmp[i][j] = c[i * ldc + j];
    for (int i = 0; i < MR; ++i) {
      acc[i][0] = *(const v8f*)&tmp[i][0];
      acc[i][1] = *(const v8f*)&tmp[i][8];
    }
  }
  const float* arow[MR];
  for (int i = 0; i < MR; ++i) arow[i] = a + (size_t)(i < mr ? i : 0) * lda;
  for (int k = 0; k < kc; ++k) {
    const v8f b0 = *(const v8f*)(bp + (size_t)k * NR);
    const v8f b1 = *(const v8f*)(bp + (size_t)k * NR + 8);
    for (int i = 0; i < MR; ++i) {
      const float av = arow[i][k];
      const v8f a8 = {av, av, av, av, av, av, av, av};
      acc[i][0] += a8 * b0; /* contracted to one FMA per lane under -ffp-contract=fast */
      acc[i][1] += a8 * b1;
    }
  }
  if (mr == MR && nr == NR) {
    for (int i = 0; i < MR; ++i) {
      *(v8f*)(c + i * ldc) = acc[i][0];
      *(v8f*)(c + i * ldc + 8) = acc[i][1];
    }
  } else {
    for (int i = 0; i < MR; ++i) {
      *(v8f*)&tmp[i][0] = acc[i][0];
      *(v8f*)&tmp[i][8] = acc[i][1];
    }
    for (int i = 0; i < mr; ++i)
      for (int j = 0; j < nr; ++j) c[i * ldc + j] = tmp[i][j];
  }
}

/* C32[M][N] = sum over k in [k_begin, k_end) ; returns 0 on success */
static int gemm_f32_range(const uint16_t* A, const uint16_t* B, int M, int N, int K, int dtype,
                          int k_begin, int k_end, float* C32) {
  const int kk = k_end - k_begin;
  if (kk <= 0) {
    memset(C32, 0, (size_t)M * N * sizeof(float));
    return 0;
  }
  const int npanels = (N + NR - 1) / NR;
  float* Af = (float*)malloc((size_t)M * kk * sizeof(float));
  float* Bp = (float*)calloc((size_t)npanels * kk * NR, sizeof(float));
  if (!Af || !Bp) {
    free(Af);
    free(Bp);
    return -1;
  }
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m)
    for (int k = 0; k < kk; ++k) {
      const uint16_t h = A[(size_t)m * K + k_begin + k];
      Af[(size_t)m * kk + k] = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(h) : oracle_f16_bits_to_f32(h);
    }
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n) {
    float* dst = Bp + (size_t)(n / NR) * kk * NR + (n % NR);
    for (int k = 0; k < kk; ++k) {
      const uint16_t h = B[(size_t)n * K + k_begin + k];
      dst[(size_t)k * NR] = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(h) : oracle_f16_bits_to_f32(h);
    }
  }
  const int mblocks = (M + MR - 1) / MR;
#pragma omp parallel for schedule(dynamic, 4)
  for (int mb = 0; mb < mblocks; ++mb) {
    const int m0 = mb * MR;
    const int mr = (M - m0) < MR ? (M - m0) : MR;
    for (int k0 = 0; k0 < kk; k0 += KC) {
      const int kc = (kk - k0) < KC ? (kk - k0) : KC;
      for (int pn = 0; pn < npanels; ++pn) {
        const int n0 = pn * NR;
        const int nr = (N - n0) < NR ? (N - n0) : NR;
        micro_6x16(Af + (size_t)m0 * kk + k0, (size_t)kk, Bp + ((size_t)pn * kk + k0) * NR, kc,
                   C32 + (size_t)m0 * N + n0, (size_t)N, mr, nr, k0 == 0);
      }
    }
  }
  free(Af);
  free(Bp);
  return 0;
}

/* C32 (optional) = fp32 result, C16 (optional) = same rounded to the 16-bit dtype */
int oracle_gemmrc(const uint16_t* A, const uint16_t* B, int M, int N, int K, int dtype, float* C32,
                  uint16_t* C16) {
  float* out = C32 ? C32 : (float*)malloc((size_t)M * N * sizeof(float));
  if (!out) return -1;
  int rc = gemm_f32_range(A, B, M, N, K, dtype, 0, K, out);
  if (rc == 0 && C16) oracle_from_f32(out, C16, (size_t)M * N, dtype);
  if (!C32) free(out);
  return rc;
}

/* Plain triple loop with a double accumulator: the slow, obviously-right cross-check. */
void oracle_gemmrc_naive_f64(const uint16_t* A, const uint16_t* B, int M, int N, int K, int dtype,
                             double* C64) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double s = 0.0;
      for (int k = 0; k < K; ++k) {
        const uint16_t ha = A[(size_t)m * K + k], hb = B[(size_t)n * K + k];
        const float a = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(ha) : oracle_f16_bits_to_f32(ha);
        const float b = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(hb) : oracle_f16_bits_to_f32(hb);
        s += (double)a * (double)b;
      }
      C64[(size_t)m * N + n] = s;
    }
}

/* K elements per slice: equal whole tiles of `ktile` per slice. */
int oracle_split_k_len(int K, int splits, int ktile) {
  const int ktiles = (K + ktile - 1) / ktile;
  return ((ktiles + splits - 1) / splits) * ktile;
}

int oracle_gemmrc_splitk(const uint16_t* A, const uint16_t* B, int M, int N, int K, int dtype,
                         int splits, int ktile, float* C32, uint16_t* C16) {
  if (splits < 1) return -2;
  const size_t mn = (size_t)M * N;
  float* sum = C32 ? C32 : (float*)malloc(mn * sizeof(float));
  float* part = (float*)malloc(mn * sizeof(float));
  if (!sum || !part) return -1;
  const int len = oracle_split_k_len(K, splits, ktile);
  for (int s = 0; s < splits; ++s) {
    int kb = s * len, ke = kb + len;
    if (kb > K) kb = K;
    if (ke > K) ke = K;
    int rc = gemm_f32_range(A, B, M, N, K, dtype, kb, ke, s == 0 ? sum : part);
    if (rc) return rc;
    if (s > 0) {
#pragma omp parallel for schedule(static)
      for (ptrdiff_t i = 0; i < (ptrdiff_t)mn; ++i) sum[i] += part[i];
    }
  }
  if (C16) oracle_from_f32(sum, C16, mn, dtype);
  free(part);
  if (!C32) free(sum);
  return 0;
}

/* Y = LayerNorm_N(A * B^T) * gamma + beta, statistics in double from the fp32 GEMM result. */
int oracle_gemmrc_ln(const uint16_t* A, const uint16_t* B, const uint16_t* gamma,
                     const uint16_t* beta, float eps, int M, int N, int K, int dtype, float* Y32,
                     uint16_t* Y16) {
  const size_t mn = (size_t)M * N;
  float* x = (float*)malloc(mn * sizeof(float));
  float* g = (float*)malloc((size_t)N * sizeof(float));
  float* b = (float*)malloc((size_t)N * sizeof(float));
  if (!x || !g || !b) return -1;
  int rc = gemm_f32_range(A, B, M, N, K, dtype, 0, K, x);
  if (rc) return rc;
  oracle_to_f32(gamma, g, (size_t)N, dtype);
  oracle_to_f32(beta, b, (size_t)N, dtype);
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    const float* xr = x + (size_t)m * N;
    double s = 0.0;
    for (int n = 0; n < N; ++n) s += xr[n];
    const double mean = s / N;
    double q = 0.0;
    for (int n = 0; n < N; ++n) {
      const double d = xr[n] - mean;
      q += d * d;
    }
    const double rstd = 1.0 / sqrt(q / N + (double)eps);
    for (int n = 0; n < N; ++n) {
      const float y = (float)((xr[n] - mean) * rstd * g[n] + b[n]);
      if (Y32) Y32[(size_t)m * N + n] = y;
      if (Y16)
        Y16[(size_t)m * N + n] = dtype == ORACLE_BF16 ? oracle_f32_to_bf16_bits(y) : oracle_f32_to_f16_bits(y);
    }
  }
  free(x);
  free(g);
  free(b);
  return 0;
}

/* ---------------------------------------------------------------- error metrics */

/* max |got - ref| and RMS(ref); `got` is 16-bit, `ref` fp32. Also max |ref|. */
void oracle_compare(const uint16_t* got, const float* ref, size_t n, int dtype, double* max_abs_err,
                    double* rms_ref, double* max_abs_ref, double* max_bf16_excess) {
  double me = 0.0, ss = 0.0, mr = 0.0, mx = 0.0;
#pragma omp parallel for schedule(static) reduction(max : me, mr, mx) reduction(+ : ss)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    const float g = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(got[i]) : oracle_f16_bits_to_f32(got[i]);
    const double r = ref[i];
    const double e = fabs((double)g - r);
    if (e > me) me = e;
    if (fabs(r) > mr) mr = fabs(r);
    ss += r * r;
    /* error beyond the unavoidable half-ulp of an 8-bit significand */
    const double ex = e - fabs(r) * (1.0 / 256.0);
    if (ex > mx) mx = ex;
  }
  *max_abs_err = me;
  *rms_ref = n ? sqrt(ss / (double)n) : 0.0;
  *max_abs_ref = mr;
  if (max_bf16_excess) *max_bf16_excess = mx;
}

/* ---------------------------------------------------------------- host-side formulas */

/* cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:44-57 with the SM count as a parameter
 * (the reference hard-codes 108).  Float arithmetic on purpose: it is what the reference does. */
/* y32[i] = silu(float(x[i])) in fp32 (may be NULL), y16[i] = its RN 16-bit rounding (may be NULL). */
void oracle_silu(const uint16_t* x, uint16_t* y16, float* y32, size_t n, int dtype) {
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) {
    const float v = dtype == 1 ? oracle_bf16_bits_to_f32(x[i]) : oracle_f16_bits_to_f32(x[i]);
    const float r = v / (1.0f + expf(-v));
    if (y32) y32[i] = r;
    if (y16) y16[i] = dtype == 1 ? oracle_f32_to_bf16_bits(r) : oracle_f32_to_f16_bits(r);
  }
}

int oracle_slice_heuristic(int tiles, float units) {
  int split_k_slices = 1;
  if ((float)tiles < units) {
    split_k_slices = (int)((units - 1.0f) / (float)tiles + 1.0f);
    float waves = (float)split_k_slices * (float)tiles / units;
    float rem = waves - (float)(int)waves;
    while (rem < 0.5f) {
      split_k_slices++;
      waves = (float)split_k_slices * (float)tiles / units;
      rem = waves - (float)(int)waves;
    }
  }
  return split_k_slices;
}

/* cuda/include/gemm_utils.h:3-5 */
double oracle_tflops(double m, double n, double k, double ms) { return 2.0 * m * n * k / ms / 1e9; }
