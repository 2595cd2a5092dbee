// Bandwidth-bound companions of the tiled kernel: the split-K reduction and the LayerNorm
// normalisation pass.  Both stream fp32 from the workspace once and write 16-bit once.
#include "aux_kernels.h"

#include <type_traits>

#include "elementwise.h"
#include "tile_map.h"

namespace beam {

namespace {

template <typename T>
struct Vec4Of;
template <>
struct Vec4Of<_Float16> { typedef _Float16 type __attribute__((ext_vector_type(4))); };
template <>
struct Vec4Of<__bf16> { typedef __bf16 type __attribute__((ext_vector_type(4))); };

typedef float f32x4 __attribute__((ext_vector_type(4)));

// C[i] = round( ws[0][i] + ws[1][i] + ... + ws[S-1][i] ), slices added in index order.
// The fixed order is what makes split-K bit-reproducible (the reference delegates this to
// CUTLASS's reduce kernel, cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:73-75).
template <typename T>
__global__ void __launch_bounds__(64) splitk_reduce_kernel(const float* __restrict__ ws, T* __restrict__ C,
                                                            size_t mn, int splits, int* sync_header) {
  typedef typename Vec4Of<T>::type vec4;
  // the latest call on this workspace is not a one-launch one: whatever time-out its header records is not this call's
  if (sync_header != nullptr && blockIdx.x == 0 && threadIdx.x == 0) sync_header[kSkLaunchTag] = 0;
  const size_t quads = mn / 4;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += stride) {
    const float* src = ws + q * 4;
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    int z = 0;
    // Batches of 16, 8, 4, 2, 1 slices: all loads of a batch in flight before the first add, the
    // adds in slice order (slice 0 starts the sum, so that the sign of an all-zero sum is kept).
    auto batch = [&](auto n_tag) {
      constexpr int NB = decltype(n_tag)::value;
      while (z + NB <= splits) {
        f32x4 v[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) v[u] = *(const f32x4*)(src + (size_t)(z + u) * mn);
        if (z == 0) s = v[0];
        else s += v[0];
#pragma unroll
        for (int u = 1; u < NB; ++u) s += v[u];
        z += NB;
      }
    };
    batch(std::integral_constant<int, 16>{});
    batch(std::integral_constant<int, 8>{});
    batch(std::integral_constant<int, 4>{});
    batch(std::integral_constant<int, 2>{});
    batch(std::integral_constant<int, 1>{});
    vec4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (T)s[e];
    *(vec4*)(C + q * 4) = o;
  }
  // tail (mn not a multiple of 4)
  const size_t t = quads * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < mn) {
    float s = ws[t];
    for (int z = 1; z < splits; ++z) s += ws[(size_t)z * mn + t];
    C[t] = (T)s;
  }
}

// One workgroup per row: merge the per-column-tile (mean, M2) pairs in tile order (Chan's
// update), then y = (x - mean) * rstd * gamma + beta from the fp32 x.
template <typename T>
__global__ void __launch_bounds__(256) ln_apply_kernel(const float* __restrict__ X,
                                                        const float* __restrict__ stats,
                                                        const T* __restrict__ gamma,
                                                        const T* __restrict__ beta, T* __restrict__ Y,
                                                        int N, int tiles_n, int block_n, float eps) {
  typedef typename Vec4Of<T>::type vec4;
  const int m = blockIdx.x;
  const float* st = stats + (size_t)m * tiles_n * 2;
  float mean = 0.0f, m2 = 0.0f, cnt = 0.0f;
  for (int t = 0; t < tiles_n; ++t) {
    int cw = N - t * block_n;
    cw = cw > block_n ? block_n : cw;
    const float nb = (float)cw;
    const float tot = cnt + nb;
    const float delta = st[2 * t] - mean;
    mean += delta * (nb / tot);
    m2 += st[2 * t + 1] + delta * delta * (cnt * nb / tot);
    cnt = tot;
  }
  const float rstd = 1.0f / sqrtf(m2 / (float)N + eps);
  const float* x = X + (size_t)m * N;
  T* y = Y + (size_t)m * N;
  if ((N & 3) == 0) {
    for (int n = threadIdx.x * 4; n < N; n += blockDim.x * 4) {
      const f32x4 v = *(const f32x4*)(x + n);
      const vec4 g = *(const vec4*)(gamma + n);
      const vec4 b = *(const vec4*)(beta + n);
      vec4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (T)((v[e] - mean) * rstd * (float)g[e] + (float)b[e]);
      *(vec4*)(y + n) = o;
    }
  } else {
    for (int n = threadIdx.x; n < N; n += blockDim.x)
      y[n] = (T)((x[n] - mean) * rstd * (float)gamma[n] + (float)beta[n]);
  }
}

// y[i] = silu(x[i]) over a flat 16-bit array: 16 bytes per lane per access, four accesses in flight,
// then the elements after the last whole vector.
template <typename T>
__global__ void __launch_bounds__(256) silu_kernel(const T* __restrict__ x, T* __restrict__ y, size_t count) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  const size_t vecs = count / 8;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; v + 3 * stride < vecs; v += 4 * stride) {
    vec8 in[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) in[u] = *(const vec8*)(x + (v + u * stride) * 8);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      vec8 out;
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = silu_16<T>(in[u][e]);
      *(vec8*)(y + (v + u * stride) * 8) = out;
    }
  }
  for (; v < vecs; v += stride) {
    const vec8 in = *(const vec8*)(x + v * 8);
    vec8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = silu_16<T>(in[e]);
    *(vec8*)(y + v * 8) = out;
  }
  const size_t i = vecs * 8 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) y[i] = silu_16<T>(x[i]);
}

// gemmrc for problems the tiled kernels do not take: K not a multiple of 8 (rows of A and B are then not
// 16-byte aligned), operands or output at odd addresses, and the [K][N] layout with N not a multiple of 8.
// A plain LDS-tiled fp32 kernel: 64 x 64 outputs per workgroup, 16 K elements per step, 4 x 4 outputs per
// thread, every access bounds-checked element by element.  Same arithmetic contract (16-bit inputs, fp32
// accumulation, one rounding), far from the same speed; it exists so that no well-formed problem is refused
// (the reference's Triton matmul masks any edge: python/beam/triton_kernels/gemm.py:62-63,75).
// OUT32: write fp32 (the input of the row-wise LayerNorm below) instead of the 16-bit type.
template <typename T, bool B_KMAJOR, bool OUT32>
__global__ void __launch_bounds__(256) generic_gemm_kernel(const T* __restrict__ A, const T* __restrict__ B, void* __restrict__ Cv,
                                                            int M, int N, int K) {
  constexpr int TS = 64, KS = 16;
  __shared__ float as[KS][TS + 1], bs[KS][TS + 1];
  const int tid = threadIdx.x;
  const int row0 = blockIdx.y * TS, col0 = blockIdx.x * TS;
  const int ty = tid / 16, tx = tid % 16;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += KS) {
    // 64 rows x 16 k of each operand: thread t fetches row t / 4, k (t % 4) * 4 .. + 3
    const int lr = tid / 4, lk = (tid % 4) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int m = row0 + lr, n = col0 + lr;
      as[lk + e][lr] = (m < M && k < K) ? (float)A[(size_t)m * K + k] : 0.0f;
      bs[lk + e][lr] = (n < N && k < K) ? (float)(B_KMAJOR ? B[(size_t)k * N + n] : B[(size_t)n * K + k]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = as[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = row0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = col0 + tx * 4 + j;
      if (n >= N) continue;
      if (OUT32) ((float*)Cv)[(size_t)m * N + n] = acc[i][j];
      else ((T*)Cv)[(size_t)m * N + n] = (T)acc[i][j];
    }
  }
}

// Row-wise LayerNorm of fp32 X for the generic path: one workgroup per row; mean, then M2 about it (two passes
// over the row, no cancellation), then y = (x - mean) * rstd * gamma + beta.  Scalar accesses: no alignment
// is assumed of anything.
template <typename T>
__global__ void __launch_bounds__(256) ln_rows_kernel(const float* __restrict__ X, const T* __restrict__ gamma,
                                                       const T* __restrict__ beta, T* __restrict__ Y, int N, float eps) {
  __shared__ float red[256];
  const float* x = X + (size_t)blockIdx.x * N;
  T* y = Y + (size_t)blockIdx.x * N;
  auto block_sum = [&](float v) {
    red[threadIdx.x] = v;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
      if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
      __syncthreads();
    }
    const float total = red[0];
    __syncthreads();
    return total;
  };
  float s = 0.0f;
  for (int n = threadIdx.x; n < N; n += 256) s += x[n];
  const float mean = block_sum(s) / (float)N;
  float q = 0.0f;
  for (int n = threadIdx.x; n < N; n += 256) {
    const float d = x[n] - mean;
    q += d * d;
  }
  const float rstd = 1.0f / sqrtf(block_sum(q) / (float)N + eps);
  for (int n = threadIdx.x; n < N; n += 256) y[n] = (T)((x[n] - mean) * rstd * (float)gamma[n] + (float)beta[n]);
}

// In front of a fused GEMM+LayerNorm launch that is being recorded into a graph: the launch's arguments, its
// nonce among them, repeat from replay to replay, so the part of its tag that changes is this counter in the
// workspace header.  Whatever the word held before, it holds something else afterwards.
__global__ void ln_replay_bump_kernel(int* hdr) { hdr[kLnHdrReplay] = hdr[kLnHdrReplay] + 1; }

__global__ void empty_kernel(int* p) {
  if (p && threadIdx.x == 0x7fffffff) *p = 1;  // never true: keeps the argument alive
}

__global__ void zero_u16_kernel(unsigned short* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

__global__ void zero_ints_kernel(int* p, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0;
}

__global__ void fill_floats_kernel(float* p, size_t n, float v) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

}  // namespace

hipError_t launch_silu(const void* x, void* y, size_t count, int dtype, hipStream_t stream) {
  size_t blocks = (count / 8 + 4 * 256 - 1) / (4 * 256);
  if (blocks < 1) blocks = 1;
  if (blocks > 8192) blocks = 8192;
  if (dtype == BEAM_BF16)
    hipLaunchKernelGGL(silu_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, stream, (const __bf16*)x,
                       (__bf16*)y, count);
  else
    hipLaunchKernelGGL(silu_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, stream, (const _Float16*)x,
                       (_Float16*)y, count);
  return hipGetLastError();
}

hipError_t launch_fill_floats(float* floats, size_t n, float value, hipStream_t stream) {
  hipLaunchKernelGGL(fill_floats_kernel, dim3(256), dim3(256), 0, stream, floats, n, value);
  return hipGetLastError();
}

hipError_t launch_generic_gemm(const void* A, const void* B, void* C, int M, int N, int K, int dtype, bool b_kmajor,
                               bool out_fp32, hipStream_t stream) {
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64), 1);
#define BEAM_GENERIC(T, KM, O32) \
  hipLaunchKernelGGL((generic_gemm_kernel<T, KM, O32>), grid, dim3(256), 0, stream, (const T*)A, (const T*)B, C, M, N, K)
#define BEAM_GENERIC_T(T)                                   \
  do {                                                      \
    if (b_kmajor && out_fp32) BEAM_GENERIC(T, true, true);  \
    else if (b_kmajor) BEAM_GENERIC(T, true, false);        \
    else if (out_fp32) BEAM_GENERIC(T, false, true);        \
    else BEAM_GENERIC(T, false, false);                     \
  } while (0)
  if (dtype == BEAM_BF16) BEAM_GENERIC_T(__bf16);
  else BEAM_GENERIC_T(_Float16);
#undef BEAM_GENERIC_T
#undef BEAM_GENERIC
  return hipGetLastError();
}

hipError_t launch_ln_rows(const float* X, const void* gamma, const void* beta, void* Y, int M, int N, float eps, int dtype,
                          hipStream_t stream) {
  if (dtype == BEAM_BF16)
    hipLaunchKernelGGL(ln_rows_kernel<__bf16>, dim3((unsigned)M), dim3(256), 0, stream, X, (const __bf16*)gamma, (const __bf16*)beta,
                       (__bf16*)Y, N, eps);
  else
    hipLaunchKernelGGL(ln_rows_kernel<_Float16>, dim3((unsigned)M), dim3(256), 0, stream, X, (const _Float16*)gamma,
                       (const _Float16*)beta, (_Float16*)Y, N, eps);
  return hipGetLastError();
}

hipError_t launch_ln_replay_bump(int* header, hipStream_t stream) {
  hipLaunchKernelGGL(ln_replay_bump_kernel, dim3(1), dim3(1), 0, stream, header);
  return hipGetLastError();
}

hipError_t launch_zero_u16(void* p, size_t n, hipStream_t stream) {
  size_t blocks = (n + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(zero_u16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (unsigned short*)p, n);
  return hipGetLastError();
}

hipError_t launch_empty(int workgroups, int threads, hipStream_t stream) {
  hipLaunchKernelGGL(empty_kernel, dim3((unsigned)workgroups), dim3((unsigned)threads), 0, stream, (int*)nullptr);
  return hipGetLastError();
}

hipError_t launch_zero_ints(int* ints, int n, hipStream_t stream) {
  hipLaunchKernelGGL(zero_ints_kernel, dim3(1), dim3(256), 0, stream, ints, n);
  return hipGetLastError();
}

hipError_t launch_splitk_reduce(const float* ws, void* C, size_t mn, int splits, int dtype, int* sync_header,
                                hipStream_t stream) {
  // one wavefront per workgroup: even a 256 x 256 output spreads over 256 CUs
  size_t quads = (mn + 3) / 4;
  size_t blocks = (quads + 63) / 64;
  if (blocks < 1) blocks = 1;
  if (blocks > 16384) blocks = 16384;
  if (dtype == BEAM_BF16)
    hipLaunchKernelGGL(splitk_reduce_kernel<__bf16>, dim3((unsigned)blocks), dim3(64), 0, stream, ws,
                       (__bf16*)C, mn, splits, sync_header);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<_Float16>, dim3((unsigned)blocks), dim3(64), 0, stream, ws,
                       (_Float16*)C, mn, splits, sync_header);
  return hipGetLastError();
}

hipError_t launch_ln_apply(const float* X, const float* stats, const void* gamma, const void* beta,
                           void* Y, int M, int N, int tiles_n, int block_n, float eps, int dtype,
                           hipStream_t stream) {
  if (dtype == BEAM_BF16)
    hipLaunchKernelGGL(ln_apply_kernel<__bf16>, dim3(M), dim3(256), 0, stream, X, stats,
                       (const __bf16*)gamma, (const __bf16*)beta, (__bf16*)Y, N, tiles_n, block_n, eps);
  else
    hipLaunchKernelGGL(ln_apply_kernel<_Float16>, dim3(M), dim3(256), 0, stream, X, stats,
                       (const _Float16*)gamma, (const _Float16*)beta, (_Float16*)Y, N, tiles_n,
                       block_n, eps);
  return hipGetLastError();
}

}  // namespace beam
