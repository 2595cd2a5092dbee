// Measurement kernels that are not operators (declared in include/beam_hip_debug.h): the split-K partial kernel
// with nothing but its loads (kEpiProbeLoads in gemm_kernel.h) and the register-only matrix-core loop.
#include "gemm_w4.h"
#include "kernel_set.h"

namespace beam {

hipError_t launch_probe_splitk_loads(const GemmParams& p, int block_m, int block_n, dim3 grid, hipStream_t stream) {
  if (block_m == 64 && block_n == 128) {
    constexpr int DA = deep_a_slots(64, 128);
    return launch_gemm<_Float16, 64, 128, 2, 2, kEpiProbeLoads, DA, DA - 1>(p, grid, stream);
  }
  if (block_m == 64 && block_n == 64) {
    constexpr int DA = deep_a_slots(64, 64);
    return launch_gemm<_Float16, 64, 64, 2, 2, kEpiProbeLoads, DA, DA - 1>(p, grid, stream);
  }
  return hipErrorInvalidValue;
}

// ---- what the matrix cores sustain with operands in registers -----------------------------------------
// One wavefront per SIMD, as in gemm_w4.h, and the same instruction stream minus everything that is not an
// MFMA: 8 A and 8 B fragments in ordinary registers, 64 accumulator blocks in the accumulation registers,
// a pass = the 64 block products in that kernel's order (rows in turn, B fragments forwards and backwards
// alternately, so consecutive MFMAs share an operand).  The 32x32x16 form covers the same 128 x 128 x 32
// per pass with 4 x 4 blocks of 16 accumulation registers and fragments of 32 rows.
// Operands: N(0,1) / sqrt(8192) from a counter hash (the distribution of the headline workload's operands)
// or zeros.  The accumulators random-walk with a standard deviation of 6e-4 sqrt(passes): no overflow.
namespace {

__device__ float g_probe_sink[1 << 18];  // one word per thread of the largest grid (1024 workgroups)

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// element `i` of thread `gid`: N(0,1) * scale by Box-Muller on two hashed uniforms
__device__ __forceinline__ float probe_normal(unsigned gid, unsigned i, float scale) {
  const unsigned h1 = probe_hash(gid * 0x9E3779B1u + i * 2u + 1u), h2 = probe_hash(h1 ^ 0x85EBCA6Bu);
  const float u1 = ((float)(h1 >> 8) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
  const float u2 = (float)(h2 >> 8) * (1.0f / 16777216.0f);
  return scale * sqrtf(-2.0f * __logf(u1)) * __cosf(6.2831853f * u2);
}

template <typename T>
struct Mfma32;
template <>
struct Mfma32<_Float16> {
  template <int BLK>
  static __device__ __forceinline__ void fma(f16x8 b, f16x8 a) {
    asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(b), "v"(a), "n"(16 * BLK), "n"(16 * BLK + 15));
  }
  template <int BLK>
  static __device__ __forceinline__ void first(f16x8 b, f16x8 a) {
    asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, 0" ::"v"(b), "v"(a), "n"(16 * BLK), "n"(16 * BLK + 15));
  }
};
template <>
struct Mfma32<__bf16> {
  template <int BLK>
  static __device__ __forceinline__ void fma(bf16x8 b, bf16x8 a) {
    asm volatile("v_mfma_f32_32x32x16_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(b), "v"(a), "n"(16 * BLK), "n"(16 * BLK + 15));
  }
  template <int BLK>
  static __device__ __forceinline__ void first(bf16x8 b, bf16x8 a) {
    asm volatile("v_mfma_f32_32x32x16_bf16 a[%2:%3], %0, %1, 0" ::"v"(b), "v"(a), "n"(16 * BLK), "n"(16 * BLK + 15));
  }
};

// A pass is 1024 matrix-core cycles either way: SHAPE 0, 64 MFMAs of 16x16x32 (16 cycles each, the 8 x 8 blocks
// once); SHAPE 1, 32 MFMAs of 32x32x16 (32 cycles each, the 4 x 4 blocks twice).
template <typename T, int SHAPE>
__global__ void __launch_bounds__(256) mfma_ceiling_kernel(int passes, int zeros) {
  using vec8 = typename ElemTraits<T>::vec8;
  constexpr int F = SHAPE == 0 ? 8 : 4;  // fragments per operand
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  w4_claim_acc_registers();
  vec8 fa[F], fb[F];
#pragma unroll
  for (int i = 0; i < F; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      fa[i][e] = (T)(zeros ? 0.0f : probe_normal(gid, (unsigned)(i * 8 + e), 0.011048543f));
      fb[i][e] = (T)(zeros ? 0.0f : probe_normal(gid, (unsigned)(64 + i * 8 + e), 0.011048543f));
    }
  // the accumulators start from a product, not from whatever the registers held
  w4_static_for<0, F * F>([&](auto m_tag) __attribute__((always_inline)) {
    constexpr int m = decltype(m_tag)::value;
    constexpr int i = m / F, b = (i & 1) ? F - 1 - (m % F) : (m % F);
    if constexpr (SHAPE == 0) W4Mfma<T>::template first<F * i + b>(fb[b], fa[i]);
    else Mfma32<T>::template first<F * i + b>(fb[b], fa[i]);
  });
  for (int pass = 0; pass < passes; ++pass) {
    w4_static_for<0, (SHAPE == 0 ? 1 : 2) * F * F>([&](auto m_tag) __attribute__((always_inline)) {
      constexpr int m = decltype(m_tag)::value % (F * F);
      constexpr int i = m / F, b = (i & 1) ? F - 1 - (m % F) : (m % F);
      if constexpr (SHAPE == 0) W4Mfma<T>::template fma<F * i + b>(fb[b], fa[i]);
      else Mfma32<T>::template fma<F * i + b>(fb[b], fa[i]);
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");  // the last results have left the matrix core
  const float s = w4_acc_read<0>() + w4_acc_read<85>() + w4_acc_read<170>() + w4_acc_read<255>();
  if (gid < (1u << 18)) g_probe_sink[gid] = s;
}

template <typename T, int SHAPE>
hipError_t launch_mfma_ceiling_t(int workgroups, int passes, int zeros, hipStream_t stream) {
  hipLaunchKernelGGL((mfma_ceiling_kernel<T, SHAPE>), dim3((unsigned)workgroups), dim3(256), 0, stream, passes, zeros);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_probe_mfma(int dtype, int mfma_shape, int workgroups, int passes, int zeros, hipStream_t stream) {
  if (workgroups < 1 || workgroups > 1024 || passes < 0 || mfma_shape < 0 || mfma_shape > 1) return hipErrorInvalidValue;
  if (dtype == BEAM_BF16)
    return mfma_shape == 0 ? launch_mfma_ceiling_t<__bf16, 0>(workgroups, passes, zeros, stream)
                           : launch_mfma_ceiling_t<__bf16, 1>(workgroups, passes, zeros, stream);
  return mfma_shape == 0 ? launch_mfma_ceiling_t<_Float16, 0>(workgroups, passes, zeros, stream)
                         : launch_mfma_ceiling_t<_Float16, 1>(workgroups, passes, zeros, stream);
}

}  // namespace beam
