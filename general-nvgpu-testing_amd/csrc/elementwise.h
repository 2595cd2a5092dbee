// Elementwise functions shared by the tiled kernel's side job and the standalone streaming kernel.
#pragma once

#include <hip/hip_runtime.h>

namespace beam {

// silu(x) = x / (1 + exp(-x)) in fp32 (hardware exp2 and reciprocal, about 1 ulp each: far inside
// the rounding of a 16-bit result).  Same formula as the reference's side job,
// cuda/cute_kernels/cute_gemm_ln.cu:191-192.
//
// WIDE_RANGE: the hardware reciprocal flushes denormal results, which 1 / (1 + exp(-x)) is for x below
// -87.3 although x times it is still a normal fp32 number down to x = -88.7 (where exp(-x) overflows
// and the formula gives -0).  bf16 can hold a result that small, so for bf16 numerator and
// denominator are scaled by 2^-64 in that range; an fp16 result is -0 there either way.
//
// The product passes through an empty asm so that it stays a plain fp32 multiply: a multiply that
// feeds the 16-bit conversion directly is selected as a mixed-precision fma with a +0 addend,
// which turns the -0 of silu(-0) into +0.
template <bool WIDE_RANGE>
__device__ __forceinline__ float silu_f32(float x) {
  const float d = 1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  float r;
  if (WIDE_RANGE) {
    const bool big = d > 0x1p64f;
    const float ds = big ? d * 0x1p-64f : d;
    const float xs = big ? x * 0x1p-64f : x;
    r = xs * __builtin_amdgcn_rcpf(ds);
  } else {
    r = x * __builtin_amdgcn_rcpf(d);
  }
  asm("" : "+v"(r));
  return r;
}

template <typename T>
__device__ __forceinline__ T silu_16(T x) {
  return (T)silu_f32<sizeof(T) == 2 && !__is_same(T, _Float16)>((float)x);
}

}  // namespace beam
