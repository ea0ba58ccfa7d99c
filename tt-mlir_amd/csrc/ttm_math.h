// Scalar math shared by the compute kernels.
#pragma once
#include <hip/hip_runtime.h>

// erfc(z) for z >= 0 as a degree-5 polynomial in t = 1/(1 + p z) times exp(-z^2)
// (Abramowitz & Stegun 7.1.26, absolute error <= 1.5e-7).
__device__ __forceinline__ float ttm_erfc_pos(float z) {
  const float t = __frcp_rn(fmaf(0.3275911f, z, 1.0f));
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  return p * t * __expf(-z * z);
}

// gelu(x) = 0.5 x (1 + erf(x / sqrt 2)); uses erfc on the negative side so the tail keeps its
// relative accuracy.  Absolute error <= 0.5 |x| 1.5e-7, far below bf16 output resolution; used by
// fused epilogues whose result is rounded to bf16.  The stand-alone eltwise kernel uses erff.
__device__ __forceinline__ float ttm_gelu_fast(float x) {
  const float e = ttm_erfc_pos(fabsf(x) * 0.70710678118654752f);
  const float one_plus_erf = x < 0.0f ? e : 2.0f - e;
  return 0.5f * x * one_plus_erf;
}

__device__ __forceinline__ float ttm_gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }
__device__ __forceinline__ float ttm_sigmoid(float x) { return __frcp_rn(1.0f + __expf(-x)); }
__device__ __forceinline__ float ttm_silu(float x) { return x * ttm_sigmoid(x); }
