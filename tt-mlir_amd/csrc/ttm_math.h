// Scalar math shared by the compute kernels.
#pragma once
#include <hip/hip_runtime.h>

// gelu(x) = x Phi(x) for fused epilogues whose result is rounded to bf16.  With u = min(|x|, 6) and
// Q(u) = 1 - Phi(u) = 2^P(u) / 2, where P is a degree-6 fit of log2(2 Q) on [0, 6] (max error 6.6e-5, i.e. 4.6e-5
// relative in Q):  gelu(x) = (x + |x|) / 2 - u Q(u), which is x Q for x < 0 and x - x Q for x > 0.  One v_exp_f32 and
// ten other instructions, no reciprocal and no branch (the epilogue of a 256 x 256 block evaluates this 65 536
// times while the matrix cores idle).  Against the exact function: absolute error <= 7e-6, relative error <= 5e-5
// on the negative side down to x = -6, where gelu = -6e-9; beyond that the result saturates at that value (positive
// side: x - 6e-9).  NaN propagates through x + |x|.  The stand-alone eltwise kernel uses erff.
__device__ __forceinline__ float ttm_gelu_fast(float x) {
  const float u = fminf(fabsf(x), 6.0f);
  float p = fmaf(2.299055450e-05f, u, -6.110930699e-04f);
  p = fmaf(p, u, 7.195388433e-03f);
  p = fmaf(p, u, -5.118424445e-02f);
  p = fmaf(p, u, -4.612746239e-01f);
  p = fmaf(p, u, -1.150171638e+00f);
  p = fmaf(p, u, -6.547099474e-05f);
  const float q2 = __builtin_amdgcn_exp2f(p);   // 2 Q(u)
  return 0.5f * fmaf(-u, q2, x + fabsf(x));
}

__device__ __forceinline__ float ttm_gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }
__device__ __forceinline__ float ttm_sigmoid(float x) { return __frcp_rn(1.0f + __expf(-x)); }
__device__ __forceinline__ float ttm_silu(float x) { return x * ttm_sigmoid(x); }
