// Pivot arithmetic shared by the Cholesky kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace im {
namespace {

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// Square root of a pivot and the reciprocal of that root, IEEE-rounded, without what the compiler
// adds for tiny, huge and special inputs, and in few dependent steps: the chain from one pivot to
// the next bounds the factor.  With s = v_sqrt_f32(x) and y = v_rsq_f32(x) (both within an ulp),
// d = fma(fma(-s, s, x), y / 2, s) is the rounded root (the exact residual times the root's
// derivative); rinv is v_rcp_f32(d) plus one Newton step.  Both equal sqrtf(x) and
// 1.0f / sqrtf(x) bit for bit for every x in [2^-96, inf) (checked over all such floats by
// im_check_pivot_sqrt; a reciprocal seeded from y or from 1 / s instead is one ulp off for a
// few hundred of them); other inputs take the library forms.
__device__ __forceinline__ bool pivot_in_range(float x) { return x >= 0x1p-96f && x < __builtin_inff(); }
__device__ __forceinline__ void pivot_sqrt_rcp_fast(float x, float &d, float &rinv) {
  const float s = __builtin_amdgcn_sqrtf(x);
  const float y = __builtin_amdgcn_rsqf(x);
  d = fma_(fma_(-s, s, x), 0.5f * y, s);
  const float r = __builtin_amdgcn_rcpf(d);
  rinv = fma_(fma_(-d, r, 1.0f), r, r);
}
// d = sqrtf(x), rinv = 1.0f / d; `checked`: the lanes whose x is a pivot (the others may hold anything)
__device__ __forceinline__ void pivot_sqrt_rcp(float x, bool checked, float &d, float &rinv) {
  pivot_sqrt_rcp_fast(x, d, rinv);
  if (__builtin_expect(__any(checked && !pivot_in_range(x)), 0)) {
    d = sqrtf(x);
    rinv = 1.0f / d;
  }
}

}  // namespace
}  // namespace im
