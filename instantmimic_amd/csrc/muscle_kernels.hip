// Muscle moment-arm contractions for gfx950.
//
//   tau[w, root + j]  = sum over the entries e of torque dof j (torque-sorted order) of
//                       A[w, e] * f[w, muscle(e)]
//     reference: src/instantmimic/muscle/muscle_qfrc_projector.py:2941-2961
//   qDeriv[w, elem]  += h * sum over the element's chunks of 16 pairs, in order, of
//                       (s[w, muscle(i)] * A[w, i]) * A[w, j]
//     reference: muscle_qfrc_projector.py:736-774 (one block per world, no atomics)
//
// Both are bandwidth bound: a world's moment row (a few KB) is read once, staged in
// LDS, and gathered from there.  Summation order and fused multiply-adds follow the
// reference (Warp lowers `total += a * b` to one fma under NVRTC's default contraction).
#include <hip/hip_runtime.h>

#include "common.h"

namespace im {
namespace {

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// One wavefront per world, four worlds per workgroup.
__global__ __launch_bounds__(256) void muscle_project_kernel(
    const float *__restrict__ moment, int64_t ldm, const float *__restrict__ force, int64_t ldf,
    const int32_t *__restrict__ offsets, const int32_t *__restrict__ entry_idx,
    const int32_t *__restrict__ entry_muscle, int nentry, int nmuscle, int ntorque, int root,
    float *__restrict__ qfrc, int64_t ldq, int nworld) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int w = blockIdx.x * 4 + wv;
  if (w >= nworld) return;  // wave-uniform; no workgroup barrier below
  float *prod = lds + (size_t)wv * nentry;  // A[e] and f[muscle(e)] side by side is not needed:
  const float *mw = moment + (int64_t)w * ldm, *fw = force + (int64_t)w * ldf;
  // stage A[w, :] (coalesced); forces are gathered straight from the row (L1 resident)
  for (int e = lane; e < nentry; e += 64) prod[e] = mw[e];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (int j = lane; j < ntorque; j += 64) {
    float total = 0.0f;
    const int e1 = offsets[j + 1];
    for (int s = offsets[j]; s < e1; ++s) {
      const int e = entry_idx[s];
      total = fma_(prod[e], fw[entry_muscle[e]], total);
    }
    qfrc[(int64_t)w * ldq + root + j] = total;
  }
}

// One workgroup of 256 per world.
__global__ __launch_bounds__(256) void muscle_gather_kernel(
    const float *__restrict__ moment, int64_t ldm, const float *__restrict__ slope, int64_t lds_,
    const int32_t *__restrict__ entry_muscle, int nentry, const int32_t *__restrict__ elem_ids,
    int nelem, const int32_t *__restrict__ chunk_offsets, const int32_t *__restrict__ chunk_pairs,
    int chunk_count, float timestep, float *__restrict__ qderiv, int64_t ldq) {
  extern __shared__ float lds[];
  float *m = lds;                      // [nentry + 1]
  float *weighted = m + nentry + 1;    // [nentry + 1]
  float *partial = weighted + nentry + 1;  // [chunk_count]
  const int lane = threadIdx.x, width = blockDim.x;
  const int64_t w = blockIdx.x;
  for (int e = lane; e < nentry; e += width) {
    const float v = moment[w * ldm + e];
    m[e] = v;
    weighted[e] = slope[w * lds_ + entry_muscle[e]] * v;
  }
  if (lane == 0) {
    m[nentry] = 0.0f;
    weighted[nentry] = 0.0f;
  }
  __syncthreads();
  for (int c = lane; c < chunk_count; c += width) {
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int packed = chunk_pairs[(size_t)k * chunk_count + c];
      total = fma_(weighted[packed & 0xFFFF], m[packed >> 16], total);
    }
    partial[c] = total;
  }
  __syncthreads();
  for (int slot = lane; slot < nelem; slot += width) {
    float acc = 0.0f;
    const int c1 = chunk_offsets[slot + 1];
    for (int c = chunk_offsets[slot]; c < c1; ++c) acc = acc + partial[c];
    float *q = qderiv + w * ldq + elem_ids[slot];
    *q = fma_(timestep, acc, *q);
  }
}

}  // namespace
}  // namespace im

extern "C" {

int im_muscle_project(const float *moment, int64_t ld_moment, const float *force, int64_t ld_force,
                      const int32_t *torque_entry_offsets, const int32_t *torque_entry_idx,
                      const int32_t *entry_muscle, int nentry, int nmuscle, int ntorque,
                      int root_dof_count, float *qfrc, int64_t ld_qfrc, int nworld, void *stream) {
  if (nworld < 0 || nentry < 0 || ntorque < 0) return IM_ERR_ARG;
  if (nworld == 0 || ntorque == 0) return IM_OK;
  if (!moment || !force || !torque_entry_offsets || !torque_entry_idx || !entry_muscle || !qfrc) return IM_ERR_ARG;
  if (ld_moment < nentry || ld_force < nmuscle || ld_qfrc < root_dof_count + ntorque) return IM_ERR_STRIDE;
  const size_t lds_bytes = (size_t)4 * nentry * sizeof(float);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::muscle_project_kernel, dim3((nworld + 3) / 4), dim3(256), lds_bytes, (hipStream_t)stream,
                     moment, ld_moment, force, ld_force, torque_entry_offsets, torque_entry_idx, entry_muscle,
                     nentry, nmuscle, ntorque, root_dof_count, qfrc, ld_qfrc, nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_muscle_implicit_gather(const float *moment, int64_t ld_moment, const float *slope, int64_t ld_slope,
                              const int32_t *entry_muscle, int nentry, const int32_t *elem_ids, int nelem,
                              const int32_t *chunk_offsets, const int32_t *chunk_pairs, int chunk_count,
                              float timestep, float *qderiv, int64_t ld_qderiv, int nworld, void *stream) {
  if (nworld < 0 || nentry < 0 || nelem < 0 || chunk_count < 0) return IM_ERR_ARG;
  if (nworld == 0 || nelem == 0) return IM_OK;
  if (!moment || !slope || !entry_muscle || !elem_ids || !chunk_offsets || !chunk_pairs || !qderiv) return IM_ERR_ARG;
  if (nentry >= 0x7FFF) return IM_ERR_UNSUPPORTED;  // two entry indices share one int32
  if (ld_moment < nentry) return IM_ERR_STRIDE;
  const size_t lds_bytes = sizeof(float) * (2 * ((size_t)nentry + 1) + chunk_count);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::muscle_gather_kernel, dim3(nworld), dim3(256), lds_bytes, (hipStream_t)stream, moment,
                     ld_moment, slope, ld_slope, entry_muscle, nentry, elem_ids, nelem, chunk_offsets, chunk_pairs,
                     chunk_count, timestep, qderiv, ld_qderiv);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
