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

#include <algorithm>
#include <vector>

#include "common.h"

namespace im {
namespace {

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// One workgroup of two wavefronts per world; with 4 nentry + 2 nentry + 4 nmuscle bytes of LDS
// sixteen and more of them fit a CU, so 4096 worlds are all resident at once.  A and the
// muscle of every term are first brought into LDS in the order the rows consume them (every
// lane busy, twelve terms' look-ups in flight per lane), the force row as it is; then lane j of
// the first wavefront runs row j's chain of fused multiply-adds over consecutive LDS words.
// Same terms, same order per row as the reference kernel.
__global__ __launch_bounds__(128) void muscle_project_kernel(
    const float *__restrict__ moment, int64_t ldm, const float *__restrict__ force, int64_t ldf,
    const int32_t *__restrict__ offsets, const int32_t *__restrict__ entry_idx,
    const int32_t *__restrict__ entry_muscle, int nentry, int nmuscle, int ntorque, int root,
    float *__restrict__ qfrc, int64_t ldq, int nworld) {
  extern __shared__ float lds[];
  constexpr int NT = 128, UN = 12;
  const int tid = threadIdx.x;
  const int64_t w = blockIdx.x;
  float *av = lds;                                      // [nentry] A[entry_idx[s]]
  float *fs = av + nentry;                              // [nmuscle] the world's forces
  unsigned short *ms = (unsigned short *)(fs + nmuscle);  // [nentry] entry_muscle[entry_idx[s]]
  const float *mw = moment + w * ldm, *fw = force + w * ldf;
  // Every array is read from memory in its own order (coalesced); the permutation into the
  // rows' order goes through LDS, in place: gather into registers, barrier, write back.
  for (int i = tid; i < nmuscle; i += NT) fs[i] = fw[i];
  if (nentry <= UN * NT) {
    int e[UN], m[UN];
    float x[UN];
#pragma unroll
    for (int k = 0; k < UN; ++k) {
      const int i = tid + NT * k < nentry ? tid + NT * k : nentry - 1;
      e[k] = entry_idx[i];
      m[k] = entry_muscle[i];
      x[k] = mw[i];
    }
#pragma unroll
    for (int k = 0; k < UN; ++k)
      if (tid + NT * k < nentry) {
        av[tid + NT * k] = x[k];
        ms[tid + NT * k] = (unsigned short)m[k];
      }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < UN; ++k) {
      x[k] = av[e[k]];
      m[k] = ms[e[k]];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < UN; ++k)
      if (tid + NT * k < nentry) {
        av[tid + NT * k] = x[k];
        ms[tid + NT * k] = (unsigned short)m[k];
      }
  } else {
    // more entries than one trip holds: gathered from memory, twelve look-ups in flight per lane
    for (int s0 = tid; s0 < nentry; s0 += UN * NT) {
      int e[UN], m[UN];
      float x[UN];
#pragma unroll
      for (int k = 0; k < UN; ++k) e[k] = entry_idx[s0 + NT * k < nentry ? s0 + NT * k : nentry - 1];
#pragma unroll
      for (int k = 0; k < UN; ++k) {
        m[k] = entry_muscle[e[k]];
        x[k] = mw[e[k]];
      }
#pragma unroll
      for (int k = 0; k < UN; ++k)
        if (s0 + NT * k < nentry) {
          av[s0 + NT * k] = x[k];
          ms[s0 + NT * k] = (unsigned short)m[k];
        }
    }
  }
  __syncthreads();
  for (int j = tid; j < ntorque; j += NT) {
    float total = 0.0f;
    const int e1 = offsets[j + 1];
    int s = offsets[j];
    for (; s + 3 < e1; s += 4) {  // four terms' operands read before the first is used
      const float a0 = av[s], a1 = av[s + 1], a2 = av[s + 2], a3 = av[s + 3];
      const float f0 = fs[ms[s]], f1 = fs[ms[s + 1]], f2 = fs[ms[s + 2]], f3 = fs[ms[s + 3]];
      total = fma_(a0, f0, total);
      total = fma_(a1, f1, total);
      total = fma_(a2, f2, total);
      total = fma_(a3, f3, total);
    }
    for (; s < e1; ++s) total = fma_(av[s], fs[ms[s]], total);
    qfrc[w * ldq + root + j] = total;
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
  for (int e0 = lane; e0 < nentry; e0 += 8 * width) {  // eight entries' loads in flight per lane
    float v[8], sl[8];
    int mu[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int e = e0 + k * width < nentry ? e0 + k * width : nentry - 1;
      v[k] = moment[w * ldm + e];
      mu[k] = entry_muscle[e];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) sl[k] = slope[w * lds_ + mu[k]];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int e = e0 + k * width;
      if (e < nentry) {
        m[e] = v[k];
        weighted[e] = sl[k] * v[k];
      }
    }
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
    float *q = qderiv + w * ldq + elem_ids[slot];
    const float q0 = *q;  // requested before the sum, used after it
    for (int c = chunk_offsets[slot]; c < c1; ++c) acc = acc + partial[c];
    *q = fma_(timestep, acc, q0);
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
  if (nentry == 0) return IM_ERR_ARG;  // entry indices are clamped to nentry - 1
  if (!moment || !force || !torque_entry_offsets || !torque_entry_idx || !entry_muscle || !qfrc) return IM_ERR_ARG;
  if (ld_moment < nentry || ld_force < nmuscle || ld_qfrc < root_dof_count + ntorque) return IM_ERR_STRIDE;
  if (nmuscle > 65535) return IM_ERR_UNSUPPORTED;  // muscle ids travel as 16 bits
  const size_t lds_bytes = sizeof(float) * ((size_t)nentry + nmuscle) + 2 * (((size_t)nentry + 1) & ~(size_t)1);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::muscle_project_kernel, dim3(nworld), dim3(128), lds_bytes, (hipStream_t)stream,
                     moment, ld_moment, force, ld_force, torque_entry_offsets, torque_entry_idx, entry_muscle,
                     nentry, nmuscle, ntorque, root_dof_count, qfrc, ld_qfrc, nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_muscle_gather_tables(const int32_t *pair_elem_id, const int32_t *pair_entry_i, const int32_t *pair_entry_j,
                            int npair, int nentry, int32_t *elem_ids, int32_t *chunk_offsets, int32_t *chunk_pairs,
                            int *nelem, int *chunk_count) {
  if (npair < 0 || nentry < 0 || !nelem || !chunk_count || (npair > 0 && !pair_elem_id)) return IM_ERR_ARG;
  if (nentry >= 0x7FFF) return IM_ERR_UNSUPPORTED;  // two entry indices share one int32
  // pairs in the order of their M element, ties in list order
  std::vector<int> order(npair);
  for (int q = 0; q < npair; ++q) order[q] = q;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return pair_elem_id[a] < pair_elem_id[b]; });
  // first pass: elements and their chunks of 16 pairs
  int elems = 0, chunks = 0;
  for (int q = 0; q < npair;) {
    int end = q;
    while (end < npair && pair_elem_id[order[end]] == pair_elem_id[order[q]]) ++end;
    if (elem_ids) elem_ids[elems] = pair_elem_id[order[q]];
    if (chunk_offsets) chunk_offsets[elems] = chunks;
    chunks += (end - q + 15) / 16;
    ++elems;
    q = end;
  }
  if (chunk_offsets) chunk_offsets[elems] = chunks;
  *nelem = elems;
  *chunk_count = chunks;
  if (!chunk_pairs) return IM_OK;
  if (!pair_entry_i || !pair_entry_j || !chunk_offsets) return IM_ERR_ARG;
  // second pass: pair k of chunk c at k * chunk_count + c, the padding names entry `nentry` twice
  for (size_t v = 0; v < (size_t)16 * chunks; ++v) chunk_pairs[v] = nentry | (nentry << 16);
  int slot = 0, rank = 0;
  for (int q = 0; q < npair; ++q) {
    if (q > 0 && pair_elem_id[order[q]] != pair_elem_id[order[q - 1]]) {
      ++slot;
      rank = 0;
    }
    const int i = pair_entry_i[order[q]], j = pair_entry_j[order[q]];
    if (i < 0 || j < 0 || i >= nentry || j >= nentry) return IM_ERR_ARG;
    chunk_pairs[(size_t)(rank % 16) * chunks + chunk_offsets[slot] + rank / 16] = i | (j << 16);
    ++rank;
  }
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
