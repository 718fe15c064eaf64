// Steps either side of the solve that walk a world's small trees: the product M v over M's
// tree CSR, the bottom-up accumulation of per-body quantities, and the projection of body
// wrenches onto joint torques.  A world's data is a few hundred bytes to a few KB: several
// worlds share a workgroup, each world's rows travel through LDS with coalesced loads, and the
// level loops run there.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace im {
namespace {

constexpr int kThreads = 256;
constexpr size_t kLdsLimit = 64 * 1024;

// ---- M v -----------------------------------------------------------------------------------
// T lanes per world (a power of two, 8..64): lane d of a world owns dofs d, d + T, ...
__global__ __launch_bounds__(kThreads) void mul_m_kernel(
    const float *__restrict__ M, int64_t ldm, int nM, const int32_t *__restrict__ rowadr,
    const int32_t *__restrict__ col, const int32_t *__restrict__ madr,
    const float *__restrict__ vec, int64_t ldv, const uint8_t *__restrict__ skip,
    float *__restrict__ out, int64_t ldo, int nv, int nworld, int lanes) {
  extern __shared__ float lds[];
  const int per_block = kThreads / lanes;
  const int stride = nM + nv;
  const int64_t w0 = (int64_t)blockIdx.x * per_block;
  // a world's M and vec rows, one world after the other, loads coalesced over the block
  for (int i = threadIdx.x; i < per_block * stride; i += kThreads) {
    const int lw = i / stride, k = i - lw * stride;
    const int64_t w = w0 + lw < nworld ? w0 + lw : nworld - 1;
    lds[i] = k < nM ? M[w * ldm + k] : vec[w * ldv + (k - nM)];
  }
  __syncthreads();
  const int lw = threadIdx.x / lanes, lane = threadIdx.x & (lanes - 1);
  const int64_t w = w0 + lw;
  if (w >= nworld || (skip && skip[w])) return;
  const float *m = lds + lw * stride, *v = m + nM;
  for (int dof = lane; dof < nv; dof += lanes) {
    float value = 0.0f;
    for (int k = rowadr[dof]; k < rowadr[dof + 1]; ++k) value = fmaf(m[madr[k]], v[col[k]], value);
    out[w * ldo + dof] = value;
  }
}

// ---- bottom-up accumulation -----------------------------------------------------------------
// Folds one level's bodies into their parents: one writer per (parent, component), the
// children added in the order the level lists them.
__device__ __forceinline__ void fold_level(float *values, int components,
                                           const int32_t *__restrict__ parent,
                                           const int32_t *__restrict__ bodies, int pstart,
                                           int start, int end, bool skip_root_parent, int lane,
                                           int lanes) {
  const int pcount = start - pstart;
  for (int entry = lane; entry < pcount * components; entry += lanes) {
    const int parent_id = bodies[pstart + entry / components];
    const int component = entry % components;
    if (skip_root_parent && parent_id == 0) continue;
    float value = values[parent_id * components + component];
    for (int c = start; c < end; ++c) {
      const int body = bodies[c];
      if (body != 0 && parent[body] == parent_id) value = value + values[body * components + component];
    }
    values[parent_id * components + component] = value;
  }
}

__global__ __launch_bounds__(kThreads) void tree_accumulate_kernel(
    const int32_t *__restrict__ parent, const int32_t *__restrict__ bodies,
    const int32_t *__restrict__ offsets, int levels, int components, int skip_root_parent,
    float *__restrict__ values, int64_t ldw, int nbody, int nworld, int lanes) {
  extern __shared__ float lds[];
  const int per_block = kThreads / lanes;
  const int stride = nbody * components;
  const int64_t w0 = (int64_t)blockIdx.x * per_block;
  for (int i = threadIdx.x; i < per_block * stride; i += kThreads) {
    const int lw = i / stride, k = i - lw * stride;
    const int64_t w = w0 + lw < nworld ? w0 + lw : nworld - 1;
    lds[i] = values[w * ldw + k];
  }
  __syncthreads();
  const int lw = threadIdx.x / lanes, lane = threadIdx.x & (lanes - 1);
  float *mine = lds + lw * stride;
  // every wavefront of the block walks the same levels, so the barriers are uniform
  for (int level = levels - 1; level > 0; --level) {
    fold_level(mine, components, parent, bodies, offsets[level - 1], offsets[level],
               offsets[level + 1], skip_root_parent != 0, lane, lanes);
    __syncthreads();
  }
  for (int i = threadIdx.x; i < per_block * stride; i += kThreads) {
    const int lw2 = i / stride, k = i - lw2 * stride;
    if (w0 + lw2 < nworld) values[(w0 + lw2) * ldw + k] = lds[i];
  }
}

// ---- body wrenches onto joint torques --------------------------------------------------------
struct WrenchArgs {
  const float *force, *torque, *xipos, *com, *cdof;
  int64_t ldf, ldt, ldx, ldc, ldd;
  const int32_t *rootid, *dof_body, *parent, *bodies, *offsets;
  int levels, nbody, root, ntorque, out_offset;
  float *mean;
  int64_t ldo;
  int nworld, lanes;
};

__global__ __launch_bounds__(kThreads) void project_wrenches_kernel(WrenchArgs a) {
  extern __shared__ float lds[];
  const int per_block = kThreads / a.lanes;
  const int stride = 6 * a.nbody;
  const int64_t w0 = (int64_t)blockIdx.x * per_block;
  // force and the moment about the root's subtree centre, per body
  for (int i = threadIdx.x; i < per_block * a.nbody; i += kThreads) {
    const int lw = i / a.nbody, body = i - lw * a.nbody;
    const int64_t w = w0 + lw < a.nworld ? w0 + lw : a.nworld - 1;
    const float *f = a.force + w * a.ldf + 3 * body, *t = a.torque + w * a.ldt + 3 * body;
    const float *x = a.xipos + w * a.ldx + 3 * body, *c = a.com + w * a.ldc + 3 * a.rootid[body];
    const float fx = f[0], fy = f[1], fz = f[2];
    const float rx = x[0] - c[0], ry = x[1] - c[1], rz = x[2] - c[2];
    float *o = lds + lw * stride + 6 * body;
    o[0] = fx;
    o[1] = fy;
    o[2] = fz;
    o[3] = t[0] + (ry * fz - rz * fy);
    o[4] = t[1] + (rz * fx - rx * fz);
    o[5] = t[2] + (rx * fy - ry * fx);
  }
  __syncthreads();
  const int lw = threadIdx.x / a.lanes, lane = threadIdx.x & (a.lanes - 1);
  float *mine = lds + lw * stride;
  for (int level = a.levels - 1; level > 0; --level) {
    fold_level(mine, 6, a.parent, a.bodies, a.offsets[level - 1], a.offsets[level],
               a.offsets[level + 1], false, lane, a.lanes);
    __syncthreads();
  }
  const int64_t w = w0 + lw;
  if (w >= a.nworld) return;
  for (int j = lane; j < a.ntorque; j += a.lanes) {
    const int dof = j + a.root;
    const float *v = mine + 6 * a.dof_body[dof];
    const float *cd = a.cdof + w * a.ldd + 6 * (int64_t)dof;
    const float lin = cd[3] * v[0] + cd[4] * v[1] + cd[5] * v[2];
    const float ang = cd[0] * v[3] + cd[1] * v[4] + cd[2] * v[5];
    a.mean[w * a.ldo + j + a.out_offset] = lin + ang;
  }
}

// Lanes per world: the smallest power of two in 8..64 that covers `work` items (64 beyond).
int lanes_for(int work) {
  int lanes = 8;
  while (lanes < 64 && lanes < work) lanes *= 2;
  return lanes;
}
// Widens the lane count until a block's worlds fit in LDS; 0 when one world alone does not.
int fit_lanes(int lanes, size_t floats_per_world) {
  while (lanes <= kThreads && (kThreads / lanes) * floats_per_world * 4 > kLdsLimit) lanes *= 2;
  return lanes <= kThreads ? lanes : 0;
}

}  // namespace
}  // namespace im

using namespace im;

extern "C" int im_mul_m_sparse(const float *M, int64_t ld_M, int nM, const int32_t *mulm_rowadr,
                               const int32_t *mulm_col, const int32_t *mulm_madr,
                               const float *vec, int64_t ld_vec, const uint8_t *skip_world,
                               float *out, int64_t ld_out, int nv, int nworld, void *stream) {
  if (nworld < 0 || nv < 0 || nM < 0) return IM_ERR_ARG;
  if (nworld == 0 || nv == 0) return IM_OK;
  if (!M || !mulm_rowadr || !mulm_col || !mulm_madr || !vec || !out) return IM_ERR_ARG;
  if (ld_M < nM || ld_vec < nv || ld_out < nv) return IM_ERR_STRIDE;
  const int lanes = fit_lanes(lanes_for(nv), (size_t)nM + nv);
  if (!lanes) return IM_ERR_UNSUPPORTED;
  const int per_block = kThreads / lanes;
  const size_t lds_bytes = (size_t)per_block * ((size_t)nM + nv) * 4;
  hipLaunchKernelGGL(mul_m_kernel, dim3((unsigned)((nworld + per_block - 1) / per_block)),
                     dim3(kThreads), lds_bytes, (hipStream_t)stream, M, ld_M, nM, mulm_rowadr,
                     mulm_col, mulm_madr, vec, ld_vec, skip_world, out, ld_out, nv, nworld, lanes);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_tree_accumulate(const int32_t *body_parentid, const int32_t *level_bodies,
                                  const int32_t *level_offsets, int levels, int components,
                                  int skip_root_parent, float *values, int64_t ld_world,
                                  int nbody, int nworld, void *stream) {
  if (nworld < 0 || nbody < 0 || levels < 0 || components < 0) return IM_ERR_ARG;
  if (nworld == 0 || nbody == 0 || components == 0 || levels <= 1) return IM_OK;
  if (!body_parentid || !level_bodies || !level_offsets || !values) return IM_ERR_ARG;
  if (ld_world < (int64_t)nbody * components) return IM_ERR_STRIDE;
  const int lanes = fit_lanes(lanes_for(nbody * components), (size_t)nbody * components);
  if (!lanes) return IM_ERR_UNSUPPORTED;
  const int per_block = kThreads / lanes;
  const size_t lds_bytes = (size_t)per_block * nbody * components * 4;
  hipLaunchKernelGGL(tree_accumulate_kernel,
                     dim3((unsigned)((nworld + per_block - 1) / per_block)), dim3(kThreads),
                     lds_bytes, (hipStream_t)stream, body_parentid, level_bodies, level_offsets,
                     levels, components, skip_root_parent, values, ld_world, nbody, nworld, lanes);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_project_body_wrenches(const im_body_wrenches *wrenches,
                                        const im_wrench_topology *topology, int root_dof_count,
                                        int torque_dim, int output_dof_offset, float *mean,
                                        int64_t ld_mean, int nworld, void *stream) {
  if (nworld < 0 || torque_dim < 0 || root_dof_count < 0 || output_dof_offset < 0 || !topology ||
      topology->body_count < 0 || topology->levels < 0)
    return IM_ERR_ARG;
  if (nworld == 0 || torque_dim == 0) return IM_OK;
  const int nbody = topology->body_count;
  if (!wrenches || !wrenches->body_force || !wrenches->body_torque || !wrenches->xipos ||
      !wrenches->subtree_com || !wrenches->cdof || !wrenches->body_rootid || !mean ||
      !topology->dof_bodyid || !topology->body_parentid || !topology->level_bodies ||
      !topology->level_offsets || nbody == 0)
    return IM_ERR_ARG;
  if (ld_mean < (int64_t)output_dof_offset + torque_dim) return IM_ERR_STRIDE;
  const int lanes = fit_lanes(lanes_for(6 * nbody), (size_t)6 * nbody);
  if (!lanes) return IM_ERR_UNSUPPORTED;
  const int per_block = kThreads / lanes;
  WrenchArgs a{wrenches->body_force, wrenches->body_torque, wrenches->xipos,
               wrenches->subtree_com, wrenches->cdof, wrenches->ld_body_force,
               wrenches->ld_body_torque, wrenches->ld_xipos, wrenches->ld_subtree_com,
               wrenches->ld_cdof, wrenches->body_rootid, topology->dof_bodyid,
               topology->body_parentid, topology->level_bodies, topology->level_offsets,
               topology->levels, nbody, root_dof_count, torque_dim, output_dof_offset, mean,
               ld_mean, nworld, lanes};
  hipLaunchKernelGGL(project_wrenches_kernel,
                     dim3((unsigned)((nworld + per_block - 1) / per_block)), dim3(kThreads),
                     (size_t)per_block * 6 * nbody * 4, (hipStream_t)stream, a);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
