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

// Copies per_block worlds' rows of `stride` floats into LDS, `fetch(world, k)` giving element
// k of a world's row.  Four elements per thread and trip, their loads issued before the first
// store (indices past the end are clamped, their values dropped).
template <typename Fetch>
__device__ __forceinline__ void stage_rows(float *lds, int per_block, int stride, int64_t w0,
                                           int nworld, Fetch fetch) {
  const int total = per_block * stride;
  for (int i0 = threadIdx.x; i0 < total; i0 += 4 * kThreads) {
    float r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * kThreads < total ? i0 + u * kThreads : total - 1;
      const int lw = i / stride, k = i - lw * stride;
      r[u] = fetch(w0 + lw < nworld ? w0 + lw : (int64_t)nworld - 1, k);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i0 + u * kThreads < total) lds[i0 + u * kThreads] = r[u];
  }
}

// ---- M v -----------------------------------------------------------------------------------
// T lanes per world (a power of two, 8..64): lane d of a world owns dofs d, d + T, ...
// The row tables sit in LDS beside the worlds' rows, one word col | madr << 16 per term: lanes
// of a wavefront read different rows, and such gathers cost a cache lookup per lane when they
// go to memory.
__global__ __launch_bounds__(kThreads) void mul_m_kernel(
    const float *__restrict__ M, int64_t ldm, int nM, const int32_t *__restrict__ rowadr,
    const int32_t *__restrict__ col, const int32_t *__restrict__ madr,
    const float *__restrict__ vec, int64_t ldv, const uint8_t *__restrict__ skip,
    float *__restrict__ out, int64_t ldo, int nv, int nworld, int lanes, int nterm) {
  extern __shared__ float lds[];
  const int per_block = kThreads / lanes;
  const int stride = nM + nv;
  const int64_t w0 = (int64_t)blockIdx.x * per_block;
  uint32_t *term = (uint32_t *)(lds + per_block * stride);  // [nterm]
  int *radr = (int *)(term + nterm);                         // [nv + 1]
  for (int k = threadIdx.x; k < nterm; k += kThreads) term[k] = (uint32_t)col[k] | (uint32_t)madr[k] << 16;
  for (int k = threadIdx.x; k <= nv; k += kThreads) radr[k] = rowadr[k];
  // a world's M and vec rows, one world after the other, loads coalesced over the block
  stage_rows(lds, per_block, stride, w0, nworld, [&](int64_t w, int k) {
    return k < nM ? M[w * ldm + k] : vec[w * ldv + (k - nM)];
  });
  __syncthreads();
  const int lw = threadIdx.x / lanes, lane = threadIdx.x & (lanes - 1);
  const int64_t w = w0 + lw;
  if (w >= nworld || (skip && skip[w])) return;
  const float *m = lds + lw * stride, *v = m + nM;
  for (int dof = lane; dof < nv; dof += lanes) {
    float value = 0.0f;
    const int end = radr[dof + 1];
    // four terms' operands at a time; a term past the row's end repeats the last one and is
    // dropped
    for (int k = radr[dof]; k < end; k += 4) {
      float a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t t = term[k + u < end ? k + u : end - 1];
        a[u] = m[t >> 16];
        b[u] = v[t & 0xffffu];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) value = k + u < end ? fmaf(a[u], b[u], value) : value;
    }
    out[w * ldo + dof] = value;
  }
}

// ---- bottom-up accumulation -----------------------------------------------------------------
// The level tables as the folds read them, in LDS: tb[c] = level_bodies[c],
// tb[nbody + c] = that body's parent (-1 for body 0, which is never a child), and behind them
// the levels + 1 level offsets.
__device__ __forceinline__ void stage_tree(int *tb, const int32_t *__restrict__ parent,
                                           const int32_t *__restrict__ bodies,
                                           const int32_t *__restrict__ offsets, int nbody,
                                           int levels) {
  for (int c = threadIdx.x; c < nbody; c += kThreads) {
    const int body = bodies[c];
    tb[c] = body;
    tb[nbody + c] = body != 0 ? parent[body] : -1;
  }
  for (int l = threadIdx.x; l <= levels; l += kThreads) tb[2 * nbody + l] = offsets[l];
}
__host__ __device__ inline size_t tree_words(int nbody, int levels) {
  return 2 * (size_t)nbody + (size_t)levels + 1;
}

// Folds one level's bodies into their parents: one writer per (parent, component), the
// children added in the order the level lists them.  Four children's parents and values are
// read before the first is added; one that belongs to another parent is dropped.
__device__ __forceinline__ void fold_level(float *values, int components, float inv_components,
                                           const int *tb, int nbody, int pstart, int start,
                                           int end, bool skip_root_parent, int lane, int lanes) {
  const int pcount = start - pstart;
  for (int entry = lane; entry < pcount * components; entry += lanes) {
    // entry / components through the reciprocal: exact while entry stays below 2^20
    const int pi = (int)(((float)entry + 0.5f) * inv_components);
    const int parent_id = tb[pstart + pi];
    const int component = entry - pi * components;
    if (skip_root_parent && parent_id == 0) continue;
    float value = values[parent_id * components + component];
    for (int c = start; c < end; c += 4) {
      int par[4];
      float x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int cc = c + u < end ? c + u : end - 1;
        par[u] = c + u < end ? tb[nbody + cc] : -2;
        x[u] = values[tb[cc] * components + component];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) value = par[u] == parent_id ? value + x[u] : value;
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
  int *tb = (int *)(lds + per_block * stride);
  stage_tree(tb, parent, bodies, offsets, nbody, levels);
  stage_rows(lds, per_block, stride, w0, nworld, [&](int64_t w, int k) { return values[w * ldw + k]; });
  __syncthreads();
  const int lw = threadIdx.x / lanes, lane = threadIdx.x & (lanes - 1);
  float *mine = lds + lw * stride;
  const int *loff = tb + 2 * nbody;
  const float inv_components = 1.0f / (float)components;
  // every wavefront of the block walks the same levels, so the barriers are uniform
  for (int level = levels - 1; level > 0; --level) {
    fold_level(mine, components, inv_components, tb, nbody, loff[level - 1], loff[level],
               loff[level + 1], skip_root_parent != 0, lane, lanes);
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
  int *tb = (int *)(lds + per_block * stride);
  stage_tree(tb, a.parent, a.bodies, a.offsets, a.nbody, a.levels);
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
    fold_level(mine, 6, 1.0f / 6.0f, tb, a.nbody, tb[2 * a.nbody + level - 1], tb[2 * a.nbody + level],
               tb[2 * a.nbody + level + 1], false, lane, a.lanes);
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
int fit_lanes(int lanes, size_t floats_per_world, size_t shared_words = 0) {
  while (lanes <= kThreads && ((kThreads / lanes) * floats_per_world + shared_words) * 4 > kLdsLimit)
    lanes *= 2;
  return lanes <= kThreads ? lanes : 0;
}

}  // namespace
}  // namespace im

using namespace im;

extern "C" int im_mul_m_sparse(const float *M, int64_t ld_M, int nM, const int32_t *mulm_rowadr,
                               const int32_t *mulm_col, const int32_t *mulm_madr, int nterm,
                               const float *vec, int64_t ld_vec, const uint8_t *skip_world,
                               float *out, int64_t ld_out, int nv, int nworld, void *stream) {
  if (nworld < 0 || nv < 0 || nM < 0 || nterm < 0) return IM_ERR_ARG;
  if (nworld == 0 || nv == 0) return IM_OK;
  if (!M || !mulm_rowadr || !mulm_col || !mulm_madr || !vec || !out) return IM_ERR_ARG;
  if (ld_M < nM || ld_vec < nv || ld_out < nv) return IM_ERR_STRIDE;
  const size_t shared_words = (size_t)nterm + nv + 1;
  if (nM >= 65536 || nv >= 65536) return IM_ERR_UNSUPPORTED;  // a term is packed into 16 + 16 bits
  const int lanes = fit_lanes(lanes_for(nv), (size_t)nM + nv, shared_words);
  if (!lanes) return IM_ERR_UNSUPPORTED;
  const int per_block = kThreads / lanes;
  const size_t lds_bytes = ((size_t)per_block * ((size_t)nM + nv) + shared_words) * 4;
  hipLaunchKernelGGL(mul_m_kernel, dim3((unsigned)((nworld + per_block - 1) / per_block)),
                     dim3(kThreads), lds_bytes, (hipStream_t)stream, M, ld_M, nM, mulm_rowadr,
                     mulm_col, mulm_madr, vec, ld_vec, skip_world, out, ld_out, nv, nworld, lanes, nterm);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_tree_accumulate(const int32_t *body_parentid, const int32_t *level_bodies,
                                  const int32_t *level_offsets, int levels, int components,
                                  int skip_root_parent, float *values, int64_t ld_world,
                                  int nbody, int nworld, void *stream) {
  if (nworld < 0 || nbody < 0 || levels < 0 || components < 0 || levels > nbody) return IM_ERR_ARG;
  if (nworld == 0 || nbody == 0 || components == 0 || levels <= 1) return IM_OK;
  if (!body_parentid || !level_bodies || !level_offsets || !values) return IM_ERR_ARG;
  if (ld_world < (int64_t)nbody * components) return IM_ERR_STRIDE;
  const int lanes = fit_lanes(lanes_for(nbody * components), (size_t)nbody * components, tree_words(nbody, levels));
  if (!lanes) return IM_ERR_UNSUPPORTED;
  const int per_block = kThreads / lanes;
  const size_t lds_bytes = ((size_t)per_block * nbody * components + tree_words(nbody, levels)) * 4;
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
      topology->body_count < 0 || topology->levels < 0 || topology->levels > topology->body_count)
    return IM_ERR_ARG;
  if (nworld == 0 || torque_dim == 0) return IM_OK;
  const int nbody = topology->body_count;
  if (!wrenches || !wrenches->body_force || !wrenches->body_torque || !wrenches->xipos ||
      !wrenches->subtree_com || !wrenches->cdof || !wrenches->body_rootid || !mean ||
      !topology->dof_bodyid || !topology->body_parentid || !topology->level_bodies ||
      !topology->level_offsets || nbody == 0)
    return IM_ERR_ARG;
  if (ld_mean < (int64_t)output_dof_offset + torque_dim) return IM_ERR_STRIDE;
  const int lanes = fit_lanes(lanes_for(6 * nbody), (size_t)6 * nbody, tree_words(nbody, topology->levels));
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
                     ((size_t)per_block * 6 * nbody + tree_words(nbody, topology->levels)) * 4, (hipStream_t)stream, a);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
