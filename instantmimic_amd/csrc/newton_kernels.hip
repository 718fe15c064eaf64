// The parts of a Newton iteration around the linear solve that the reference writes itself
// (src/instantmimic/utils/mjw_kernels/newton_stages.py, newton_fusion.py): the gradient, the
// line search's J v, the step along the search direction, the list of the rows whose state
// changed, and the convergence test.  Each runs for all worlds in one launch; the scalar search
// for the step length and the evaluation of the constraints' new states sit between them in the
// reference's loop and are upstream code.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace im {
namespace {

constexpr int kThreads = 256;
constexpr size_t kLdsLimit = 64 * 1024;

// ---- Newton gradient ---------------------------------------------------------------------------
// qfrc_constraint = J' efc_force, grad = Ma - qfrc_smooth - qfrc_constraint, grad . grad.
// L lanes per world (32 up to 32 dofs, else 64), a lane per dof, the rows of J streamed ROWS
// at a time (a row of J is contiguous over the lanes); the nonzero entries of efc_force sit in
// LDS with their row numbers, and only those rows of J are read.
struct GradArgs {
  const int32_t *nefc;
  const float *J, *force, *smooth, *Ma, *alpha;
  const int32_t *changed;
  const uint8_t *done;
  float *qc, *grad, *grad_dot, *decrement, *scale;
  uint8_t *unchanged;
  int64_t ldf, lds_, ldm, ldq, ldg;
  int njmax, nv, block, nworld, lanes;
};

template <int ROWS>
__global__ __launch_bounds__(kThreads) void newton_gradient_kernel(GradArgs a) {
  extern __shared__ float lds[];
  const int L = a.lanes, per_block = kThreads / L;
  const int lw = threadIdx.x / L, lane = threadIdx.x & (L - 1);
  const int64_t w_raw = (int64_t)blockIdx.x * per_block + lw;
  const bool live = w_raw < a.nworld;
  const int64_t w = live ? w_raw : (int64_t)a.nworld - 1;
  // [njmax] the nonzero forces, [njmax] their rows, then [nv] grad, then [64] lane sums
  float *f = lds + lw * (2 * a.njmax + a.nv + 64);
  int *rowl = (int *)(f + a.njmax);
  float *gl = f + 2 * a.njmax, *part = gl + a.nv;
  const bool done = a.done && a.done[w] != 0;
  const bool changed = !a.changed || a.changed[w] != 0;
  int nefc = a.nefc ? a.nefc[w] : a.njmax;
  nefc = nefc < a.njmax ? nefc : a.njmax;
  nefc = nefc > 0 ? nefc : 0;
  const bool work = !done && changed;
  // A row whose force is zero (every satisfied constraint) adds nothing to J' f and is not read:
  // the world's lanes list the other rows in order, by ballot.
  int cnt = 0;
  if (work) {
    const int shift = (threadIdx.x & 63) & ~(L - 1);  // where the world's lanes start in the wavefront
    const uint64_t group = L == 64 ? ~0ull : 0xFFFFFFFFull;
    for (int r0 = 0; r0 < nefc; r0 += L) {
      const int r = r0 + lane;
      const float v = r < nefc ? a.force[w * a.ldf + r] : 0.0f;
      const uint64_t mask = (__ballot(v != 0.0f) >> shift) & group;
      if (v != 0.0f) {
        const int pos = cnt + __popcll(mask & ((1ull << lane) - 1));
        f[pos] = v;
        rowl[pos] = r;
      }
      cnt += __popcll(mask);
    }
  }
  __syncthreads();  // every thread of the block reaches the barriers: nothing above returns
  if (work) {
    const float *Jw = a.J + w * (int64_t)a.njmax * a.nv;
    for (int dof = lane; dof < a.nv; dof += L) {
      const float ma = a.Ma[w * a.ldm + dof], sm = a.smooth[w * a.lds_ + dof];  // on their way beside the rows of J
      float sum = 0.0f;
      for (int p0 = 0; p0 < cnt; p0 += ROWS) {
        float jv[ROWS];
#pragma unroll
        for (int u = 0; u < ROWS; ++u) jv[u] = Jw[(int64_t)rowl[p0 + u < cnt ? p0 + u : cnt - 1] * a.nv + dof];
#pragma unroll
        for (int u = 0; u < ROWS; ++u) sum = p0 + u < cnt ? fmaf(jv[u], f[p0 + u], sum) : sum;
      }
      const float g = ma - sm - sum;
      if (live) {
        a.qc[w * a.ldq + dof] = sum;
        a.grad[w * a.ldg + dof] = g;
      }
      gl[dof] = g;
    }
  }
  __syncthreads();
  // grad . grad as a block of `block` lanes would sum it: lane `rank` adds its dofs rank,
  // rank + block, .. in order, 32 lanes fold in a shuffle-down tree, the folds are added in order
  if (work) {
    for (int rank = lane; rank < a.block; rank += L) {
      float p = 0.0f;
      for (int dof = rank; dof < a.nv; dof += a.block) p = fmaf(gl[dof], gl[dof], p);
      part[rank] = p;
    }
  }
  __syncthreads();
  if (work && lane < 32) {
    float total = 0.0f;
    for (int wv = 0; wv < a.block / 32; ++wv) {
      float v = part[32 * wv + lane];
      for (int off = 16; off > 0; off >>= 1) v = v + __shfl_down(v, off, 32);
      total = total + v;
    }
    if (lane == 0 && live) {
      a.grad_dot[w] = total;
      a.decrement[w] = 0.0f;
      a.scale[w] = 1.0f;
    }
  }
  if (lane == 0 && live) {
    a.unchanged[w] = (done || !changed) ? 1 : 0;
    if (!done && !changed) {
      const float sigma = a.scale[w], new_sigma = sigma - a.alpha[w];
      float ratio = 0.0f;
      if (sigma != 0.0f) ratio = new_sigma / sigma;
      const float ratio_sq = ratio * ratio;
      a.grad_dot[w] = a.grad_dot[w] * ratio_sq;
      a.decrement[w] = a.decrement[w] * ratio_sq;
      a.scale[w] = new_sigma;
    }
  }
}

// ---- J v per constraint row ------------------------------------------------------------------
// One wavefront takes 64 rows of one world: the rows (contiguous in memory) travel through LDS
// with coalesced loads, U in flight per lane (the launcher picks U so that one batch covers the
// 64 rows: a wavefront then waits for memory once), and a lane then walks its own row (rows sit
// an odd number of words apart in LDS).  Up to 50 dofs the sum is one chain of fused
// multiply-adds; beyond, partial sums over 20 dofs each are added with a rounding of their own.
template <int U>
__global__ __launch_bounds__(64) void newton_jv_kernel(
    const float *__restrict__ J, int njmax, const int32_t *__restrict__ nefc_p,
    const float *__restrict__ search, int64_t lds_, const uint8_t *__restrict__ skip,
    float *__restrict__ jv, int64_t ldj, int nv, int chunks, const float *__restrict__ minus, int64_t ldm) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x;
  const int64_t w = blockIdx.x / chunks;
  const int r0 = (int)(blockIdx.x % chunks) * 64;
  if (skip && skip[w]) return;  // the whole wavefront: no barrier is left behind
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  if (r0 >= nefc) return;
  const int rows = nefc - r0 < 64 ? nefc - r0 : 64;
  const int stride = nv | 1;
  float *sv = lds + 64 * stride;  // [nv] the search direction
  const float *src = J + (w * njmax + r0) * (int64_t)nv;
  const int total = rows * nv;
  const float inv_nv = 1.0f / (float)nv;
  for (int i0 = lane; i0 < total; i0 += U * 64) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = src[i0 + 64 * u < total ? i0 + 64 * u : total - 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + 64 * u;
      if (i < total) {
        const int r = (int)(((float)i + 0.5f) * inv_nv);  // i / nv, exact while i stays below 2^20
        lds[r * stride + (i - r * nv)] = v[u];
      }
    }
  }
  for (int i = lane; i < nv; i += 64) sv[i] = search[w * lds_ + i];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (lane < rows) {
    const float *row = lds + lane * stride;
    // a chain of fused multiply-adds over [i0, i1), eight operand pairs read ahead of the first
    auto chain = [&](int i0, int i1) {
      float p = 0.0f;
      int i = i0;
      for (; i + 8 <= i1; i += 8) {
        float x[8], y[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          x[u] = row[i + u];
          y[u] = sv[i + u];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) p = fmaf(x[u], y[u], p);
      }
      for (; i < i1; ++i) p = fmaf(row[i], sv[i], p);
      return p;
    };
    float acc = 0.0f;
    if (nv > 50) {
      for (int start = 0; start < nv; start += 20) acc = acc + chain(start, start + 20 < nv ? start + 20 : nv);
    } else {
      acc = chain(0, nv);
    }
    jv[w * ldj + r0 + lane] = minus ? acc - minus[w * ldm + r0 + lane] : acc;
  }
}

// ---- the step along the search direction and the rows whose state changed ----------------------
// qacc += alpha search, Ma += alpha mv (contracted), Jaref = Jaref + alpha * jv (two roundings,
// as the reference spells it out); one thread per element, a world per blockIdx.y.
__global__ __launch_bounds__(kThreads) void newton_advance_kernel(
    const float *__restrict__ alpha, const float *__restrict__ search, int64_t lds_,
    const float *__restrict__ mv, int64_t ldm, const float *__restrict__ jv, int64_t ldj,
    const int32_t *__restrict__ nefc_p, const uint8_t *__restrict__ done, float *__restrict__ qacc, int64_t ldq,
    float *__restrict__ Ma, int64_t lda, float *__restrict__ jaref, int64_t ldr, int nv, int njmax) {
  const int64_t w = blockIdx.y;
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (done && done[w]) return;
  const float a = alpha[w];
  if (i < nv) {
    qacc[w * ldq + i] = fmaf(a, search[w * lds_ + i], qacc[w * ldq + i]);
    Ma[w * lda + i] = fmaf(a, mv[w * ldm + i], Ma[w * lda + i]);
  }
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  if (i < nefc) jaref[w * ldr + i] = jaref[w * ldr + i] + a * jv[w * ldj + i];
}

// Rows whose state differs between two state arrays: the ones whose being quadratic flipped are
// listed in ascending order (64 rows per ballot), the others only counted.  One wavefront per
// world, four worlds per workgroup.
__global__ __launch_bounds__(kThreads) void newton_changed_rows_kernel(
    const int32_t *__restrict__ old_state, const int32_t *__restrict__ new_state, int njmax,
    const int32_t *__restrict__ nefc_p, int quad, const uint8_t *__restrict__ done,
    int32_t *__restrict__ ids, int ld_ids, int32_t *__restrict__ quad_count,
    int32_t *__restrict__ state_count, int nworld) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (w >= nworld || (done && done[w])) return;  // a whole wavefront: no barrier follows
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  const int32_t *so = old_state + w * njmax, *sn = new_state + w * njmax;
  int count = 0, any = 0;
  for (int base = 0; base < nefc; base += 64) {
    const int r = base + lane;
    int o = 0, n = 0;
    if (r < nefc) {
      o = so[r];
      n = sn[r];
    }
    const bool flip = r < nefc && ((o == quad) != (n == quad));
    const unsigned long long mask = __ballot(flip);
    if (flip) {
      const int slot = count + __popcll(mask & ((1ull << lane) - 1ull));
      if (slot < ld_ids) ids[w * ld_ids + slot] = r;
    }
    count += __popcll(mask);
    any += __popcll(__ballot(r < nefc && o != n));
  }
  if (lane == 0) {
    quad_count[w] = count;
    state_count[w] = any;
  }
}

// ---- convergence test of an iteration ------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void newton_converged_kernel(
    const float *__restrict__ alpha, const float *__restrict__ improvement, const float *__restrict__ grad_dot,
    const float *__restrict__ decrement, const float *__restrict__ tolerance, int ntol,
    const float *__restrict__ meaninertia, int ninertia, int nv, int maxiter, int overflow_bit,
    int32_t *__restrict__ niter, int32_t *__restrict__ overflow, uint8_t *__restrict__ done,
    int32_t *__restrict__ nsolving, int nworld) {
  const int w = blockIdx.x * kThreads + threadIdx.x;
  if (w >= nworld || done[w]) return;
  const int it = niter[w] + 1;
  niter[w] = it;
  const float tol = tolerance[w % ntol], scale = meaninertia[w % ninertia] * (float)nv;
  const float imp = improvement[w];
  const bool converged = alpha[w] == 0.0f || (imp > 0.0f && imp / scale < tol) ||
                         sqrtf(grad_dot[w]) / scale < tol || 0.5f * decrement[w] / scale < tol;
  if (converged || it == maxiter) {
    if (!converged && overflow) overflow[w] = overflow[w] | overflow_bit;
    done[w] = 1;
    if (nsolving) atomicAdd(nsolving, -1);
  }
}

// ---- start and finish of the fused solve ----------------------------------------------------------
// One thread per (world, dof), a world per blockIdx.y.
__global__ __launch_bounds__(kThreads) void newton_init_empty_kernel(
    const int32_t *__restrict__ nefc, const float *__restrict__ qacc_smooth, int64_t lds_, int32_t *__restrict__ niter,
    float *__restrict__ search_dot, uint8_t *__restrict__ done, float *__restrict__ qacc, int64_t ldq, int nv) {
  const int64_t w = blockIdx.y;
  const int dof = blockIdx.x * kThreads + threadIdx.x;
  const bool empty = nefc[w] == 0;
  if (dof == 0) {
    niter[w] = 0;
    search_dot[w] = 0.0f;
    done[w] = empty ? 1 : 0;
  }
  if (empty && dof < nv) qacc[w * ldq + dof] = qacc_smooth[w * lds_ + dof];
}

__global__ __launch_bounds__(kThreads) void qfrc_from_grad_kernel(
    const int32_t *__restrict__ nefc, const float *__restrict__ smooth, int64_t lds_, const float *__restrict__ Ma,
    int64_t ldm, const float *__restrict__ grad, int64_t ldg, const float *__restrict__ scale,
    float *__restrict__ out, int64_t ldo, int nv) {
  const int64_t w = blockIdx.y;
  const int dof = blockIdx.x * kThreads + threadIdx.x;
  if (dof >= nv) return;
  float v = 0.0f;
  if (nefc[w] != 0) {
    const float g = scale[w] * grad[w * ldg + dof];
    v = Ma[w * ldm + dof] - smooth[w * lds_ + dof] - g;
  }
  out[w * ldo + dof] = v;
}

// The dense symmetric matrix of a tree CSR M, padded with zeros to (pad, pad): element (i, j)
// is M[elemid[i * nv + j]] where the table names one, else 0.  One thread per element.
__global__ __launch_bounds__(kThreads) void dense_from_csr_kernel(
    const float *__restrict__ M, int64_t ldM, const int32_t *__restrict__ elemid, int nv, int pad,
    float *__restrict__ H) {
  const int64_t w = blockIdx.y;
  const int e = blockIdx.x * kThreads + threadIdx.x;
  if (e >= pad * pad) return;
  const int i = e / pad, j = e - i * pad;
  float v = 0.0f;
  if (i < nv && j < nv) {
    const int id = elemid[i * nv + j];
    if (id >= 0) v = M[w * ldM + id];
  }
  H[w * (int64_t)pad * pad + e] = v;
}

}  // namespace
}  // namespace im

using namespace im;

extern "C" int im_newton_gradient(const int32_t *nefc, const float *J, int njmax, const float *efc_force,
                                  int64_t ld_force, const float *qfrc_smooth, int64_t ld_smooth,
                                  const float *efc_Ma, int64_t ld_Ma, const int32_t *state_changed_count,
                                  const float *alpha, const uint8_t *done, float *qfrc_constraint,
                                  int64_t ld_constraint, float *grad, int64_t ld_grad, float *grad_dot,
                                  float *newton_decrement, float *grad_scale, uint8_t *search_unchanged, int nv,
                                  int block, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || njmax < 0) return IM_ERR_ARG;
  if (block != 32 && block != 64) return IM_ERR_UNSUPPORTED;
  if (nworld == 0) return IM_OK;
  if (!J || !efc_force || !qfrc_smooth || !efc_Ma || !alpha || !qfrc_constraint || !grad ||
      !grad_dot || !newton_decrement || !grad_scale || !search_unchanged)
    return IM_ERR_ARG;
  if (ld_force < njmax || ld_smooth < nv || ld_Ma < nv || ld_constraint < nv || ld_grad < nv) return IM_ERR_STRIDE;
  const int lanes = nv <= 32 ? 32 : 64, per_block = kThreads / lanes;
  const size_t lds_bytes = (size_t)per_block * (2 * (size_t)njmax + nv + 64) * 4;
  if (lds_bytes > kLdsLimit) return IM_ERR_UNSUPPORTED;
  GradArgs a{nefc, J, efc_force, qfrc_smooth, efc_Ma, alpha, state_changed_count, done, qfrc_constraint, grad,
             grad_dot, newton_decrement, grad_scale, search_unchanged, ld_force, ld_smooth, ld_Ma, ld_constraint,
             ld_grad, njmax, nv, block, nworld, lanes};
  // a launch of few workgroups (up to four per CU) has few wavefronts to hide the memory's latency
  // with and asks for sixteen rows at a time; with more of them eight measured faster
  const unsigned nblocks = (unsigned)((nworld + per_block - 1) / per_block);
  if (nblocks <= 1024)
    hipLaunchKernelGGL(newton_gradient_kernel<16>, dim3(nblocks), dim3(kThreads), lds_bytes, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL(newton_gradient_kernel<8>, dim3(nblocks), dim3(kThreads), lds_bytes, (hipStream_t)stream, a);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

namespace {
int launch_jv(const float *J, int njmax, const int32_t *nefc, const float *search, int64_t ld_search,
              const uint8_t *skip_world, float *jv, int64_t ld_jv, const float *minus, int64_t ld_minus, int nv,
              int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || njmax < 0) return IM_ERR_ARG;
  if (nworld == 0 || njmax == 0) return IM_OK;
  if (!J || !search || !jv) return IM_ERR_ARG;
  if (ld_search < nv || ld_jv < njmax || (minus && ld_minus < njmax)) return IM_ERR_STRIDE;
  const size_t lds_bytes = (64 * (size_t)(nv | 1) + nv) * 4;
  if (lds_bytes > kLdsLimit || 64 * (int64_t)nv >= (1 << 20)) return IM_ERR_UNSUPPORTED;
  const int chunks = (njmax + 63) / 64;
  if ((int64_t)nworld * chunks > 0x7fffffff) return IM_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((int64_t)nworld * chunks));
#define IM_JV(U)                                                                                          \
  hipLaunchKernelGGL(newton_jv_kernel<U>, grid, dim3(64), lds_bytes, (hipStream_t)stream, J, njmax, nefc, \
                     search, ld_search, skip_world, jv, ld_jv, nv, chunks, minus, ld_minus)
  // 64 rows of nv words are nv words per lane
  if (nv <= 16) IM_JV(16);
  else if (nv <= 32) IM_JV(32);
  else if (nv <= 48) IM_JV(48);
  else IM_JV(64);
#undef IM_JV
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
}  // namespace

extern "C" int im_newton_jv(const float *J, int njmax, const int32_t *nefc, const float *search, int64_t ld_search,
                            const uint8_t *skip_world, float *jv, int64_t ld_jv, int nv, int nworld, void *stream) {
  return launch_jv(J, njmax, nefc, search, ld_search, skip_world, jv, ld_jv, nullptr, 0, nv, nworld, stream);
}

extern "C" int im_newton_init_jaref(const float *J, int njmax, const int32_t *nefc, const float *qacc, int64_t ld_qacc,
                                    const float *aref, int64_t ld_aref, float *Jaref, int64_t ld_Jaref, int nv,
                                    int nworld, void *stream) {
  if (!aref) return IM_ERR_ARG;
  return launch_jv(J, njmax, nefc, qacc, ld_qacc, nullptr, Jaref, ld_Jaref, aref, ld_aref, nv, nworld, stream);
}

extern "C" int im_dense_from_csr(const float *M, int64_t ldM, const int32_t *elemid, int nv, int pad, float *H,
                                 int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || pad < nv) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!M || !elemid || !H) return IM_ERR_ARG;
  const int per = pad * pad;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(dense_from_csr_kernel, dim3((unsigned)((per + kThreads - 1) / kThreads), (unsigned)nw),
                       dim3(kThreads), 0, (hipStream_t)stream, M + w0 * ldM, ldM, elemid, nv, pad,
                       H + (int64_t)w0 * per);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_newton_advance(const float *alpha, const float *search, int64_t ld_search, const float *mv,
                                 int64_t ld_mv, const float *jv, int64_t ld_jv, const int32_t *nefc,
                                 const uint8_t *done, float *qacc, int64_t ld_qacc, float *efc_Ma, int64_t ld_Ma,
                                 float *Jaref, int64_t ld_Jaref, int nv, int njmax, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || njmax < 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!alpha || !search || !mv || !qacc || !efc_Ma || (njmax > 0 && (!jv || !Jaref))) return IM_ERR_ARG;
  if (ld_search < nv || ld_mv < nv || ld_qacc < nv || ld_Ma < nv || ld_jv < njmax || ld_Jaref < njmax)
    return IM_ERR_STRIDE;
  const int n = nv > njmax ? nv : njmax;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {  // the grid's y dimension carries the world
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(newton_advance_kernel, dim3((unsigned)((n + kThreads - 1) / kThreads), (unsigned)nw),
                       dim3(kThreads), 0, (hipStream_t)stream, alpha + w0, search + w0 * ld_search, ld_search,
                       mv + w0 * ld_mv, ld_mv, jv ? jv + w0 * ld_jv : nullptr, ld_jv, nefc ? nefc + w0 : nullptr,
                       done ? done + w0 : nullptr, qacc + w0 * ld_qacc, ld_qacc, efc_Ma + w0 * ld_Ma, ld_Ma,
                       Jaref ? Jaref + w0 * ld_Jaref : nullptr, ld_Jaref, nv, njmax);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_newton_changed_rows(const int32_t *old_state, const int32_t *new_state, int njmax,
                                      const int32_t *nefc, int quad, const uint8_t *done, int32_t *quad_changed_ids,
                                      int ld_ids, int32_t *quad_changed_count, int32_t *state_changed_count,
                                      int nworld, void *stream) {
  if (nworld < 0 || njmax < 0 || ld_ids < 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!old_state || !new_state || !quad_changed_ids || !quad_changed_count || !state_changed_count)
    return IM_ERR_ARG;
  const int per_block = kThreads / 64;
  hipLaunchKernelGGL(newton_changed_rows_kernel, dim3((unsigned)((nworld + per_block - 1) / per_block)),
                     dim3(kThreads), 0, (hipStream_t)stream, old_state, new_state, njmax, nefc, quad, done,
                     quad_changed_ids, ld_ids, quad_changed_count, state_changed_count, nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_newton_converged(const float *alpha, const float *improvement, const float *grad_dot,
                                   const float *newton_decrement, const float *opt_tolerance, int ntolerance,
                                   const float *stat_meaninertia, int nmeaninertia, int nv, int maxiter,
                                   int overflow_bit, int32_t *niter, int32_t *overflow, uint8_t *done,
                                   int32_t *nsolving, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || ntolerance <= 0 || nmeaninertia <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!alpha || !improvement || !grad_dot || !newton_decrement || !opt_tolerance || !stat_meaninertia || !niter ||
      !done)
    return IM_ERR_ARG;
  hipLaunchKernelGGL(newton_converged_kernel, dim3((unsigned)((nworld + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     (hipStream_t)stream, alpha, improvement, grad_dot, newton_decrement, opt_tolerance, ntolerance,
                     stat_meaninertia, nmeaninertia, nv, maxiter, overflow_bit, niter, overflow, done, nsolving,
                     nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_newton_init_empty_worlds(const int32_t *nefc, const float *qacc_smooth, int64_t ld_smooth,
                                           int32_t *solver_niter, float *search_dot, uint8_t *done, float *qacc,
                                           int64_t ld_qacc, int nv, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!nefc || !qacc_smooth || !solver_niter || !search_dot || !done || !qacc) return IM_ERR_ARG;
  if (ld_smooth < nv || ld_qacc < nv) return IM_ERR_STRIDE;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(newton_init_empty_kernel, dim3((unsigned)((nv + kThreads - 1) / kThreads), (unsigned)nw),
                       dim3(kThreads), 0, (hipStream_t)stream, nefc + w0, qacc_smooth + w0 * ld_smooth, ld_smooth,
                       solver_niter + w0, search_dot + w0, done + w0, qacc + w0 * ld_qacc, ld_qacc, nv);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_qfrc_constraint_from_grad(const int32_t *nefc, const float *qfrc_smooth, int64_t ld_smooth,
                                            const float *efc_Ma, int64_t ld_Ma, const float *grad, int64_t ld_grad,
                                            const float *grad_scale, float *qfrc_constraint, int64_t ld_constraint,
                                            int nv, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!nefc || !qfrc_smooth || !efc_Ma || !grad || !grad_scale || !qfrc_constraint) return IM_ERR_ARG;
  if (ld_smooth < nv || ld_Ma < nv || ld_grad < nv || ld_constraint < nv) return IM_ERR_STRIDE;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(qfrc_from_grad_kernel, dim3((unsigned)((nv + kThreads - 1) / kThreads), (unsigned)nw),
                       dim3(kThreads), 0, (hipStream_t)stream, nefc + w0, qfrc_smooth + w0 * ld_smooth, ld_smooth,
                       efc_Ma + w0 * ld_Ma, ld_Ma, grad + w0 * ld_grad, ld_grad, grad_scale + w0,
                       qfrc_constraint + w0 * ld_constraint, ld_constraint, nv);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
