// Static-pattern sparse L'DL of the Newton Hessian: initial assembly on the pattern
// slots, level-scheduled numeric factor, forward solve through the augmented row,
// backward solve, search direction and its two dot products.  One workgroup per world.
//
// Reference: src/instantmimic/utils/mjw_kernels/sparse_hessian.py
//   assembly (tile of 4 rows, per slot v = fmaf(J[r][a] * Dc[r], J[r][b], v))      :578-630
//   level factor (team lanes stride the terms, shuffle-down tree, w = N - v)        :410-452
//   backward pushes per level, search = -x, (x.x, g.x) reduced warp then block      :453-479
//   hfactor layout: [0,nfac) packed H, [nfac,2nfac) N = L D, [2nfac,2nfac+n) 1/D,
//   last element = pattern-violation counter                                        :488-489, 634-635
// The tables come from the host planner (instantmimic_amd/mjw_kernels/sparse_hessian.py)
// instead of generated source; team widths and block width are the plan's, so the
// order in which a team sums an entry's terms is the reference's.
#include <hip/hip_runtime.h>

#include <cstring>
#include <vector>

#include "common.h"

struct im_sparse_plan {
  int nv, nv_pad, block, nslots, nlevels;
  void *blob = nullptr;
  int ntables = 0;
  const int32_t *t[22] = {};
  int sizes[22] = {};
};

namespace im {
namespace {

enum { LP, LT, ES, EC, RP, RAB, RKL, ORIG, BL, BS, BI, BJ, PM, SA, SB, SM, NINIT,
       PAIR = NINIT, FL, FR, RS, RKP, RK, NTABLES };

struct SparseDev {
  const int32_t *t[NTABLES];
  int nv, nv_pad, nslots, nlevels;
};

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// level-scheduled numeric factor: team lanes stride an entry's terms, shuffle-down tree
__device__ __forceinline__ void factor_levels(const SparseDev &P, float *N, float *iD, int lane, int block) {
  const int32_t *LPt = P.t[LP], *LTt = P.t[LT], *ESt = P.t[ES], *ECt = P.t[EC], *RPt = P.t[RP];
  const uint32_t *RABt = (const uint32_t *)P.t[RAB], *RKLt = (const uint32_t *)P.t[RKL];
  for (int l = 0; l < P.nlevels; ++l) {
    const int e0 = LPt[l], e1 = LPt[l + 1], T = LTt[l];
    const int tl = lane & (T - 1), team = lane / T, teams = block / T;
    for (int eb = e0; eb < e1; eb += teams) {
      const int e = eb + team;
      float v = 0.0f;
      int sl = 0, col = -1;
      if (e < e1) {
        sl = ESt[e];
        col = ECt[e];
        for (int r = RPt[e]; r < RPt[e + 1]; ++r) {
          const uint32_t ab = RABt[r], kl = RKLt[r];
          const float *pa = N + (ab & 0xFFFFu), *pb = N + (ab >> 16), *pd = iD + (kl & 0xFFFFu);
          const int len = (int)(kl >> 16);
          for (int t = tl; t < len; t += T) v = fma_(pa[t] * pb[t], pd[t], v);
        }
      }
      for (int off = T >> 1; off > 0; off >>= 1) v = v + __shfl_down(v, off, T);
      if (e < e1 && tl == 0) {
        const float wv = N[sl] - v;
        N[sl] = wv;
        if (col >= 0) iD[col] = 1.0f / wv;
      }
    }
    __syncthreads();
  }
}

// backward pushes by level (root first), search = -x, (x.x, g.x) reduced warp then block
__device__ __forceinline__ void backward_sums(const SparseDev &P, float *N, const float *iD,
                                              const float *__restrict__ gw, float *__restrict__ search,
                                              float *red, float *search_dot, float *decrement, int lane,
                                              int block) {
  const int n = P.nv, rhs = P.nslots - n, nw = (block + 31) / 32;
  const int32_t *ORIGt = P.t[ORIG];
  // backward solve, root level first
  const int32_t *BLt = P.t[BL], *BSt = P.t[BS], *BIt = P.t[BI], *BJt = P.t[BJ];
  for (int l = 0; l < P.nlevels; ++l) {
    for (int p = BLt[l] + lane; p < BLt[l + 1]; p += block) {
      const int i = BIt[p], j = BJt[p];
      N[rhs + j] = fma_(-N[BSt[p]], N[rhs + i] * iD[i], N[rhs + j]);
    }
    __syncthreads();
  }
  float s0 = 0.0f, s1 = 0.0f;
  for (int j = lane; j < n; j += block) {
    const int d = ORIGt[j];
    const float v = N[rhs + j] * iD[j];
    search[d] = -v;
    s0 = fma_(v, v, s0);
    s1 = fma_(gw[d], v, s1);
  }
  for (int o = 16; o > 0; o >>= 1) {
    s0 = s0 + __shfl_down(s0, o, 32);
    s1 = s1 + __shfl_down(s1, o, 32);
  }
  if ((lane & 31) == 0) {
    red[lane >> 5] = s0;
    red[nw + (lane >> 5)] = s1;
  }
  __syncthreads();
  if (lane == 0) {
    float ra = 0.0f, rb = 0.0f;
    for (int i = 0; i < nw; ++i) {
      ra = ra + red[i];
      rb = rb + red[nw + i];
    }
    *search_dot = ra;
    *decrement = rb;
  }
}

__global__ void sparse_init_kernel(SparseDev P, const uint8_t *__restrict__ done,
                                   const int32_t *__restrict__ nefc_p, const float *__restrict__ J,
                                   int njmax, const float *__restrict__ D,
                                   const int32_t *__restrict__ state, int quad,
                                   const float *__restrict__ M, int ldM,
                                   const float *__restrict__ grad, int ldg, float *__restrict__ U_,
                                   float *__restrict__ search_, float *__restrict__ search_dot,
                                   float *__restrict__ decrement) {
  extern __shared__ float lds[];
  const int w = blockIdx.x, lane = threadIdx.x, block = blockDim.x;
  if (done && done[w]) return;
  const int n = P.nv, nslots = P.nslots, nfac = nslots - n, rhs = nfac;
  const int words = (n + 31) / 32, nw = (block + 31) / 32;
  float *N = lds;                      // [nslots]
  float *iD = N + nslots;              // [n]
  float *red = iD + n;                 // [2][nw]
  float *Jc = red + 2 * nw;            // [4][n]
  float *Dc = Jc + 4 * n;              // [4]
  unsigned *rm = (unsigned *)(Dc + 4); // [4][words] row supports
  int *bad = (int *)(rm + 4 * words);  // [4]
  float *U = U_ + (size_t)w * P.nv_pad * P.nv_pad;
  const float *Mw = M + (size_t)w * ldM;
  const float *gw = grad + (size_t)w * ldg;
  const float *Jw = J + (size_t)w * njmax * n;
  const int32_t *SAt = P.t[SA], *SBt = P.t[SB], *SMt = P.t[SM], *PMt = P.t[PM];

  for (int s = lane; s < nfac; s += block) {
    const int e = SMt[s];
    N[s] = e >= 0 ? Mw[e] : 0.0f;
  }
  int nefc = nefc_p[w];
  nefc = nefc < njmax ? nefc : njmax;
  for (int k = 0; k < nefc; k += 4) {
    __syncthreads();
    for (int q = lane; q < 4 * n; q += block) {
      const int r = q / n;
      Jc[q] = (k + r < nefc) ? Jw[(size_t)(k + r) * n + (q - r * n)] : 0.0f;
    }
    if (lane < 4) {
      float d = 0.0f;
      if (k + lane < nefc && state[(size_t)w * njmax + k + lane] == quad) d = D[(size_t)w * njmax + k + lane];
      Dc[lane] = d;
      bad[lane] = 0;
    }
    for (int q = lane; q < 4 * words; q += block) rm[q] = 0u;
    __syncthreads();
    // every active row's dof support must lie in the pattern
    for (int q = lane; q < 4 * n; q += block) {
      const int r = q / n, d = q - r * n;
      if (Dc[r] != 0.0f && Jc[q] != 0.0f) atomicOr(&rm[r * words + d / 32], 1u << (d % 32));
    }
    __syncthreads();
    for (int q = lane; q < 4 * n; q += block) {
      const int r = q / n, d = q - r * n;
      if ((rm[r * words + d / 32] >> (d % 32)) & 1u) {
        bool b = false;
        for (int p = 0; p < words; ++p) b = b || (rm[r * words + p] & ~(unsigned)PMt[d * words + p]) != 0u;
        if (b) bad[r] = 1;
      }
    }
    for (int s = lane; s < nfac; s += block) {
      const int a = SAt[s], b = SBt[s];
      float v = N[s];
#pragma unroll
      for (int r = 0; r < 4; ++r) v = fma_(Jc[r * n + a] * Dc[r], Jc[r * n + b], v);
      N[s] = v;
    }
    __syncthreads();
    if (lane < 4 && bad[lane]) atomicAdd(U + P.nv_pad * P.nv_pad - 1, 1.0f);
  }
  __syncthreads();
  for (int s = lane; s < nfac; s += block) U[s] = N[s];
  // numeric factor; the right-hand side is row n of the augmented matrix
  const int32_t *ORIGt = P.t[ORIG];
  for (int j = lane; j < n; j += block) N[rhs + j] = gw[ORIGt[j]];
  __syncthreads();
  factor_levels(P, N, iD, lane, block);
  for (int s = lane; s < nfac; s += block) U[nfac + s] = N[s];
  for (int j = lane; j < n; j += block) U[2 * nfac + j] = iD[j];
  backward_sums(P, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, block);
}

// Per-iteration factor stage: changed rows' dof union, incremental update of packed H,
// refactor -- or, with no changed row, a forward solve with the stored factor -- then the
// backward solve.  Reference: sparse_hessian.py:488-547 (modes 0, 1, 2) inside
// newton_stages.factor_factory (:614-742, union :651-679).  The factor lives in hfactor
// between launches ([nfac, 2 nfac) and 1/D behind it) where the reference keeps it in a
// resident block's shared memory.  The workgroup is one wavefront (block 32 or 64).
__global__ void sparse_update_kernel(SparseDev P, const uint8_t *__restrict__ done,
                                     const int32_t *__restrict__ state_changes,
                                     const int32_t *__restrict__ changes, const int32_t *__restrict__ ids,
                                     int ld_ids, const float *__restrict__ J, int njmax,
                                     const float *__restrict__ D, const int32_t *__restrict__ state, int quad,
                                     const float *__restrict__ grad, int ldg, float *__restrict__ U_,
                                     int32_t *__restrict__ uni_, float *__restrict__ search_,
                                     float *__restrict__ search_dot, float *__restrict__ decrement) {
  extern __shared__ float lds[];
  const int w = blockIdx.x, lane = threadIdx.x, block = blockDim.x;
  if ((done && done[w]) || state_changes[w] == 0) return;
  const int n = P.nv, nslots = P.nslots, nfac = nslots - n, rhs = nfac;
  const int nw = (block + 31) / 32;
  float *N = lds;             // [nslots]
  float *iD = N + nslots;     // [n]
  float *red = iD + n;        // [2][nw]
  int *ul = (int *)(red + 2 * nw);  // [n] ascending dofs touched by the changed rows
  float *U = U_ + (size_t)w * P.nv_pad * P.nv_pad;
  const float *gw = grad + (size_t)w * ldg;
  const float *Jw = J + (size_t)w * njmax * n;
  const float *Dw = D + (size_t)w * njmax;
  const int32_t *sw = state + (size_t)w * njmax, *idw = ids + (size_t)w * ld_ids;
  const int32_t *ORIGt = P.t[ORIG];
  int count = changes[w];
  count = count < ld_ids ? count : ld_ids;
  if (count > 0) {
    int nu = 0;
    for (int base = 0; base < n; base += block) {
      const int dof = base + lane;
      bool hit = false;
      if (dof < n)
        for (int t = 0; t < count && !hit; ++t) hit = Jw[(size_t)idw[t] * n + dof] != 0.0f;
      const unsigned long long mask = __ballot(hit);
      if (hit) ul[nu + __popcll(mask & ((1ull << lane) - 1ull))] = dof;
      nu += __popcll(mask);
    }
    __syncthreads();
    int32_t *uni = uni_ + (size_t)w * (n + 1);
    for (int i = lane; i < nu; i += block) uni[i] = ul[i];
    if (lane == 0) uni[n] = nu;
    const int32_t *PAIRt = P.t[PAIR];
    const int npair = nu * (nu + 1) / 2;
    for (int e = lane; e < npair; e += block) {
      // e = cj (cj + 1) / 2 + ri with ri <= cj, found exactly
      int cj = (int)((sqrtf((float)(8 * e + 1)) - 1.0f) * 0.5f);
      while ((cj + 1) * (cj + 2) / 2 <= e) ++cj;
      while (cj * (cj + 1) / 2 > e) --cj;
      const int row = ul[e - cj * (cj + 1) / 2], col = ul[cj];
      float delta = 0.0f;
      for (int t = 0; t < count; ++t) {
        const int r = idw[t];
        const float a = Jw[(size_t)r * n + row], b = Jw[(size_t)r * n + col];
        float da = Dw[r] * a;
        if (sw[r] != quad) da = -da;
        if (a != 0.0f && b != 0.0f) delta = fma_(da, b, delta);
      }
      if (delta != 0.0f) {
        const int sl = PAIRt[row * n + col];
        if (sl >= 0) U[sl] = U[sl] + delta;
        else atomicAdd(U + P.nv_pad * P.nv_pad - 1, 1.0f);
      }
    }
    __syncthreads();
    for (int s = lane; s < nfac; s += block) N[s] = U[s];
    for (int j = lane; j < n; j += block) N[rhs + j] = gw[ORIGt[j]];
    __syncthreads();
    factor_levels(P, N, iD, lane, block);
    for (int s = lane; s < nfac; s += block) U[nfac + s] = N[s];
    for (int j = lane; j < n; j += block) U[2 * nfac + j] = iD[j];
  } else {
    for (int s = lane; s < nfac; s += block) N[s] = U[nfac + s];
    for (int j = lane; j < n; j += block) iD[j] = U[2 * nfac + j];
    __syncthreads();
    const int32_t *FLt = P.t[FL], *FRt = P.t[FR], *RSt = P.t[RS], *RKPt = P.t[RKP], *RKt = P.t[RK];
    for (int l = 0; l < P.nlevels; ++l) {
      for (int q = FLt[l] + lane; q < FLt[l + 1]; q += block) {
        const int j = FRt[q];
        float v = gw[ORIGt[j]];
        const float *rowp = N + RSt[j];
        const int k0 = RKPt[j], k1 = RKPt[j + 1];
        for (int t = 0; t < k1 - k0; ++t) {
          const int k = RKt[k0 + t];
          v = fma_(-(rowp[t] * iD[k]), N[rhs + k], v);
        }
        N[rhs + j] = v;
      }
      __syncthreads();
    }
  }
  backward_sums(P, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, block);
}

}  // namespace
}  // namespace im

extern "C" {

int im_sparse_plan_create(int nv, int nv_pad, int block, int nslots, int nlevels, int ntables,
                          const int32_t *const *tables, const int *sizes, im_sparse_plan **out) {
  if (!out) return IM_ERR_ARG;
  *out = nullptr;
  if (!tables || !sizes || (ntables != im::NINIT && ntables != im::NTABLES) || nv <= 0 || nslots <= nv)
    return IM_ERR_ARG;
  if (block != 32 && block != 64) return IM_ERR_UNSUPPORTED;
  auto *pl = new im_sparse_plan;
  pl->nv = nv; pl->nv_pad = nv_pad; pl->block = block; pl->nslots = nslots; pl->nlevels = nlevels;
  pl->ntables = ntables;
  size_t total = 0;
  for (int i = 0; i < ntables; ++i) total += ((size_t)sizes[i] * 4 + 15) / 16 * 16;
  std::vector<char> host(total, 0);
  size_t off = 0;
  std::vector<size_t> offs(ntables);
  for (int i = 0; i < ntables; ++i) {
    offs[i] = off;
    memcpy(host.data() + off, tables[i], (size_t)sizes[i] * 4);
    off += ((size_t)sizes[i] * 4 + 15) / 16 * 16;
    pl->sizes[i] = sizes[i];
  }
  if (hipMalloc(&pl->blob, total) != hipSuccess || hipMemcpy(pl->blob, host.data(), total, hipMemcpyHostToDevice) != hipSuccess) {
    im::set_hip_error(hipGetLastError());
    if (pl->blob) (void)hipFree(pl->blob);
    delete pl;
    return IM_ERR_HIP;
  }
  for (int i = 0; i < ntables; ++i) pl->t[i] = (const int32_t *)((char *)pl->blob + offs[i]);
  *out = pl;
  return IM_OK;
}

void im_sparse_plan_destroy(im_sparse_plan *plan) {
  if (!plan) return;
  if (plan->blob) (void)hipFree(plan->blob);
  delete plan;
}

int im_sparse_init_factor(const im_sparse_plan *plan, const uint8_t *done, const int32_t *nefc,
                          const float *J, int njmax, const float *D, const int32_t *state, int quad,
                          const float *M, int ldM, const float *grad, int ldg, float *hfactor,
                          float *search, float *search_dot, float *decrement, int nworld, void *stream) {
  if (!plan || nworld < 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!nefc || !J || !D || !state || !M || !grad || !hfactor || !search || !search_dot || !decrement) return IM_ERR_ARG;
  if (ldg < plan->nv) return IM_ERR_STRIDE;
  im::SparseDev P;
  for (int i = 0; i < im::NTABLES; ++i) P.t[i] = plan->t[i];
  P.nv = plan->nv; P.nv_pad = plan->nv_pad; P.nslots = plan->nslots; P.nlevels = plan->nlevels;
  const int n = plan->nv, words = (n + 31) / 32, nw = (plan->block + 31) / 32;
  const size_t lds_bytes = 4 * ((size_t)plan->nslots + n + 2 * nw + 4 * n + 4 + 4 * words + 4);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::sparse_init_kernel, dim3(nworld), dim3(plan->block), lds_bytes, (hipStream_t)stream, P,
                     done, nefc, J, njmax, D, state, quad, M, ldM, grad, ldg, hfactor, search, search_dot, decrement);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_sparse_update_factor(const im_sparse_plan *plan, const uint8_t *done, const int32_t *state_changes,
                            const int32_t *changes, const int32_t *ids, int ld_ids, const float *J, int njmax,
                            const float *D, const int32_t *state, int quad, const float *grad, int ldg,
                            float *hfactor, int32_t *dof_union, float *search, float *search_dot,
                            float *decrement, int nworld, void *stream) {
  if (!plan || nworld < 0 || ld_ids < 0) return IM_ERR_ARG;
  if (plan->ntables != im::NTABLES) return IM_ERR_UNSUPPORTED;  // built without the update tables
  if (nworld == 0) return IM_OK;
  if (!state_changes || !changes || !ids || !J || !D || !state || !grad || !hfactor || !dof_union || !search ||
      !search_dot || !decrement)
    return IM_ERR_ARG;
  if (ldg < plan->nv) return IM_ERR_STRIDE;
  im::SparseDev P;
  for (int i = 0; i < im::NTABLES; ++i) P.t[i] = plan->t[i];
  P.nv = plan->nv; P.nv_pad = plan->nv_pad; P.nslots = plan->nslots; P.nlevels = plan->nlevels;
  const int n = plan->nv, nw = (plan->block + 31) / 32;
  const size_t lds_bytes = 4 * ((size_t)plan->nslots + n + 2 * nw + n);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::sparse_update_kernel, dim3(nworld), dim3(plan->block), lds_bytes, (hipStream_t)stream, P,
                     done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, hfactor,
                     dof_union, search, search_dot, decrement);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
