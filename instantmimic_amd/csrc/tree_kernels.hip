// Fused Hessian assembly + kinematic-tree L'DL + solve for gfx950, one wavefront
// per world.
//
// What is computed (reference statements):
//   H[e]  = M[e] + sum_r fmaf(J[r][a] * Dc[r], J[r][b], .)   rows ascending
//           (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:589, 622-629)
//   x     = (L'DL)^-1 y on M's CSR pattern, leaves first
//           (src/instantmimic/utils/mjw_kernels/tree_ldl.py:215-305)
// with the plan's groups accumulating their trunk contributions from zero and
// the trunk summing them in group order, so that every floating-point operation
// and its order equal the reference's generated straight-line code.  Arithmetic
// convention: t - a*b*c is fmaf(-(a*b), c, t) and s - a*b is fmaf(-a, b, s) (what
// a contracting compiler makes of the reference's expressions); this file is
// compiled with -ffp-contract=off and spells every fused operation.
//
// Mapping.  A world is served by one 64-lane wavefront (workgroup of 64).  The
// nM entries of H live in registers, entry e in lane e % 64, register e / 64,
// and never move: the assembly accumulates into them, eliminations update them
// in place.  When dof k is eliminated its (final) row is published to LDS and
// every lane whose entry belongs to an ancestor row applies its update from two
// LDS reads.  The right-hand side rides along, one dof per lane.  Constraint
// rows are staged through LDS in chunks, inactive rows are dropped while staging,
// and the next chunk's global loads are in flight while the current one is summed.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

#include "common.h"
#include "tree_row16.h"
#include <cstdlib>
#include <vector>

namespace im {
namespace gen {
namespace {
std::vector<const Row16Entry *> &registry() {
  static std::vector<const Row16Entry *> r;
  return r;
}
}  // namespace
Row16Register::Row16Register(const Row16Entry *e) { registry().push_back(e); }
const Row16Entry *find_row16(uint64_t key) {
  for (const Row16Entry *e : registry())
    if (e->key == key) return e;
  return nullptr;
}
}  // namespace gen

namespace {

// FNV-1a over the CSR structure and the plan; the generator computes the same key
// (instantmimic_amd/codegen/tree_row16.py: structure_key).
uint64_t tree_key(const im_tree_plan &pl) {
  uint64_t h = 0xCBF29CE484222325ull;
  auto mix = [&](uint32_t v) {
    h ^= v;
    h *= 0x100000001B3ull;
  };
  mix(pl.nv);
  for (int v : pl.rowadr) mix(v);
  for (int v : pl.rownnz) mix(v);
  mix(pl.nM);
  for (int v : pl.colind) mix(v);
  mix((uint32_t)pl.groups.size());
  for (const auto &g : pl.groups) {
    mix((uint32_t)g.size());
    for (int v : g) mix(v);
  }
  mix((uint32_t)pl.trunk.size());
  for (int v : pl.trunk) mix(v);
  return h;
}

constexpr int kPF = 16;  // global-load registers per lane and chunk (1024 floats)

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

template <int SPL, int NVP, bool ASM>
__global__ __launch_bounds__(64) void tree_kernel(
    TreeDev P, const float *__restrict__ M, int64_t ldM, const float *__restrict__ J,
    int njmax, const float *__restrict__ D, const int32_t *__restrict__ state,
    const int32_t *__restrict__ nefc_p, int quad, const float *__restrict__ y,
    int64_t ldy, float *__restrict__ x, int64_t ldx, float *__restrict__ Hout,
    int rc, float inv_nv, int njpad, unsigned flags, const unsigned char *__restrict__ skip) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x;
  const int w = blockIdx.x;
  if (skip && skip[w]) return;  // the workgroup is this world's one wavefront
  const int nv = P.nv, nM = P.nM;

  float *T = lds;                      // [nM]   published rows (unscaled)
  float *Sp = T + nM;                  // [64]   published right-hand sides
  float *Di = Sp + 64;                 // [64]   inverse pivots
  float *X = Di + 64;                  // [64]   solution
  int *col = (int *)(X + 64);          // [nM]
  float *Dc = (float *)(col + nM);     // [njpad]
  float *Jc = Dc + njpad;              // [rc * NVP]
  float *JDc = Jc + rc * NVP;          // [rc * NVP]

  // ---- per-lane constants -------------------------------------------------
  int se[SPL];        // CSR entry, -1 when the register is unused
  uint32_t sd[SPL];   // a | b << 8 | p << 16 | q << 24
  bool strunk[SPL];   // the entry's row is a trunk dof
  float h[SPL];
  float acc[IM_MAX_GROUPS][SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int e = P.slot_e[i * 64 + lane];
    const uint32_t d = P.slot_d[i * 64 + lane];
    se[i] = e < 0 ? -1 : (e & 0xFFFF);
    strunk[i] = e >= 0 && ((e >> 30) & 1);
    sd[i] = d;
    h[i] = se[i] >= 0 ? M[(int64_t)w * ldM + se[i]] : 0.0f;
#pragma unroll
    for (int j = 0; j < IM_MAX_GROUPS; ++j) acc[j][i] = 0.0f;
  }
  const int dd = P.dof_d[lane];
  const bool isdof = dd >= 0;
  const int drow = dd & 0xFFFF;
  const int ddepth = isdof ? ((dd >> 16) & 0xFF) : -1;
  const bool dtrunk = isdof && ((dd >> 24) & 1);
  float s = isdof ? y[(int64_t)w * ldy + lane] : 0.0f;
  float sacc[IM_MAX_GROUPS] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int e = lane; e < nM; e += 64) col[e] = P.colind[e];

  // ---- assembly -------------------------------------------------------------
  if (ASM) {
    int nefc = nefc_p ? nefc_p[w] : njmax;
    nefc = nefc < njmax ? nefc : njmax;
    nefc = __builtin_amdgcn_readfirstlane(nefc);
    const float *Dw = D + (int64_t)w * njmax;
    const int32_t *Sw = state + (int64_t)w * njmax;
    for (int r = lane; r < njpad; r += 64) {
      float dc = 0.0f;
      if (r < nefc && Sw[r] == quad) dc = Dw[r];
      Dc[r] = dc;
    }
    const float *Jw = J + (int64_t)w * njmax * nv;
    const int nchunk = (nefc + rc - 1) / rc;
    float cur[kPF], nxt[kPF];
    int offa[SPL], offb[SPL];  // float offsets of a and b inside a staged row
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      offa[i] = sd[i] & 0xFF;
      offb[i] = (sd[i] >> 8) & 0xFF;
    }
    {
      const int rows = nefc < rc ? nefc : rc;
#pragma unroll
      for (int u = 0; u < kPF; ++u) {
        const int q = lane + 64 * u;
        cur[u] = q < rows * nv ? Jw[q] : 0.0f;
      }
    }
    __syncthreads();  // Dc visible
    for (int c = 0; c < nchunk; ++c) {
      {
        const int r1 = (c + 1) * rc;
        int rows = nefc - r1;
        rows = rows < rc ? rows : rc;
        const float *Jn = Jw + (int64_t)r1 * nv;
#pragma unroll
        for (int u = 0; u < kPF; ++u) {
          const int q = lane + 64 * u;
          nxt[u] = q < rows * nv ? Jn[q] : 0.0f;
        }
      }
      // rows of this chunk that contribute, as a bit mask (rc <= 64)
      const int r0 = c * rc;
      const float mydc = lane < rc ? Dc[r0 + lane] : 0.0f;
      const uint64_t amask = __ballot(mydc != 0.0f);
      const int nact = __popcll(amask);
#pragma unroll
      for (int u = 0; u < kPF; ++u) {
        // element -> (row, column) of the chunk
        const int q = lane + 64 * u;
        const int r = (int)(((float)q + 0.5f) * inv_nv);
        if (r < rc && ((amask >> r) & 1ull)) {
          const int dst = __popcll(amask & ((1ull << r) - 1ull)) * NVP + (q - r * nv);
          const float dc = Dc[r0 + r];
          Jc[dst] = cur[u];
          JDc[dst] = cur[u] * dc;
        }
      }
      __syncthreads();
      int rl = 0;
      for (; rl + 4 <= nact; rl += 4) {
        const float *ja = JDc + rl * NVP;
        const float *jb = Jc + rl * NVP;
        float va[4][SPL], vb[4][SPL];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int i = 0; i < SPL; ++i) {
            va[t][i] = ja[t * NVP + offa[i]];
            vb[t][i] = jb[t * NVP + offb[i]];
          }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int i = 0; i < SPL; ++i) h[i] = fma_(va[t][i], vb[t][i], h[i]);
      }
      for (; rl < nact; ++rl) {
        const float *ja = JDc + rl * NVP;
        const float *jb = Jc + rl * NVP;
#pragma unroll
        for (int i = 0; i < SPL; ++i) h[i] = fma_(ja[offa[i]], jb[offb[i]], h[i]);
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < kPF; ++u) cur[u] = nxt[u];
    }
    if (Hout) {
#pragma unroll
      for (int i = 0; i < SPL; ++i)
        if (se[i] >= 0) Hout[(int64_t)w * nM + se[i]] = h[i];
    }
  }

  // ---- leaves-first elimination ----------------------------------------------
  for (int st = 0; st < P.nsteps; ++st) {
    const int4 info = P.steps[st];
    const int gid = info.z;
    if (gid < 0) {
      // trunk rows: own value plus the groups' contributions in group order
#pragma unroll
      for (int j = 0; j < IM_MAX_GROUPS; ++j) {
        if (j < P.ngroups) {
#pragma unroll
          for (int i = 0; i < SPL; ++i) h[i] = h[i] + acc[j][i];
          s = s + sacc[j];
        }
      }
      continue;
    }
    const int rk = info.x, cnt = info.y, k = info.w;
    const uint64_t anc = P.anc[st];
#pragma unroll
    for (int i = 0; i < SPL; ++i)
      if (se[i] >= 0 && (int)((sd[i] >> 8) & 0xFF) == k) T[se[i]] = h[i];
    if (lane == k) Sp[k] = s;
    __syncthreads();
    const float dk = 1.0f / T[rk + cnt];
    const float sk = Sp[k];
    if (lane == 0) Di[k] = dk;
    const bool togroup = gid < IM_MAX_GROUPS;
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      if (se[i] >= 0 && ((anc >> ((sd[i] >> 8) & 0xFF)) & 1ull)) {
        const float v = T[rk + ((sd[i] >> 16) & 0xFF)] * T[rk + (sd[i] >> 24)];
        if (togroup && strunk[i]) {
          if (gid == 0) acc[0][i] = fma_(-v, dk, acc[0][i]);
          else if (gid == 1) acc[1][i] = fma_(-v, dk, acc[1][i]);
          else if (gid == 2) acc[2][i] = fma_(-v, dk, acc[2][i]);
          else acc[3][i] = fma_(-v, dk, acc[3][i]);
        } else {
          h[i] = fma_(-v, dk, h[i]);
        }
      }
    }
    if (isdof && ((anc >> lane) & 1ull)) {
      const float ms = T[rk + ddepth] * dk;
      if (togroup && dtrunk) {
        if (gid == 0) sacc[0] = fma_(-ms, sk, sacc[0]);
        else if (gid == 1) sacc[1] = fma_(-ms, sk, sacc[1]);
        else if (gid == 2) sacc[2] = fma_(-ms, sk, sacc[2]);
        else sacc[3] = fma_(-ms, sk, sacc[3]);
      } else {
        s = fma_(-ms, sk, s);
      }
    }
  }
  __syncthreads();

  // ---- back substitution, root first --------------------------------------------
  const float di = isdof ? Di[lane] : 0.0f;
  float xv = s * di;
  for (int t = 0; t < P.maxdepth; ++t) {
    if (ddepth == t) X[lane] = xv;
    __syncthreads();
    if (ddepth > t) {
      const int a = col[drow + t];
      const float ms = T[drow + t] * di;
      xv = fma_(-ms, X[a], xv);
    }
  }
  if (isdof) x[(int64_t)w * ldx + lane] = (flags & IM_FLAG_NEGATE) ? -xv : xv;
}

using KernelFn = void (*)(TreeDev, const float *, int64_t, const float *, int,
                          const float *, const int32_t *, const int32_t *, int,
                          const float *, int64_t, float *, int64_t, float *, int,
                          float, int, unsigned, const unsigned char *);

template <int SPL>
KernelFn pick_nvp(int nvp) {
  switch (nvp) {
    case 16: if constexpr (SPL <= 4) return tree_kernel<SPL, 16, true>; else return nullptr;
    case 32: if constexpr (SPL <= 12) return tree_kernel<SPL, 32, true>; else return nullptr;
    case 48: return tree_kernel<SPL, 48, true>;
    case 64: return tree_kernel<SPL, 64, true>;
  }
  return nullptr;
}

KernelFn pick(bool assemble, int spl, int nvp) {
  switch (spl) {
    case 2: return assemble ? pick_nvp<2>(nvp) : tree_kernel<2, 16, false>;
    case 4: return assemble ? pick_nvp<4>(nvp) : tree_kernel<4, 16, false>;
    case 6: return assemble ? pick_nvp<6>(nvp) : tree_kernel<6, 16, false>;
    case 8: return assemble ? pick_nvp<8>(nvp) : tree_kernel<8, 16, false>;
    case 12: return assemble ? pick_nvp<12>(nvp) : tree_kernel<12, 16, false>;
    case 16: return assemble ? pick_nvp<16>(nvp) : tree_kernel<16, 16, false>;
  }
  return nullptr;
}

int round_spl(int need) {
  for (int s : {2, 4, 6, 8, 12, 16})
    if (need <= s) return s;
  return 0;
}

int round_nvp(int nv) {
  for (int s : {16, 32, 48, 64})
    if (nv <= s) return s;
  return 0;
}

// Every float whose bit pattern lies in [first, last]: does the short reciprocal of the pivot
// chain (tree_row16.h) give the bits of the division?  In-range values must, the others are
// counted only when they claim to be in range.
__global__ void check_reciprocal_kernel(uint32_t first, uint32_t last, unsigned long long *mismatches) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  unsigned long long bad = 0;
  for (uint64_t u = (uint64_t)first + blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; u <= last; u += stride) {
    const float x = __builtin_bit_cast(float, (uint32_t)u);
    if (!gen::im_reciprocal_in_range(x)) continue;
    bad += __builtin_bit_cast(uint32_t, gen::im_reciprocal_fast(x)) != __builtin_bit_cast(uint32_t, 1.0f / x);
  }
  if (bad) atomicAdd(mismatches, bad);
}

// Constraint rows whose dofs do not all lie on one root-to-leaf chain: such a row has products
// outside M's pattern, which the fused kernels cannot hold (they are dropped).  One wavefront per
// world, a lane per dof; a row counts when its weight is not zero and some dof with a nonzero
// entry is unrelated to another one.  The check of the reference's sparse assembly
// (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:605-621) on the tree pattern.
__global__ __launch_bounds__(64) void tree_violation_kernel(const uint64_t *__restrict__ related, int nv,
                                                            const float *__restrict__ J, int njmax,
                                                            const float *__restrict__ D,
                                                            const int32_t *__restrict__ state,
                                                            const int32_t *__restrict__ nefc_p, int quad,
                                                            float *__restrict__ violations) {
  const int64_t w = blockIdx.x;
  const int lane = threadIdx.x;
  int ne = nefc_p ? nefc_p[w] : njmax;
  ne = ne < njmax ? ne : njmax;
  const uint64_t mine = lane < nv ? related[lane] : ~0ull;
  const float *Jw = J + w * (int64_t)njmax * nv;
  int bad_rows = 0;
  for (int r0 = 0; r0 < ne; r0 += 4) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // four rows' entries in flight
      const int r = r0 + u < ne ? r0 + u : ne - 1;
      v[u] = lane < nv ? Jw[(int64_t)r * nv + lane] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int r = r0 + u;
      if (r >= ne) break;
      const bool counted = state[w * njmax + r] == quad && D[w * njmax + r] != 0.0f;
      const uint64_t row = __ballot(v[u] != 0.0f);
      const bool off_pattern = v[u] != 0.0f && (row & ~mine) != 0;
      if (counted && __any(off_pattern)) ++bad_rows;
    }
  }
  if (lane == 0 && bad_rows) violations[w] = violations[w] + (float)bad_rows;
}

// One launch of the generated kernels for `niter` iterations (see the kernels' prologue); the
// table-driven kernel takes one iteration at a time.
struct Iterations {
  int niter = 1;
  int64_t state_it = 0, y_it = 0, x_it = 0;
};

int launch(const im_tree_plan *plan, bool assemble, const float *M, int64_t ldM,
           const float *J, int njmax, const float *D, const int32_t *state,
           const int32_t *nefc, int quad, const float *y, int64_t ldy, float *x,
           int64_t ldx, float *Hout, int nworld, unsigned flags, void *stream,
           Iterations its = Iterations(), const unsigned char *skip = nullptr) {
  if (!plan || nworld < 0) return IM_ERR_ARG;
  if (!plan->device_ready) return IM_ERR_UNSUPPORTED;
  if (nworld == 0) return IM_OK;
  if (!M || !y || !x) return IM_ERR_ARG;
  if (ldM < plan->nM || ldy < plan->nv || ldx < plan->nv) return IM_ERR_STRIDE;
  // njmax >= 1: the kernels clamp row indices to njmax - 1
  if (assemble && (!J || !D || !state || njmax <= 0)) return IM_ERR_ARG;
  if (plan->row16) {
    const auto *e = (const gen::Row16Entry *)plan->row16;
    void *args[] = {&M,     &ldM,      &J,         &njmax,        &D,        &state,   &nefc,
                    &quad,  &y,        &ldy,       &x,            &ldx,      &Hout,    &nworld,
                    &flags, &its.niter, &its.state_it, &its.y_it, &its.x_it, &skip};
    // staged rows plus the four worlds' active-row lists (row id and D per constraint row)
    const size_t lds = assemble ? (size_t)e->lds_bytes + 32 * std::max<size_t>(((size_t)njmax + 15) / 16 * 16, 64)
                                : (size_t)e->solve_lds_bytes;
    const void *fn = !assemble ? e->solve : (njmax <= e->short_rows ? e->fused : e->fused_long);
    if (fn && lds <= 160 * 1024) {
      // four wavefronts per four worlds: in the fused kernel each assembles one world, then (in
      // both) wavefront j factors group j of all four and the first one the trunk
      // several iterations: whole rounds of the eight XCDs per iteration (spare workgroups exit)
      const unsigned quads = (unsigned)((nworld + 3) / 4);
      const unsigned grid = its.niter > 1 ? (quads + 7) / 8 * 8 * (unsigned)its.niter : quads;
      if (plan->module)
        IM_HIP_CHECK(hipModuleLaunchKernel((hipFunction_t)fn, grid, 1, 1, 256, 1, 1, (unsigned)lds,
                                           (hipStream_t)stream, args, nullptr));
      else
        IM_HIP_CHECK(hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, (hipStream_t)stream));
      return IM_OK;
    }
  }
  if (!plan->table_driven) return IM_ERR_UNSUPPORTED;  // no generated kernels attached (or they need too much LDS)
  if (its.niter > 1) {  // the table-driven kernel: one launch per iteration
    for (int it = 0; it < its.niter; ++it) {
      const int st = launch(plan, assemble, M, ldM, J, njmax, D, state + it * its.state_it, nefc, quad,
                            y + it * its.y_it, ldy, x + it * its.x_it, ldx, nullptr, nworld, flags, stream,
                            Iterations(), skip);
      if (st != IM_OK) return st;
    }
    return IM_OK;
  }
  const int nv = plan->nv, nM = plan->nM;
  const int nvp = round_nvp(nv);
  int rc = 1, njpad = 0;
  if (assemble) {
    const int cap = std::min(64 * kPF / nv, 64);
    while (rc * 2 <= cap) rc *= 2;
    njpad = (njmax + 63) / 64 * 64 + 64;
  }
  const size_t lds_floats = (size_t)nM * 2 + 64 * 3 + (assemble ? njpad + 2 * (size_t)rc * nvp : 0);
  const size_t lds_bytes = lds_floats * 4;
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  KernelFn fn = pick(assemble, plan->spl, nvp);
  if (!fn) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(64), lds_bytes, (hipStream_t)stream, plan->dev, M,
                     ldM, J, njmax, D, state, nefc, quad, y, ldy, x, ldx, Hout, rc,
                     1.0f / (float)nv, njpad, flags, skip);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

// search . search and grad . x of the tree stage of a Newton iteration, summed as the reference's
// factor stages sum them (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:462-479): lane l of
// a block of `block` lanes adds its dofs l, l + block, .. with fused multiply-adds, every 32 lanes
// fold in a shuffle-down tree, the folds are added in order.  x = -search.  A wavefront per world.
__global__ __launch_bounds__(256) void newton_search_sums_kernel(
    const unsigned char *__restrict__ skip, const float *__restrict__ grad, int64_t ldg,
    const float *__restrict__ search, int64_t lds_, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int block, int nworld) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= nworld || (skip && skip[w])) return;
  float s0 = 0.0f, s1 = 0.0f;
  for (int d = lane; d < nv && lane < block; d += block) {
    const float v = -search[w * lds_ + d];
    s0 = fma_(v, v, s0);
    s1 = fma_(grad[w * ldg + d], v, s1);
  }
  for (int o = 16; o > 0; o >>= 1) {
    s0 = s0 + __shfl_down(s0, o, 32);
    s1 = s1 + __shfl_down(s1, o, 32);
  }
  const float a1 = __shfl(s0, 32, 64), b1 = __shfl(s1, 32, 64);
  if (lane == 0) {
    float ra = 0.0f + s0, rb = 0.0f + s1;
    if (block > 32) ra = ra + a1, rb = rb + b1;
    search_dot[w] = ra;
    decrement[w] = rb;
  }
}

}  // namespace

// Lays the plan out for the kernels: entry e of H sits in lane e % 64, register
// e / 64; steps follow the plan's elimination order with one merge marker
// between the groups and the trunk.
int tree_plan_upload(im_tree_plan *pl) {
  const int nv = pl->nv, nM = pl->nM;
  pl->device_ready = false;
  if (nv > 64 && nv <= 96 && nM <= 1024 && pl->groups.size() <= IM_MAX_GROUPS) {
    // the reference's 68- to 79-dof models: generated kernels only (their lanes follow the chains,
    // not the dofs), attached by the caller; no tables of the table-driven kernel
    pl->table_driven = false;
    pl->row16 = nullptr;
    IM_HIP_CHECK(hipGetDevice(&pl->device));
    pl->device_ready = true;
    return IM_OK;
  }
  if (nv > 64 || nM > 65535 || pl->groups.size() > IM_MAX_GROUPS) return IM_ERR_UNSUPPORTED;
  const int spl = round_spl((nM + 63) / 64);
  if (!spl) return IM_ERR_UNSUPPORTED;
  pl->spl = spl;
  std::vector<char> in_trunk(nv, 0);
  for (int i : pl->trunk) in_trunk[i] = 1;
  std::vector<int32_t> slot_e(spl * 64, -1);
  std::vector<uint32_t> slot_d(spl * 64, 0);
  for (int b = 0; b < nv; ++b)
    for (int q = 0; q < pl->rownnz[b]; ++q) {
      const int e = pl->rowadr[b] + q;
      const int a = pl->colind[e];
      const int idx = (e / 64) * 64 + (e % 64);
      slot_e[idx] = e | (in_trunk[b] ? (1 << 30) : 0);
      slot_d[idx] = (uint32_t)a | ((uint32_t)b << 8) | ((uint32_t)(pl->rownnz[b] - 1) << 16) | ((uint32_t)q << 24);
    }
  std::vector<int4> steps;
  std::vector<uint64_t> anc;
  auto push = [&](int k, int gid) {
    steps.push_back(make_int4(pl->rowadr[k], pl->rownnz[k] - 1, gid, k));
    uint64_t m = 0;
    for (int p = 0; p + 1 < pl->rownnz[k]; ++p) m |= 1ull << pl->colind[pl->rowadr[k] + p];
    anc.push_back(m);
  };
  for (size_t j = 0; j < pl->groups.size(); ++j)
    for (int k : pl->groups[j]) push(k, int(j));
  if (!pl->trunk.empty()) {
    steps.push_back(make_int4(0, 0, -1, 0));
    anc.push_back(0);
    for (auto it = pl->trunk.rbegin(); it != pl->trunk.rend(); ++it) push(*it, IM_MAX_GROUPS);
  }
  std::vector<int32_t> dof_d(64, -1);
  for (int i = 0; i < nv; ++i)
    dof_d[i] = pl->rowadr[i] | ((pl->rownnz[i] - 1) << 16) | (in_trunk[i] ? (1 << 24) : 0);

  // one allocation, 16-byte aligned sections
  auto align = [](size_t v) { return (v + 15) / 16 * 16; };
  size_t off = 0;
  const size_t o_steps = off; off = align(off + steps.size() * sizeof(int4));
  const size_t o_anc = off;   off = align(off + anc.size() * sizeof(uint64_t));
  const size_t o_se = off;    off = align(off + slot_e.size() * 4);
  const size_t o_sd = off;    off = align(off + slot_d.size() * 4);
  const size_t o_dof = off;   off = align(off + dof_d.size() * 4);
  const size_t o_col = off;   off = align(off + (size_t)nM * 4);
  const size_t o_rel = off;   off = align(off + 64 * sizeof(uint64_t));
  // M's pattern row of every dof: itself, its ancestors, its descendants
  std::vector<uint64_t> related(64, 0);
  for (int b = 0; b < nv; ++b)
    for (int q = 0; q < pl->rownnz[b]; ++q) {
      const int a = pl->colind[pl->rowadr[b] + q];
      related[b] |= 1ull << a;
      related[a] |= 1ull << b;
    }
  std::vector<char> blob(off, 0);
  std::memcpy(blob.data() + o_steps, steps.data(), steps.size() * sizeof(int4));
  std::memcpy(blob.data() + o_anc, anc.data(), anc.size() * sizeof(uint64_t));
  std::memcpy(blob.data() + o_se, slot_e.data(), slot_e.size() * 4);
  std::memcpy(blob.data() + o_sd, slot_d.data(), slot_d.size() * 4);
  std::memcpy(blob.data() + o_dof, dof_d.data(), dof_d.size() * 4);
  std::memcpy(blob.data() + o_col, pl->colind.data(), (size_t)nM * 4);
  std::memcpy(blob.data() + o_rel, related.data(), 64 * sizeof(uint64_t));
  IM_HIP_CHECK(hipGetDevice(&pl->device));
  IM_HIP_CHECK(hipMalloc(&pl->dev_blob, off + 16));
  IM_HIP_CHECK(hipMemcpy(pl->dev_blob, blob.data(), off, hipMemcpyHostToDevice));
  char *base = (char *)pl->dev_blob;
  pl->next_world = (int *)(base + off);
  pl->dev.steps = (const int4 *)(base + o_steps);
  pl->dev.anc = (const uint64_t *)(base + o_anc);
  pl->dev.slot_e = (const int32_t *)(base + o_se);
  pl->dev.slot_d = (const uint32_t *)(base + o_sd);
  pl->dev.dof_d = (const int32_t *)(base + o_dof);
  pl->dev.colind = (const int32_t *)(base + o_col);
  pl->dev.related = (const uint64_t *)(base + o_rel);
  pl->dev.nv = nv;
  pl->dev.nM = nM;
  pl->dev.nsteps = int(steps.size());
  pl->dev.maxdepth = pl->maxdepth;
  pl->dev.ngroups = int(pl->groups.size());
  pl->device_ready = true;
  // a kernel generated for exactly this structure and plan, unless the generic one is forced
  const char *force = std::getenv("IMHIP_TREE_KERNEL");
  pl->row16 = (force && std::strcmp(force, "generic") == 0) ? nullptr : (const void *)gen::find_row16(tree_key(*pl));
  if (pl->row16) {
    // the fused kernels stage four dense copies of H in LDS: large trees need more than the
    // default 64 KB of dynamic LDS, which has to be granted before the first launch
    const auto *e = (const gen::Row16Entry *)pl->row16;
    if (e->lds_bytes + 32 * 64 > 48 * 1024) {
      IM_HIP_CHECK(hipFuncSetAttribute(e->fused, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      IM_HIP_CHECK(hipFuncSetAttribute(e->fused_long, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    }
    if (e->solve_lds_bytes > 48 * 1024)
      IM_HIP_CHECK(hipFuncSetAttribute(e->solve, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    // the resident Newton loop keeps its own arrays behind the stage's
    // ... and is used only where it keeps to registers and the runtime grants the LDS
    // (im_newton_solve_tree says unsupported otherwise)
    auto usable = [](const void *fn) {
      hipFuncAttributes fa{};
      const bool ok = hipFuncGetAttributes(&fa, fn) == hipSuccess && fa.localSizeBytes == 0 &&
                      hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          160 * 1024 - (int)fa.sharedSizeBytes) == hipSuccess;
      (void)hipGetLastError();
      return ok;
    };
    pl->resident_ok = usable(e->newton);
    pl->resident_long_ok = usable(e->newton_long);
  }
  return IM_OK;
}

}  // namespace im

namespace im {
__global__ void set_world_counter_kernel(int *counter, int value) { *counter = value; }
}  // namespace im

extern "C" {

int im_tree_factor_solve(const im_tree_plan *plan, const float *M, int64_t ldM,
                         const float *y, int64_t ldy, float *x, int64_t ldx,
                         int nworld, void *stream) {
  return im::launch(plan, false, M, ldM, nullptr, 0, nullptr, nullptr, nullptr, 0, y, ldy,
                    x, ldx, nullptr, nworld, 0u, stream);
}

int im_tree_pattern_violations(const im_tree_plan *plan, const float *J, int njmax, const float *D,
                               const int32_t *state, const int32_t *nefc, int quad, float *violations, int nworld,
                               void *stream) {
  if (!plan || nworld < 0 || njmax < 0) return IM_ERR_ARG;
  if (!plan->device_ready) return IM_ERR_UNSUPPORTED;
  if (!plan->table_driven) return IM_ERR_UNSUPPORTED;  // the relation masks hold 64 dofs
  if (nworld == 0 || njmax == 0) return IM_OK;
  if (!J || !D || !state || !violations) return IM_ERR_ARG;
  hipLaunchKernelGGL(im::tree_violation_kernel, dim3(nworld), dim3(64), 0, (hipStream_t)stream, plan->dev.related,
                     plan->nv, J, njmax, D, state, nefc, quad, violations);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_tree_plan_kernel_key(const im_tree_plan *plan, unsigned long long *key, int *has_kernel) {
  if (!plan || !key) return IM_ERR_ARG;
  *key = im::tree_key(*plan);
  if (has_kernel) *has_kernel = plan->row16 != nullptr;
  return IM_OK;
}

int im_tree_plan_attach_kernels(im_tree_plan *plan, const void *code_object) {
  if (!plan || !code_object) return IM_ERR_ARG;
  if (!plan->device_ready) return IM_ERR_UNSUPPORTED;
  if (plan->module) return IM_ERR_ARG;  // once per plan
  hipModule_t mod = nullptr;
  IM_HIP_CHECK(hipModuleLoadData(&mod, code_object));
  auto fail = [&](int code) {
    (void)hipModuleUnload(mod);
    return code;
  };
  unsigned long long key = 0;
  int info[5] = {0, 0, 0, 0, 0};
  hipDeviceptr_t sym = nullptr;
  size_t bytes = 0;
  if (hipModuleGetGlobal(&sym, &bytes, mod, "im_row16_key") != hipSuccess || bytes != sizeof(key) ||
      hipMemcpyDtoH(&key, sym, sizeof(key)) != hipSuccess)
    return fail(IM_ERR_STRUCTURE);
  if (hipModuleGetGlobal(&sym, &bytes, mod, "im_row16_info") != hipSuccess || bytes != sizeof(info) ||
      hipMemcpyDtoH(info, sym, sizeof(info)) != hipSuccess)
    return fail(IM_ERR_STRUCTURE);
  // the kernels are straight-line code for one structure and plan: anything else would read and
  // write out of place
  if (key != im::tree_key(*plan) || info[0] != plan->nv || info[1] != plan->nM) return fail(IM_ERR_STRUCTURE);
  if (info[2] <= 0 || info[2] + 32 * 64 > 160 * 1024 || info[3] <= 0 || info[4] < 0 || info[4] > info[2])
    return fail(IM_ERR_UNSUPPORTED);
  hipFunction_t fused = nullptr, fused_long = nullptr, solve = nullptr, newton = nullptr, newton_long = nullptr;
  if (hipModuleGetFunction(&fused, mod, "im_row16_fused") != hipSuccess ||
      hipModuleGetFunction(&fused_long, mod, "im_row16_fused_long") != hipSuccess ||
      hipModuleGetFunction(&solve, mod, "im_row16_solve") != hipSuccess)
    return fail(IM_ERR_STRUCTURE);
  if (hipModuleGetFunction(&newton, mod, "im_row16_newton") != hipSuccess ||
      hipModuleGetFunction(&newton_long, mod, "im_row16_newton_long") != hipSuccess) {
    newton = newton_long = nullptr;  // a code object without the resident loop: the stages are launched one by one
    (void)hipGetLastError();
  }
  // a fused kernel that spills registers to memory is not taken: the plan keeps the table-driven
  // kernel (the generator's callers check the code object's descriptors before they get here)
  auto spills = [](hipFunction_t f) {
    int bytes = 0;
    return hipFuncGetAttribute(&bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f) == hipSuccess && bytes > 0;
  };
  if (spills(fused) || spills(fused_long)) return fail(IM_ERR_UNSUPPORTED);
  if (spills(solve)) solve = nullptr;  // im_tree_factor_solve then takes the table-driven kernel
  const bool newton_ok = newton && !spills(newton), newton_long_ok = newton_long && !spills(newton_long);
  if (info[2] + 32 * 64 > 48 * 1024) {
    // more than the default dynamic LDS: asked for here; a runtime that refuses the request for a
    // module's function reports it at the launch
    (void)hipFuncSetAttribute((const void *)fused, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipFuncSetAttribute((const void *)fused_long, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipGetLastError();
  }
  // the resident loop's own arrays come on top of the stage's
  auto grant = [](hipFunction_t f) {
    int fixed = 0;
    (void)hipFuncGetAttribute(&fixed, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f);
    const bool ok = hipFuncSetAttribute((const void *)f, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        160 * 1024 - fixed) == hipSuccess;
    (void)hipGetLastError();
    return ok;
  };
  const bool newton_lds = newton && grant(newton), newton_long_lds = newton_long && grant(newton_long);
  // plain data, released with free() when the plan goes
  auto *e = (im::gen::Row16Entry *)std::malloc(sizeof(im::gen::Row16Entry));
  if (!e) return fail(IM_ERR_ARG);
  *e = im::gen::Row16Entry{key, info[0], info[1], info[2], info[3], "module", (const void *)fused,
                           (const void *)fused_long, (const void *)solve, (const void *)newton,
                           (const void *)newton_long, info[4]};
  if (solve && info[4] > 48 * 1024) {
    (void)hipFuncSetAttribute((const void *)solve, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipGetLastError();
  }
  plan->module = mod;
  plan->resident_ok = newton_ok && newton_lds;
  plan->resident_long_ok = newton_long_ok && newton_long_lds;
  plan->row16_own = e;
  plan->row16 = e;
  return IM_OK;
}

int im_check_reciprocal(uint32_t first_bits, uint32_t last_bits, unsigned long long *mismatches, void *stream) {
  if (!mismatches || last_bits < first_bits) return IM_ERR_ARG;
  hipLaunchKernelGGL(im::check_reciprocal_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, first_bits, last_bits,
                     mismatches);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_assemble_tree_ldl_solve_iters(const im_tree_plan *plan, const float *M, int64_t ldM, const float *J,
                                     int njmax, const float *D, const int32_t *state, int64_t state_iter_stride,
                                     const int32_t *nefc, int quad, const float *grad, int64_t ldg,
                                     int64_t grad_iter_stride, float *x, int64_t ldx, int64_t x_iter_stride,
                                     int nworld, int niter, unsigned flags, void *stream) {
  if (!plan || nworld < 0 || niter < 0 || state_iter_stride < 0 || grad_iter_stride < 0 || x_iter_stride < 0)
    return IM_ERR_ARG;
  if (niter > 1 && (state_iter_stride < (int64_t)nworld * njmax || x_iter_stride < (int64_t)(nworld - 1) * ldx + plan->nv))
    return IM_ERR_STRIDE;  // iterations must not overlap
  if (niter == 0 || nworld == 0) return IM_OK;
  if (!plan->device_ready) return IM_ERR_UNSUPPORTED;
  if (!M || !grad || !x || !J || !D || !state || njmax <= 0) return IM_ERR_ARG;
  if (ldM < plan->nM || ldg < plan->nv || ldx < plan->nv) return IM_ERR_STRIDE;
  im::Iterations its;
  its.niter = niter;
  its.state_it = state_iter_stride;
  its.y_it = grad_iter_stride;
  its.x_it = x_iter_stride;
  return im::launch(plan, true, M, ldM, J, njmax, D, state, nefc, quad, grad, ldg, x, ldx, nullptr, nworld, flags,
                    stream, its);
}

int im_assemble_tree_ldl_solve(const im_tree_plan *plan, const float *M, int64_t ldM,
                               const float *J, int njmax, const float *D,
                               const int32_t *state, const int32_t *nefc, int quad,
                               const float *grad, int64_t ldg, float *x, int64_t ldx,
                               float *Hout, int nworld, unsigned flags, void *stream) {
  return im::launch(plan, true, M, ldM, J, njmax, D, state, nefc, quad, grad, ldg, x, ldx,
                    Hout, nworld, flags, stream);
}

int im_newton_tree_stage(const im_tree_plan *plan, const uint8_t *skip, const float *M, int64_t ldM, const float *J,
                         int njmax, const float *D, const int32_t *state, const int32_t *nefc, int quad,
                         const float *grad, int64_t ldg, float *search, int64_t ld_search, float *search_dot,
                         float *decrement, int block, int nworld, void *stream) {
  if (!search_dot || !decrement || (block != 32 && block != 64)) return IM_ERR_ARG;
  const int st = im::launch(plan, true, M, ldM, J, njmax, D, state, nefc, quad, grad, ldg, search, ld_search, nullptr,
                            nworld, IM_FLAG_NEGATE, stream, im::Iterations(), skip);
  if (st != IM_OK || nworld == 0) return st;
  hipLaunchKernelGGL(im::newton_search_sums_kernel, dim3((unsigned)((nworld + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, skip, grad, ldg, search, ld_search, search_dot, decrement, plan->nv, block,
                     nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_newton_solve_tree(const im_tree_plan *plan, const im_newton_args *p, void *stream) {
  if (!plan || !p || p->nworld < 0) return IM_ERR_ARG;
  if (!plan->device_ready || !plan->row16) return IM_ERR_UNSUPPORTED;
  const auto *e = (const im::gen::Row16Entry *)plan->row16;
  if (!e->newton || !e->newton_long) return IM_ERR_UNSUPPORTED;
  if (p->nworld == 0) return IM_OK;
  const int nv = plan->nv, nM = plan->nM, njmax = p->njmax;
  im::resident::NewtonArgs a{};
  const int bad = im::resident::convert_args(*p, nv, nM, a);
  if (bad != IM_OK) return bad;
  // the factor stage's LDS (its staged tiles and exchange slots plus the four worlds' row lists), or the
  // four wavefronts' staged rows of J where those take more; the loop's own arrays behind it
  const size_t stage_bytes = (size_t)e->lds_bytes + 32 * std::max<size_t>(((size_t)njmax + 15) / 16 * 16, 64);
  const size_t stage_words = std::max(stage_bytes / 4, im::resident::staged_rows_words(nv));
  a.stage_lds_floats = (int)stage_words;
  size_t lds = 4 * (stage_words + im::resident::loop_lds_words(nv, njmax, nM, p->nterm));
  const size_t lds_lean = 4 * (stage_words + im::resident::loop_lds_words(nv, njmax, 0, p->nterm));
  if (lds_lean > 160 * 1024) return IM_ERR_UNSUPPORTED;
  const bool is_long = njmax > e->short_rows;
  if (!(is_long ? plan->resident_long_ok : plan->resident_ok)) return IM_ERR_UNSUPPORTED;  // the kernel spills registers
  const void *fn = is_long ? e->newton_long : e->newton;
  // As many workgroups as the chip keeps resident (registers and LDS); a wavefront whose world is
  // done takes the next world through the plan's counter, so the worlds that need many iterations
  // do not hold three idle wavefronts in place.
  auto resident_per_cu = [&](size_t bytes, int *per_cu) {
    if (plan->module) return hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, (hipFunction_t)fn, 256, bytes);
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, fn, 256, bytes);
  };
  int per_cu = 0, per_cu_lean = 0;
  if (lds <= 160 * 1024) IM_HIP_CHECK(resident_per_cu(lds, &per_cu));
  IM_HIP_CHECK(resident_per_cu(lds_lean, &per_cu_lean));
  // the worlds' rows of M stay in LDS unless leaving them in memory admits another workgroup per CU
  // (snu: 81 KB a workgroup with them, one per CU; 70 KB without, two)
  if (per_cu_lean > per_cu) {
    a.m_lds = 0;
    lds = lds_lean;
    per_cu = per_cu_lean;
  }
  static int ncu = 0;
  if (!ncu) {
    int dev = 0;
    IM_HIP_CHECK(hipGetDevice(&dev));
    IM_HIP_CHECK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
  }
  const int needed = (p->nworld + 3) / 4;
  const unsigned grid = (unsigned)std::min(needed, std::max(1, per_cu) * std::max(1, ncu));
  if ((int)grid < needed) {  // (a batch that is resident all at once has nothing to hand out)
    a.next_world = plan->next_world;
    hipLaunchKernelGGL(im::set_world_counter_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, plan->next_world, (int)grid * 4);
  }
  void *args[] = {&a};
  if (plan->module)
    IM_HIP_CHECK(hipModuleLaunchKernel((hipFunction_t)fn, grid, 1, 1, 256, 1, 1, (unsigned)lds, (hipStream_t)stream, args,
                                       nullptr));
  else
    IM_HIP_CHECK(hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, (hipStream_t)stream));
  return IM_OK;
}

}  // extern "C"
