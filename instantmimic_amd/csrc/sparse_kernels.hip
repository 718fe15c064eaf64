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
// The tables come from the host planner (sparse_plan.cpp) instead of generated source; team widths and block width are the plan's, so the
// order in which a team sums an entry's terms is the reference's.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <vector>

#include "common.h"
#include "newton_wave.h"
#include "sparse_plan.h"

namespace im {
namespace {

struct SparseDev {
  const int32_t *t[NHOST];
  int nv, nv_pad, nslots, nlevels;
};

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// element `index` of an array whose base is the same for the whole wavefront: an unsigned
// 32-bit offset lets the load take the base from scalar registers
template <class T>
__device__ __forceinline__ T ld_u32(const T *base, uint32_t index) {
  return *(const T *)((const char *)base + (size_t)(index * (uint32_t)sizeof(T)));
}

// value of the lane N places up in the caller's row of 16 lanes (0 past the row's end)
template <int N>
__device__ __forceinline__ float row_shl(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + N, 0xF, 0xF, true));
}

// Orders LDS writes before later reads: across the workgroup, or, when a world belongs to
// one wavefront (WAVE), across that wavefront only.
template <bool WAVE>
__device__ __forceinline__ void sync_world() {
  if (WAVE) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  } else {
    __syncthreads();
  }
}

// level-scheduled numeric factor: team lanes stride an entry's terms, shuffle-down tree.
// An entry's value depends on its team width only, not on how many teams work side by side,
// so `block` may be any multiple of the widest team.
// One level with the team width T as a compile-time constant: the operands of a lane's next four
// terms then lie at constant distances, which the LDS instructions carry themselves.
template <bool WAVE, int T>
__device__ __forceinline__ void factor_level(const SparseDev &P, float *N, float *iD, int lane, int block, int e0,
                                             int e1) {
  const int32_t *ESt = P.t[ES], *ECt = P.t[EC], *RPt = P.t[RP];
  const uint32_t *RABt = (const uint32_t *)P.t[RAB], *RKLt = (const uint32_t *)P.t[RKL];
  constexpr int tshift = __builtin_ctz((unsigned)T);
  const int tl = lane & (T - 1), team = lane >> tshift, teams = block >> tshift;
  for (int eb = e0; eb < e1; eb += teams) {
    const int e = eb + team;
    float v = 0.0f;
    int sl = 0, col = -1;
    if (e < e1) {
      sl = ESt[e];
      col = ECt[e];
      for (int r = RPt[e]; r < RPt[e + 1]; ++r) {
        const uint32_t ab = RABt[r], kl = RKLt[r];
        const float *pa = N + (ab & 0xFFFFu) + tl, *pb = N + (ab >> 16) + tl, *pd = iD + (kl & 0xFFFFu) + tl;
        const int len = (int)(kl >> 16) - tl;  // terms from this lane's first on
        // four terms' operands are read before the first is used; the sum keeps its order
        int t = 0;
        for (; t + 3 * T < len; t += 4 * T) {
          const float a0 = pa[t], b0 = pb[t], d0 = pd[t];
          const float a1 = pa[t + T], b1 = pb[t + T], d1 = pd[t + T];
          const float a2 = pa[t + 2 * T], b2 = pb[t + 2 * T], d2 = pd[t + 2 * T];
          const float a3 = pa[t + 3 * T], b3 = pb[t + 3 * T], d3 = pd[t + 3 * T];
          v = fma_(a0 * b0, d0, v);
          v = fma_(a1 * b1, d1, v);
          v = fma_(a2 * b2, d2, v);
          v = fma_(a3 * b3, d3, v);
        }
        for (; t < len; t += T) v = fma_(pa[t] * pb[t], pd[t], v);
      }
    }
    // shuffle-down tree of the team; inside a row of 16 lanes a DPP shift does it (what a lane
    // past the team's end receives is never passed on to the team's first lane)
    if (T > 32) v = v + __shfl_down(v, 32, 64);
    if (T > 16) v = v + __shfl_down(v, 16, 64);
    if (T > 8) v = v + row_shl<8>(v);
    if (T > 4) v = v + row_shl<4>(v);
    if (T > 2) v = v + row_shl<2>(v);
    if (T > 1) v = v + row_shl<1>(v);
    if (e < e1 && tl == 0) {
      const float wv = N[sl] - v;
      N[sl] = wv;
      if (col >= 0) iD[col] = 1.0f / wv;
    }
  }
}

template <bool WAVE = false>
__device__ __forceinline__ void factor_levels(const SparseDev &P, float *N, float *iD, int lane, int block) {
  const int32_t *LPt = P.t[LP], *LTt = P.t[LT];
  for (int l = 0; l < P.nlevels; ++l) {
    const int e0 = LPt[l], e1 = LPt[l + 1];
    switch (LTt[l]) {  // team widths are powers of two
      case 1: factor_level<WAVE, 1>(P, N, iD, lane, block, e0, e1); break;
      case 2: factor_level<WAVE, 2>(P, N, iD, lane, block, e0, e1); break;
      case 4: factor_level<WAVE, 4>(P, N, iD, lane, block, e0, e1); break;
      case 8: factor_level<WAVE, 8>(P, N, iD, lane, block, e0, e1); break;
      case 16: factor_level<WAVE, 16>(P, N, iD, lane, block, e0, e1); break;
      case 32: factor_level<WAVE, 32>(P, N, iD, lane, block, e0, e1); break;
      default: factor_level<WAVE, 64>(P, N, iD, lane, block, e0, e1); break;
    }
    sync_world<WAVE>();
  }
}

// backward pushes by level (root first), search = -x, (x.x, g.x) reduced warp then block.
// `nthreads` lanes work on the world; the two dot products are summed as a block of `block`
// lanes would (the plan's width: it fixes which terms a lane adds and in which order).
template <bool WAVE = false>
__device__ __forceinline__ void backward_sums(const SparseDev &P, float *N, const float *iD,
                                              const float *__restrict__ gw, float *__restrict__ search,
                                              float *red, float *search_dot, float *decrement, int lane,
                                              int nthreads, int block, const uint32_t *staged = nullptr) {
  const int n = P.nv, rhs = P.nslots - n, nw = (block + 31) / 32;
  const int32_t *ORIGt = P.t[ORIG];
  // backward solve, root level first
  const int32_t *BLt = P.t[BL], *BSt = P.t[BS], *BIt = P.t[BI], *BJt = P.t[BJ];
  if (staged) {  // the tables from LDS (stage_backward_tables): no level waits for memory
    const uint32_t *lev = staged, *push = staged + P.nlevels + 1;
    for (int l = 0; l < P.nlevels; ++l) {
      for (int p = lev[l] + lane; p < (int)lev[l + 1]; p += nthreads) {
        const uint32_t u = push[p];
        const int i = (u >> 16) & 0xFF, j = u >> 24;
        N[rhs + j] = fma_(-N[u & 0xFFFFu], N[rhs + i] * iD[i], N[rhs + j]);
      }
      sync_world<WAVE>();
    }
  } else {
    for (int l = 0; l < P.nlevels; ++l) {
      for (int p = BLt[l] + lane; p < BLt[l + 1]; p += nthreads) {
        const int i = BIt[p], j = BJt[p];
        N[rhs + j] = fma_(-N[BSt[p]], N[rhs + i] * iD[i], N[rhs + j]);
      }
      sync_world<WAVE>();
    }
  }
  float s0 = 0.0f, s1 = 0.0f;
  for (int j = lane; j < n && lane < block; j += block) {
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
  if ((lane & 31) == 0 && lane < block) {
    red[lane >> 5] = s0;
    red[nw + (lane >> 5)] = s1;
  }
  sync_world<WAVE>();
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

// dst[i] = f(i) for i < count, a lane's next eight values asked for before the first is stored: a
// plain loop waits for every load in turn, and a world's lanes are few.
template <class F>
__device__ __forceinline__ void fill_lds(float *dst, int count, int lane, int block, const F &f) {
  for (int i0 = lane; i0 < count; i0 += 8 * block) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * block;
      v[u] = f(i < count ? i : count - 1);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * block;
      if (i < count) dst[i] = v[u];
    }
  }
}

// The backward solve's tables in LDS for backward_sums: [nlevels + 1] first push of each level, then a
// word per push (slot of the factor entry | row << 16 | column << 24).  For up to 256 dofs and
// 65535 slots; a barrier must follow before backward_sums reads them.  nlevels + 1 + pushes words.
__device__ __forceinline__ void stage_backward_tables(const SparseDev &P, uint32_t *staged, int lane, int block) {
  const int32_t *BLt = P.t[BL], *BSt = P.t[BS], *BIt = P.t[BI], *BJt = P.t[BJ];
  for (int l = lane; l <= P.nlevels; l += block) staged[l] = (uint32_t)BLt[l];
  uint32_t *push = staged + P.nlevels + 1;
  fill_lds((float *)push, BLt[P.nlevels], lane, block, [&](int p) {
    return __builtin_bit_cast(float, (uint32_t)BSt[p] | ((uint32_t)BIt[p] << 16) | ((uint32_t)BJt[p] << 24));
  });
}

// Forward substitution with a stored factor: N[rhs + j] = g[j] - sum_k (N[j,k] / D[k]) N[rhs + k],
// a lane per row of a level, the row's terms in order.  The rows' tables (row, slot of its first
// term, place and count of its columns) and the gradient come into LDS first, all rows at once:
// read level by level from memory, each level waited for three memory round trips in a row.
// The column numbers of every term come in as 16-bit words: a row's chain of up to n terms runs on
// one lane, and a trip to memory per handful of terms was most of the kernel.
// `meta` holds 4 n + 2 + (nfac + 1) / 2 words.
__device__ __forceinline__ void forward_rhs_levels(const SparseDev &P, float *N, const float *iD,
                                                   const float *__restrict__ gw, int rhs, int *meta, int lane,
                                                   int block) {
  const int n = P.nv;
  const int32_t *ORIGt = P.t[ORIG];
  const int32_t *FLt = P.t[FL], *FRt = P.t[FR], *RSt = P.t[RS], *RKPt = P.t[RKP], *RKt = P.t[RK];
  int *row = meta, *first = meta + n, *cols = meta + 2 * n, *level = meta + 3 * n;  // level: [nlevels + 1]
  for (int q = lane; q < n; q += block) {
    const int j = FRt[q], k0 = RKPt[j];
    row[q] = j | ((RKPt[j + 1] - k0) << 16);
    first[q] = RSt[j];
    cols[q] = k0;
    N[rhs + q] = gw[ORIGt[q]];
  }
  for (int l = lane; l <= P.nlevels; l += block) level[l] = FLt[l];
  unsigned short *rk = (unsigned short *)(meta + 4 * n + 2);  // [nfac] columns of the terms, row after row
  for (int e0 = lane, nrk = RKPt[n]; e0 < nrk; e0 += 8 * block) {  // nrk <= nfac
    int kk[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) kk[u] = RKt[e0 + u * block < nrk ? e0 + u * block : nrk - 1];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (e0 + u * block < nrk) rk[e0 + u * block] = (unsigned short)kk[u];
  }
  __syncthreads();
  for (int l = 0; l < P.nlevels; ++l) {
    for (int q = level[l] + lane; q < level[l + 1]; q += block) {
      const int j = row[q] & 0xFFFF, len = row[q] >> 16, k0 = cols[q];
      float v = N[rhs + j];
      const float *rowp = N + first[q];
      // whole batches of eight terms without a condition (operand addresses differ by constants
      // that the LDS instructions carry), then the rest one by one
      const unsigned short *kp = rk + k0;
      const float *xs = N + rhs;
      int t = 0;
      for (; t + 8 <= len; t += 8) {
        int k[8];
        float c[8], xk[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) k[u] = kp[t + u];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          c[u] = -(rowp[t + u] * iD[k[u]]);
          xk[u] = xs[k[u]];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) v = fma_(c[u], xk[u], v);
      }
      for (; t < len; ++t) {
        const int k = kp[t];
        v = fma_(-(rowp[t] * iD[k]), xs[k], v);
      }
      N[rhs + j] = v;
    }
    __syncthreads();
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
  backward_sums(P, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, block, block);
}

// ---- initial factor, one wavefront per world --------------------------------------------
// Four worlds per workgroup share one LDS copy of the factor and solve tables; each world
// belongs to one wavefront, so its LDS traffic needs no workgroup barrier.  J'DJ is summed
// on the matrix cores: v_mfma_f32_16x16x4_f32 adds its four products to the accumulator one
// after the other with a fused multiply-add each, rows ascending, which is the order and
// rounding of `v = fmaf(J[r][a] * Dc[r], J[r][b], v)` when one operand is the rounded
// product J[r][a] * Dc[r]; the accumulators start from M.  The lower-triangle 16 x 16 tiles
// hold every (a, b) pair, and the plan's slots pick theirs (pairs outside the pattern are
// dropped, as in the reference, and their rows counted).
constexpr int kStaged = 12;  // tables LP .. BJ, the ones the factor and the solves read
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct SparseWave {
  SparseDev P;
  int staged[kStaged];        // offsets in words from the first table (the plan stores them back to back)
  int staged_words;           // length of that stretch, a multiple of 4
  int solve[5];               // update stage only: offsets of the forward-solve tables FL .. RK from FL
  int solve_words;            // length of that stretch, a multiple of 4 (0: not staged)
  const int32_t *tile_index;  // [tile][4][64]: (index into M + 1) << 16 | (slot + 1), 0 = none
  int block, nM;              // the plan's block width; length of a row of M
  int staged_rows;            // update stage: changed rows of J a world keeps in LDS, 16 or 32 (more are read from memory)
};

template <int NT>
__global__ __launch_bounds__(256, 4) void sparse_init_mfma_kernel(
    SparseWave A, const uint8_t *__restrict__ done, const int32_t *__restrict__ nefc_p,
    const float *__restrict__ J, int njmax, const float *__restrict__ D,
    const int32_t *__restrict__ state, int quad, const float *__restrict__ M, int ldM,
    const float *__restrict__ grad, int ldg, float *__restrict__ U_, float *__restrict__ search_,
    float *__restrict__ search_dot, float *__restrict__ decrement, int nworld) {
  constexpr int NTILE = NT * (NT + 1) / 2, PD = NT >= 4 ? 4 : NT == 3 ? 6 : 8;
  extern __shared__ float lds[];
  const int tid = threadIdx.x, lane = tid & 63, p = lane & 15, kq = lane >> 4;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: world data is addressed from scalar registers
  SparseDev Q = A.P;
  int32_t *tab = (int32_t *)lds;
  {
    // one flat copy, every load issued before the first store (up to 32 KB)
    const int4 *src = (const int4 *)A.P.t[0];
    const int nvec = A.staged_words >> 2;
    int4 buf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = i * 256 + tid;
      buf[i] = src[q < nvec ? q : nvec - 1];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = i * 256 + tid;
      if (q < nvec) ((int4 *)tab)[q] = buf[i];
    }
  }
#pragma unroll
  for (int i = 0; i < kStaged; ++i) Q.t[i] = tab + A.staged[i];
  const int off = A.staged_words;
  __syncthreads();  // the only workgroup barrier: worlds are independent from here on
  const int w = blockIdx.x * 4 + wv;
  if (w >= nworld || (done && done[w])) return;
  const int n = Q.nv, nslots = Q.nslots, nfac = nslots - n, rhs = nfac;
  const int nw = (A.block + 31) / 32;
  const int njp = (njmax + 3) & ~3, factor_words = (nslots + n + 2 * nw + 3) & ~3;
  const int per_world = factor_words + 2 * njp;
  float *N = lds + ((off + 3) & ~3) + wv * per_world;  // [nslots]; a row of M before the factor
  float *iD = N + nslots;                              // [n]
  float *red = iD + n;                                 // [2][nw]
  float *dl = N + factor_words;                        // [njp] weights of the listed constraint rows
  int *rowl = (int *)(dl + njp);                       // [njp] their numbers
  float *U = U_ + (size_t)w * Q.nv_pad * Q.nv_pad;
  const float *Mw = M + (size_t)w * ldM;
  const float *gw = grad + (size_t)w * ldg;
  const float *Jw = J + (size_t)w * njmax * n;
  const float *Dw = D + (size_t)w * njmax;
  const int32_t *sw = state + (size_t)w * njmax;
  int ne = nefc_p[w];
  ne = ne < njmax ? ne : njmax;
  ne = __builtin_amdgcn_readfirstlane(ne);

  // Every load below is unconditional (clamped address, value selected afterwards) and what
  // is needed first is requested first, so that each wait counts only the loads before it.
  // where in M each accumulator element starts from: two 16-bit indices a word (behind the tile table)
  int tmi[NTILE][2];
#pragma unroll
  for (int t = 0; t < NTILE; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) tmi[t][h] = A.tile_index[NTILE * 256 + (t * 2 + h) * 64 + lane];
  float mv[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const int e = c * 64 + lane;
    mv[c] = Mw[e < A.nM ? e : A.nM - 1];
  }
  int col[NT];
  bool colok[NT];
  const int words = (n + 31) / 32;
  const uint32_t *PMt = (const uint32_t *)Q.t[PM];
#pragma unroll
  for (int c = 0; c < NT; ++c) {
    colok[c] = 16 * c + p < n;
    col[c] = colok[c] ? 16 * c + p : n - 1;
  }
  // dofs outside the pattern row of dof `lane` (none for lanes past the last dof)
  unsigned long long npm;
  {
    const int dl = lane < n ? lane : n - 1;
    const uint32_t lo = PMt[dl * words], hi = PMt[dl * words + (words > 1 ? 1 : 0)];
    npm = ~((unsigned long long)lo | (words > 1 ? (unsigned long long)hi << 32 : 0ull));
    if (lane >= n) npm = 0ull;
  }
  // The first 4 PD rows are requested as they are, before anything is known of them; of the rows
  // behind them only the contributing ones are read at all: their numbers and weights go into a
  // list in row order (ballot and prefix count, 64 rows at a time), so a skipped row is one
  // that would have added (J * 0) * J everywhere.
  float g[PD][NT], gd[PD];
  int gs[PD];
  bool gv[PD];  // the register set holds a row below nefc
#pragma unroll
  for (int u = 0; u < PD; ++u) {
    const int row = 4 * u + kq, rowc = row < njmax ? row : njmax - 1;
#pragma unroll
    for (int c = 0; c < NT; ++c) g[u][c] = ld_u32(Jw, (uint32_t)(rowc * n + col[c]));
    gd[u] = ld_u32(Dw, (uint32_t)rowc);
    gs[u] = ld_u32(sw, (uint32_t)rowc);
    gv[u] = row < ne;
  }
  int cnt = 0;
  for (int r0 = 4 * PD; r0 < ne; r0 += 64) {  // the same trips for every lane
    const int r = r0 + lane, rc = r < njmax ? r : njmax - 1;
    const int sv = sw[rc];
    const float dv = Dw[rc];
    const bool act = r < ne && sv == quad;
    const unsigned long long tm = __ballot(act);
    if (act) {
      const int pos = cnt + __popcll(tm & ((1ull << lane) - 1ull));
      dl[pos] = dv;
      rowl[pos] = r;
    }
    cnt += __popcll(tm);
  }
  const int steps = ne > 4 * PD ? PD + ((cnt + 3) >> 2) : (ne + 3) >> 2;
#pragma unroll
  for (int c = 0; c < 16; ++c)
    if (c * 64 + lane < A.nM) N[c * 64 + lane] = mv[c];
  sync_world<true>();
  f32x4 acc[NTILE];
#pragma unroll
  for (int t = 0; t < NTILE; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int mi = ((tmi[t][v >> 1] >> (16 * (v & 1))) & 0xFFFF) - 1;
      const float m = N[mi < 0 ? 0 : mi];
      acc[t][v] = mi >= 0 ? m : 0.0f;
    }
  sync_world<true>();
  int nbad = 0;
  for (int s0 = 0; s0 < steps; s0 += PD) {
#pragma unroll
    for (int u = 0; u < PD; ++u) {
      if (s0 + u < steps) {
        const bool rv = gv[u];
        const float d = (rv && gs[u] == quad) ? gd[u] : 0.0f;
        float z[NT], e[NT];
#pragma unroll
        for (int c = 0; c < NT; ++c) {
          z[c] = rv ? g[u][c] : 0.0f;
          e[c] = z[c] * d;
        }
        {
          int t = 0;
#pragma unroll
          for (int ti = 0; ti < NT; ++ti)
#pragma unroll
            for (int tj = 0; tj <= ti; ++tj, ++t)
              acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(z[ti], e[tj], acc[t], 0, 0, 0);
        }
        // An active row whose dofs do not all lie in one another's pattern row is counted.  The
        // four rows' supports are assembled from the ballots with scalar instructions; lane d
        // then tests dof d of each row against the dofs outside its pattern row.
        const bool dnz = d != 0.0f;
        uint32_t blo[4] = {0u, 0u, 0u, 0u}, bhi[4] = {0u, 0u, 0u, 0u};  // rows 0, 1 | rows 2, 3 of a 16-dof block
#pragma unroll
        for (int c = 0; c < NT; ++c) {
          const unsigned long long b = __ballot(dnz & colok[c] & (z[c] != 0.0f));
          blo[c] = (uint32_t)b;
          bhi[c] = (uint32_t)(b >> 32);
        }
        // 16-bit transposition: row k's support = its 16 bits of every block side by side
        const uint32_t s0l = (blo[0] & 0xFFFFu) | (blo[1] << 16), s0h = (blo[2] & 0xFFFFu) | (blo[3] << 16);
        const uint32_t s1l = (blo[0] >> 16) | (blo[1] & 0xFFFF0000u), s1h = (blo[2] >> 16) | (blo[3] & 0xFFFF0000u);
        const uint32_t s2l = (bhi[0] & 0xFFFFu) | (bhi[1] << 16), s2h = (bhi[2] & 0xFFFFu) | (bhi[3] << 16);
        const uint32_t s3l = (bhi[0] >> 16) | (bhi[1] & 0xFFFF0000u), s3h = (bhi[2] >> 16) | (bhi[3] & 0xFFFF0000u);
        const uint32_t nl = (uint32_t)npm, nh = (uint32_t)(npm >> 32);
        const unsigned long long sup0 = ((unsigned long long)s0h << 32) | s0l, sup1 = ((unsigned long long)s1h << 32) | s1l;
        const unsigned long long sup2 = ((unsigned long long)s2h << 32) | s2l, sup3 = ((unsigned long long)s3h << 32) | s3l;
        nbad += (__ballot(((s0l & nl) | (s0h & nh)) != 0u) & sup0) != 0ull;
        nbad += (__ballot(((s1l & nl) | (s1h & nh)) != 0u) & sup1) != 0ull;
        nbad += (__ballot(((s2l & nl) | (s2h & nh)) != 0u) & sup2) != 0ull;
        nbad += (__ballot(((s3l & nl) | (s3h & nh)) != 0u) & sup3) != 0ull;
      }
      // Next use of this register set.  Issued whether or not the step above ran, so that the
      // number of loads in flight at every wait is the same on every path.
      // (step s0 + u + PD: entries 4 (s0 + u) .. + 3 of the list; past its end row 0 with weight 0)
      const int li = 4 * (s0 + u) + kq;
      const bool lv = li < cnt;
      const int nrowc = lv ? rowl[li] : 0;
#pragma unroll
      for (int c = 0; c < NT; ++c) g[u][c] = ld_u32(Jw, (uint32_t)(nrowc * n + col[c]));
      gd[u] = lv ? dl[li] : 0.0f;
      gs[u] = quad;
      gv[u] = lv;
    }
  }
  // the slots of this lane's accumulator elements (all requested before the first is used)
  int tix[NTILE][4];
#pragma unroll
  for (int t = 0; t < NTILE; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) tix[t][v] = A.tile_index[(t * 4 + v) * 64 + lane];
#pragma unroll
  for (int t = 0; t < NTILE; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int sl = (tix[t][v] & 0xFFFF) - 1;
      if (sl >= 0) N[sl] = acc[t][v];
    }
  sync_world<true>();
  for (int s = lane; s < nfac; s += 64) U[s] = N[s];
  const int32_t *ORIGt = Q.t[ORIG];
  for (int j = lane; j < n; j += 64) N[rhs + j] = gw[ORIGt[j]];
  sync_world<true>();
  factor_levels<true>(Q, N, iD, lane, 64);
  for (int s = lane; s < nfac; s += 64) U[nfac + s] = N[s];
  for (int j = lane; j < n; j += 64) U[2 * nfac + j] = iD[j];
  backward_sums<true>(Q, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, 64,
                      A.block);
  if (nbad && lane == 0) atomicAdd(U + Q.nv_pad * Q.nv_pad - 1, (float)nbad);
}

// Per-iteration factor stage, one wavefront per world (WAVES worlds per workgroup share the LDS
// copy of the factor and solve tables: four, eight or sixteen, chosen by the launcher).  Same arithmetic as
// sparse_update_kernel below; the changed constraint rows are staged in LDS (up to A.staged_rows
// of them, else they are read from memory), packed H is updated in LDS and written back whole,
// and a lane keeps four pairs' table look-ups in flight.
// a dof's elements of the staged rows lie side by side, one word more than rows per dof (17 or 33): lanes that
// read different dofs meet in no LDS bank.  32 rows where that costs a CU no world, 16 otherwise.
constexpr int kStagedRowsMax = 32;

// The factor and solve tables of a plan into LDS, for a workgroup of T threads (a flat 16-byte copy,
// every load issued before the first store); Q's table pointers then address the copy.
template <int T>
__device__ __forceinline__ void stage_update_tables(const SparseWave &A, SparseDev &Q, float *lds, int tid) {
  int32_t *tab = (int32_t *)lds;
  {
    const int4 *src = (const int4 *)A.P.t[0];
    const int nvec = A.staged_words >> 2;
    constexpr int NB = (2048 + T - 1) / T;  // the host admits at most 8192 words
    int4 buf[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int q = i * T + tid;
      buf[i] = src[q < nvec ? q : nvec - 1];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int q = i * T + tid;
      if (q < nvec) ((int4 *)tab)[q] = buf[i];
    }
  }
#pragma unroll
  for (int i = 0; i < kStaged; ++i) Q.t[i] = tab + A.staged[i];
  {
    // forward-solve tables (at most 16 KB), behind the first stretch
    const int4 *src = (const int4 *)A.P.t[FL];
    const int nvec = A.solve_words >> 2;
    constexpr int NB = (1024 + T - 1) / T;  // at most 4096 words
    int4 buf[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int q = i * T + tid;
      buf[i] = src[q < nvec ? q : 0];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int q = i * T + tid;
      if (q < nvec) ((int4 *)(tab + A.staged_words))[q] = buf[i];
    }
#pragma unroll
    for (int i = 0; i < 5; ++i) Q.t[FL + i] = tab + A.staged_words + A.solve[i];
  }
}
__host__ __device__ inline int update_world_words(int nslots, int n, int block, int staged_rows) {
  const int nw = (block + 31) / 32;
  return (nslots + n + 2 * nw + 2 * n + (staged_rows + 1) * n + staged_rows + 3) & ~3;
}

// The stage for one world and one wavefront (`world_lds`: update_world_words of LDS of its own).
__device__ __forceinline__ void sparse_update_world(
    const SparseWave &A, const SparseDev &Q, float *world_lds, const int32_t *__restrict__ changes,
    const int32_t *__restrict__ ids, int ld_ids, const float *__restrict__ J, int njmax,
    const float *__restrict__ D, const int32_t *__restrict__ state, int quad, const float *__restrict__ grad, int ldg,
    float *__restrict__ U_, int32_t *__restrict__ uni_, float *__restrict__ search_, float *__restrict__ search_dot,
    float *__restrict__ decrement, int w, int lane_in) {
  // The lane number through an opaque step: inside a resident loop the addresses formed from it
  // are then worked out where a round uses them instead of each holding a register from round to round.
  int lane = lane_in;
  asm volatile("" : "+v"(lane));
  const int n = Q.nv, nslots = Q.nslots, nfac = nslots - n, rhs = nfac;
  const int nw = (A.block + 31) / 32;
  float *N = world_lds;  // [nslots]
  float *iD = N + nslots;                            // [n]
  float *red = iD + n;                               // [2][nw]
  int *ul = (int *)(red + 2 * nw);                   // [n] ascending dofs touched by the changed rows
  unsigned *mkl = (unsigned *)(ul + n);              // [n] per dof: bit t set where staged row t is nonzero there
  const int cap = A.staged_rows, stride = cap + 1;
  float *jr = (float *)(mkl + n);                    // [n][stride] changed rows of J, a dof's elements together
  float *sd = jr + stride * n;                       // [cap] D of the row, negated for a row that left the quadratic state
  float *U = U_ + (size_t)w * Q.nv_pad * Q.nv_pad;
  const float *gw = grad + (size_t)w * ldg;
  const float *Jw = J + (size_t)w * njmax * n;
  const float *Dw = D + (size_t)w * njmax;
  const int32_t *sw = state + (size_t)w * njmax, *idw = ids + (size_t)w * ld_ids;
  const int32_t *ORIGt = Q.t[ORIG];
  int count = changes[w];
  count = count < ld_ids ? count : ld_ids;
  count = __builtin_amdgcn_readfirstlane(count);
#ifdef IM_NEWTON_STAMPS  // development aid: time per part of the stage, summed over the rounds, left in the world's dof-union row
  long long t_last = wall_clock64();
#define IM_SSTAMP(k) do { const long long t_now = wall_clock64(); if (lane == 0) uni_[(size_t)w * (n + 1) + (k)] += (int)(t_now - t_last); t_last = wall_clock64(); } while (0)
#else
#define IM_SSTAMP(k) do {} while (0)
#endif
  if (count > 0) {
    const bool staged = count <= cap;
    const bool masked = !staged && count <= 128 && 2 * count + 4 * n <= stride * n + cap;
    // requests first: the changed rows, their weights, packed H
    bool hit = false;  // whether a changed row touches this lane's dof
    if (staged) {
      const int tq = lane < count ? lane : count - 1;
      const int rq = idw[tq];
      const float dq = Dw[rq];
      const int sq = sw[rq];
      for (int s = lane; s < nfac; s += 64) N[s] = U[s];
      if (lane < cap) sd[lane] = sq == quad ? dq : -dq;
      unsigned mk = 0u;
      float *mine = jr + (lane < n ? lane : 0) * stride;
      // sixteen rows at a time: their elements of this lane's dof asked for together
#pragma unroll
      for (int half = 0; half < kStagedRowsMax / 16; ++half) {
        if (16 * half >= count) break;  // the same for every lane
        float rowv[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          const int r = __builtin_amdgcn_readlane(rq, 16 * half + t);  // (lanes at or past count hold row count - 1)
          rowv[t] = Jw[r * n + (lane < n ? lane : n - 1)];
        }
        if (lane < n) {
#pragma unroll
          for (int t = 0; t < 16; ++t) {
            if (16 * half + t < count) {
              mine[16 * half + t] = rowv[t];
              mk |= (unsigned)(rowv[t] != 0.0f) << (16 * half + t);
            }
          }
        }
      }
      if (lane < n) {
        mkl[lane] = mk;
        hit = mk != 0u;
      }
    } else if (masked) {
      // more rows than the staged capacity: their numbers, their weights and a mask of up to 128
      // rows per dof go where the staged rows would lie; J's elements then come from memory, but
      // only those of the rows that a pair's two dofs share
      int *rid = (int *)jr;                         // [count]
      float *sdv = jr + count;                      // [count]
      unsigned *mk4 = (unsigned *)(jr + 2 * count);  // [n][4]
      for (int s = lane; s < nfac; s += 64) N[s] = U[s];
      for (int t = lane; t < count; t += 64) {
        const int r = idw[t];
        rid[t] = r;
        sdv[t] = sw[r] == quad ? Dw[r] : -Dw[r];
      }
      unsigned any = 0u;
#pragma unroll
      for (int word = 0; word < 4; ++word) {
        unsigned mk = 0u;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int t0 = 32 * word + 16 * half;
          if (t0 >= count) break;  // the same for every lane
          float rowv[16];
#pragma unroll
          for (int t = 0; t < 16; ++t) rowv[t] = Jw[idw[t0 + t < count ? t0 + t : count - 1] * n + (lane < n ? lane : n - 1)];
#pragma unroll
          for (int t = 0; t < 16; ++t)
            if (t0 + t < count) mk |= (unsigned)(rowv[t] != 0.0f) << (16 * half + t);
        }
        if (lane < n) mk4[4 * lane + word] = mk;
        any |= mk;
      }
      hit = lane < n && any != 0u;
    } else {
      for (int s = lane; s < nfac; s += 64) N[s] = U[s];
      if (lane < n)
        for (int t = 0; t < count && !hit; ++t) hit = Jw[idw[t] * n + lane] != 0.0f;
    }
    // dofs touched by the changed rows, ascending (n <= 64: one ballot)
    const unsigned long long mask = __ballot(hit);
    const int nu = __popcll(mask);
    if (hit) ul[__popcll(mask & ((1ull << lane) - 1ull))] = lane;
    int32_t *uni = uni_ + (size_t)w * (n + 1);
#ifndef IM_NEWTON_STAMPS
    if (hit) uni[__popcll(mask & ((1ull << lane) - 1ull))] = lane;
    if (lane == 0) uni[n] = nu;
#endif
    const int32_t *PAIRt = Q.t[PAIR];
    int nbad = 0;
    sync_world<true>();  // `ul`, `mkl` and the staged rows are read from here on
    IM_SSTAMP(0);
    const int npair = nu * (nu + 1) / 2;
    for (int e0 = lane; e0 < npair; e0 += 4 * 64) {
      int row[4], col[4], sl[4];
      bool live[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        live[k] = e0 + 64 * k < npair;
        const int e = live[k] ? e0 + 64 * k : npair - 1;
        // e = cj (cj + 1) / 2 + ri with ri <= cj, found exactly (walking the pairs in 8 x 8 blocks
        // of (ri, cj) instead, without this arithmetic, was measured a quarter slower)
        int cj = (int)((sqrtf((float)(8 * e + 1)) - 1.0f) * 0.5f);
        while ((cj + 1) * (cj + 2) / 2 <= e) ++cj;
        while (cj * (cj + 1) / 2 > e) --cj;
        row[k] = ul[e - cj * (cj + 1) / 2];
        col[k] = ul[cj];
        sl[k] = PAIRt[row[k] * n + col[k]];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float delta = 0.0f;
        if (staged) {
          // only the rows in which both dofs are nonzero add to the pair, ascending: most pairs
          // of the union share no row at all
          const float *jrow = jr + row[k] * stride, *jcol = jr + col[k] * stride;
          for (unsigned mm = mkl[row[k]] & mkl[col[k]]; mm; mm &= mm - 1u) {
            const int t = __builtin_ctz(mm);
            delta = fma_(sd[t] * jrow[t], jcol[t], delta);
          }
        } else if (masked) {
          const int *rid = (const int *)jr;
          const float *sdv = jr + count;
          const unsigned *mk4 = (const unsigned *)(jr + 2 * count);
#pragma unroll
          for (int word = 0; word < 4; ++word) {
            if (32 * word >= count) break;  // the same for every lane
            for (unsigned mm = mk4[4 * row[k] + word] & mk4[4 * col[k] + word]; mm; mm &= mm - 1u) {
              const int t = 32 * word + __builtin_ctz(mm);
              const int r = rid[t];
              delta = fma_(sdv[t] * Jw[r * n + row[k]], Jw[r * n + col[k]], delta);
            }
          }
        } else {
          for (int t = 0; t < count; ++t) {
            const int r = idw[t];
            const float a = Jw[r * n + row[k]], b = Jw[r * n + col[k]];
            float da = Dw[r] * a;
            if (sw[r] != quad) da = -da;
            if (a != 0.0f && b != 0.0f) delta = fma_(da, b, delta);
          }
        }
        if (live[k] && delta != 0.0f) {
          if (sl[k] >= 0) N[sl[k]] = N[sl[k]] + delta;  // one pair per slot: no two lanes meet
          else ++nbad;
        }
      }
    }
    for (int o = 32; o > 0; o >>= 1) nbad += __shfl_down(nbad, o, 64);
    if (lane == 0 && nbad) atomicAdd(U + Q.nv_pad * Q.nv_pad - 1, (float)nbad);
    sync_world<true>();
    IM_SSTAMP(1);
    for (int s = lane; s < nfac; s += 64) U[s] = N[s];
    for (int j = lane; j < n; j += 64) N[rhs + j] = gw[ORIGt[j]];
    sync_world<true>();
    IM_SSTAMP(2);
    factor_levels<true>(Q, N, iD, lane, 64);
    IM_SSTAMP(3);
    for (int s = lane; s < nfac; s += 64) U[nfac + s] = N[s];
    for (int j = lane; j < n; j += 64) U[2 * nfac + j] = iD[j];
    IM_SSTAMP(4);
  } else {
    float *gl = (float *)ul;  // [n] right-hand side in elimination order
    for (int s = lane; s < nfac; s += 64) N[s] = U[nfac + s];
    for (int j = lane; j < n; j += 64) {
      iD[j] = U[2 * nfac + j];
      gl[j] = gw[ORIGt[j]];
    }
    sync_world<true>();
    const int32_t *FLt = Q.t[FL], *FRt = Q.t[FR], *RSt = Q.t[RS], *RKPt = Q.t[RKP], *RKt = Q.t[RK];
    for (int l = 0; l < Q.nlevels; ++l) {
      for (int q = FLt[l] + lane; q < FLt[l + 1]; q += 64) {
        const int j = FRt[q];
        float v = gl[j];
        const float *rowp = N + RSt[j];
        const int k0 = RKPt[j], k1 = RKPt[j + 1];
        int t = 0;
        for (; t + 3 < k1 - k0; t += 4) {
          const int ka = RKt[k0 + t], kb = RKt[k0 + t + 1], kc = RKt[k0 + t + 2], kd = RKt[k0 + t + 3];
          const float ra = rowp[t], rb = rowp[t + 1], rc = rowp[t + 2], rd = rowp[t + 3];
          const float ia = iD[ka], ib = iD[kb], ic = iD[kc], id = iD[kd];
          const float xa = N[rhs + ka], xb = N[rhs + kb], xc = N[rhs + kc], xd = N[rhs + kd];
          v = fma_(-(ra * ia), xa, v);
          v = fma_(-(rb * ib), xb, v);
          v = fma_(-(rc * ic), xc, v);
          v = fma_(-(rd * id), xd, v);
        }
        for (; t < k1 - k0; ++t) {
          const int k = RKt[k0 + t];
          v = fma_(-(rowp[t] * iD[k]), N[rhs + k], v);
        }
        N[rhs + j] = v;
      }
      sync_world<true>();
    }
    IM_SSTAMP(5);
  }
  backward_sums<true>(Q, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, 64,
                      A.block);
  IM_SSTAMP(6);
#undef IM_SSTAMP
}

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES, 16 / WAVES) void sparse_update_wave_kernel(
    SparseWave A, const uint8_t *__restrict__ done, const int32_t *__restrict__ state_changes,
    const int32_t *__restrict__ changes, const int32_t *__restrict__ ids, int ld_ids,
    const float *__restrict__ J, int njmax, const float *__restrict__ D,
    const int32_t *__restrict__ state, int quad, const float *__restrict__ grad, int ldg,
    float *__restrict__ U_, int32_t *__restrict__ uni_, float *__restrict__ search_,
    float *__restrict__ search_dot, float *__restrict__ decrement, int nworld) {
  extern __shared__ float lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  SparseDev Q = A.P;
  stage_update_tables<64 * WAVES>(A, Q, lds, tid);
  __syncthreads();  // the only workgroup barrier
  const int w = blockIdx.x * WAVES + wv;
  if (w >= nworld || (done && done[w]) || state_changes[w] == 0) return;
  float *world_lds = lds + A.staged_words + A.solve_words + wv * update_world_words(Q.nslots, Q.nv, A.block, A.staged_rows);
  sparse_update_world(A, Q, world_lds, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, U_, uni_, search_,
                      search_dot, decrement, w, lane);
}

// The resident Newton loop with this stage (newton_wave.h): a wavefront per world from the first
// line search to convergence, WAVES worlds per workgroup sharing one copy of the plan's tables.
// Per wavefront in LDS: the world's row of M and the search direction, and one area that the staged
// tile of J, the gradient's row list and the stage's factor use one after the other.
__host__ __device__ inline int resident_area_words(int nslots, int n, int block, int njmax, int staged_rows) {
  int words = update_world_words(nslots, n, block, staged_rows);
  const int tile = 64 * 17, grad = 2 * njmax + n;
  words = words > tile ? words : tile;
  words = words > grad ? words : grad;
  return (words + 3) & ~3;
}
template <int WAVES, int HELD>
__global__ __launch_bounds__(64 * WAVES, 16 / WAVES) void newton_sparse_resident_kernel(
    SparseWave A, resident::NewtonArgs a, float *__restrict__ U_, int32_t *__restrict__ uni_,
    int *__restrict__ next_world) {
  extern __shared__ float lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  SparseDev Q = A.P;
  stage_update_tables<64 * WAVES>(A, Q, lds, tid);
  const int nv = a.nv, njmax = a.njmax, nworld = a.nworld;
  uint32_t *term = (uint32_t *)(lds + A.staged_words + A.solve_words);
  int *radr = (int *)(term + a.nterm);
  const int area = resident_area_words(Q.nslots, nv, A.block, njmax, A.staged_rows);
  // (M is read from memory by the round's one product with it: its row would cost a CU a third of its worlds)
  float *mine = (float *)(radr + nv + 1) + wv * (area + resident::kept_words(nv, njmax, 0));
  resident::LoopLds L;
  L.votes = nullptr;
  L.term = term, L.radr = radr;
  L.rows = mine;  // the shared area: tile of J, then the gradient's lists, then the stage
  L.f = mine;
  L.rowl = (int *)(mine + njmax);
  L.gl = mine + 2 * njmax;
  L.m_lds = nullptr;
  L.sv = mine + area;
  L.Ma = L.sv + nv;
  L.mv = L.Ma + nv;
  L.qacc = L.mv + nv;
  L.Jaref = L.qacc + nv;
  L.jv = L.Jaref + njmax;
  L.D = L.jv + njmax;
  L.fl = L.D + njmax;
  for (int k = tid; k < a.nterm; k += 64 * WAVES) term[k] = (uint32_t)a.mulm_col[k] | (uint32_t)a.mulm_madr[k] << 16;
  for (int k = tid; k <= nv; k += 64 * WAVES) radr[k] = a.mulm_rowadr[k];
  __syncthreads();  // the only workgroup barrier
  // The grid holds as many wavefronts as the chip keeps resident; a wavefront whose world is done
  // takes the next world nobody has started (a counter in memory, set to the grid's wavefront count
  // before the launch), so the worlds that need many iterations do not hold idle neighbours in
  // place.  The counter only grows: every wavefront reaches the end of the batch.
  int64_t w = (int64_t)blockIdx.x * WAVES + wv;
  // NewtonArgs is the kernel's second parameter, behind the plan's block
  constexpr int kArgsOffset = (int)((sizeof(SparseWave) + alignof(resident::NewtonArgs) - 1) / alignof(resident::NewtonArgs) *
                                    alignof(resident::NewtonArgs));
  auto stage = [&]() __attribute__((always_inline)) {
    const resident::NewtonArgs &b = resident::kernel_args(kArgsOffset);
    sparse_update_world(A, Q, mine, b.quad_count, b.ids, b.ld_ids, b.J, b.njmax, b.D, b.state, b.quad, b.grad,
                        (int)b.ld_grad, U_, uni_, b.search, b.search_dot, b.decrement, (int)w, threadIdx.x & 63);
  };
  while (w < nworld) {
    // HELD: the rows a lane keeps in registers during the line search; the next tile of J is asked for ahead
    resident::newton_loop<HELD, -2, false, false>(kArgsOffset, L, w, stage);
    int next = 0;
    if ((threadIdx.x & 63) == 0) next = atomicAdd(next_world, 1);
    w = __builtin_amdgcn_readfirstlane(next);
  }
}

__global__ void set_counter_kernel(int *counter, int value) { *counter = value; }

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
    forward_rhs_levels(P, N, iD, gw, rhs, ul + n, lane, block);
  }
  backward_sums(P, N, iD, gw, search_ + (size_t)w * n, red, search_dot + w, decrement + w, lane, block, block);
}

// Upstream (non-fused) iteration: the dense Hessian that the upstream assembly and incremental
// update maintain is read through SH_GAT into the factor's slots and factored on the pattern, or,
// for a world whose QUADRATIC rows did not change, the stored factor solves the new gradient.
// hfactor holds [0, nfac) N = L D and [nfac, nfac + n) 1 / D.  Reference: sparse_hessian.py:639-679
// (modes 4 and 5) inside nonfused_kernel (:849-894).
__global__ void sparse_dense_factor_kernel(SparseDev P, const uint8_t *__restrict__ done,
                                           const float *__restrict__ grad, int ldg,
                                           const float *__restrict__ H, int64_t ldH,
                                           const int32_t *__restrict__ quad_changed,
                                           const int32_t *__restrict__ state_changed, int skip_unchanged,
                                           int skip_noflip, float *__restrict__ U_, float *__restrict__ search_,
                                           int ld_search, float *__restrict__ search_dot,
                                           float *__restrict__ decrement) {
  extern __shared__ float lds[];
  const int w = blockIdx.x, lane = threadIdx.x, block = blockDim.x;
  if (done && done[w]) return;
  if (skip_noflip && state_changed[w] == 0) return;
  const bool refactor = !(skip_unchanged && quad_changed[w] == 0);
  const int n = P.nv, nslots = P.nslots, nfac = nslots - n, rhs = nfac;
  const int nw = (block + 31) / 32;
  float *N = lds;          // [nslots]
  float *iD = N + nslots;  // [n]
  float *red = iD + n;     // [2][nw]
  float *U = U_ + (size_t)w * P.nv_pad * P.nv_pad;
  const float *gw = grad + (size_t)w * ldg;
  const int32_t *ORIGt = P.t[ORIG];
  // The solves' tables come into LDS, the forward solve's and then the backward solve's in the same
  // words: a world's share of LDS decides how many worlds a CU holds at once, and with every world
  // of a batch resident a launch lasts as long as one world's chain.
  int *meta = (int *)(red + 2 * nw);
  uint32_t *back = (n <= 256 && nslots <= 65535) ? (uint32_t *)meta : nullptr;
  if (refactor) {
    if (back) stage_backward_tables(P, back, lane, block);  // every use has a barrier before it
    const float *Hw = H + (size_t)w * ldH;
    const uint32_t *GATt = (const uint32_t *)P.t[GAT];
    fill_lds(N, nfac, lane, block, [&](int s) { return Hw[GATt[s]]; });
    fill_lds(N + rhs, n, lane, block, [&](int j) { return gw[ORIGt[j]]; });
    __syncthreads();
    factor_levels(P, N, iD, lane, block);
    for (int s = lane; s < nfac; s += block) U[s] = N[s];
    for (int j = lane; j < n; j += block) U[nfac + j] = iD[j];
  } else {
    fill_lds(N, nfac, lane, block, [&](int s) { return U[s]; });
    fill_lds(iD, n, lane, block, [&](int j) { return U[nfac + j]; });
    forward_rhs_levels(P, N, iD, gw, rhs, meta, lane, block);  // ends with a barrier
    if (back) {
      stage_backward_tables(P, back, lane, block);
      __syncthreads();
    }
  }
  backward_sums(P, N, iD, gw, search_ + (size_t)w * ld_search, red, search_dot + w, decrement + w, lane, block, block, back);
}

}  // namespace
}  // namespace im

extern "C" {

}  // extern "C"

namespace im {

int sparse_plan_upload(im_sparse_plan *pl) {
  pl->device_ready = false;
  // the kernels' workgroup widths; 128 lanes only in the upstream-iteration kernel
  if (pl->block != 32 && pl->block != 64 && !(pl->path == IM_SPARSE_NONFUSED && pl->block == 128)) return IM_ERR_UNSUPPORTED;
  const int nv = pl->nv, nfac = pl->nfac;
  size_t total = 0;
  size_t offs[NHOST];
  for (int i = 0; i < NHOST; ++i) {
    offs[i] = total;
    pl->sizes[i] = (int)pl->table[i].size();
    total += (pl->table[i].size() * 4 + 15) / 16 * 16;
  }
  std::vector<char> host(total, 0);
  for (int i = 0; i < NHOST; ++i) memcpy(host.data() + offs[i], pl->table[i].data(), pl->table[i].size() * 4);
  IM_HIP_CHECK(hipMalloc(&pl->blob, total + 16));  // behind the tables: the resident Newton kernel's world counter
  IM_HIP_CHECK(hipMemcpy(pl->blob, host.data(), total, hipMemcpyHostToDevice));
  pl->next_world = (int *)((char *)pl->blob + total);
  for (int i = 0; i < NHOST; ++i) pl->t[i] = (const int32_t *)((char *)pl->blob + offs[i]);
  if (nv <= 64 && pl->nslots < 65535 && !pl->table[SA].empty()) {
    const int32_t *sa = pl->table[SA].data(), *sb = pl->table[SB].data(), *sm = pl->table[SM].data();
    const int nt = (nv + 15) / 16;
    std::vector<int32_t> tix((size_t)nt * (nt + 1) / 2 * 256, 0);
    int nM = 1;
    bool fits = true;
    for (int sl = 0; sl < nfac; ++sl) {
      const int a = sa[sl], b = sb[sl], e = sm[sl];  // a <= b: tile row b, tile column a
      if (e >= 1024) { fits = false; break; }
      nM = e + 1 > nM ? e + 1 : nM;
      const int ti = b / 16, tj = a / 16, i = b % 16, j = a % 16;
      const int t = ti * (ti + 1) / 2 + tj, lane = j + 16 * (i / 4), v = i % 4;
      tix[((size_t)t * 4 + v) * 64 + lane] = ((e + 1) << 16) | (sl + 1);
    }
    // behind it, the M indices alone, two to a word (v = 0, 1 and v = 2, 3 of a lane): what the
    // kernel holds from its start until the accumulators are set
    const size_t ntile = (size_t)nt * (nt + 1) / 2;
    tix.resize(ntile * 256 + ntile * 128, 0);
    for (size_t t = 0; t < ntile; ++t)
      for (int h = 0; h < 2; ++h)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t lo = (uint32_t)tix[(t * 4 + 2 * h) * 64 + lane] >> 16, hi = (uint32_t)tix[(t * 4 + 2 * h + 1) * 64 + lane] >> 16;
          tix[ntile * 256 + (t * 2 + h) * 64 + lane] = (int32_t)(lo | (hi << 16));
        }
    if (fits) {
      IM_HIP_CHECK(hipMalloc((void **)&pl->tile_index, tix.size() * 4));
      IM_HIP_CHECK(hipMemcpy(pl->tile_index, tix.data(), tix.size() * 4, hipMemcpyHostToDevice));
      pl->nM = nM;
    }
  }
  pl->device_ready = true;
  return IM_OK;
}

}  // namespace im

extern "C" {

void im_sparse_plan_destroy(im_sparse_plan *plan) {
  if (!plan) return;
  if (plan->blob) (void)hipFree(plan->blob);
  if (plan->tile_index) (void)hipFree(plan->tile_index);
  delete plan;
}

int im_sparse_init_factor(const im_sparse_plan *plan, const uint8_t *done, const int32_t *nefc,
                          const float *J, int njmax, const float *D, const int32_t *state, int quad,
                          const float *M, int ldM, const float *grad, int ldg, float *hfactor,
                          float *search, float *search_dot, float *decrement, int nworld, void *stream) {
  if (!plan || nworld < 0 || njmax <= 0) return IM_ERR_ARG;  // rows are clamped to njmax - 1
  if (!plan->device_ready || plan->path != IM_SPARSE_FUSED) return IM_ERR_UNSUPPORTED;
  if (nworld == 0) return IM_OK;
  if (!nefc || !J || !D || !state || !M || !grad || !hfactor || !search || !search_dot || !decrement) return IM_ERR_ARG;
  if (ldg < plan->nv) return IM_ERR_STRIDE;
  im::SparseDev P;
  for (int i = 0; i < im::NHOST; ++i) P.t[i] = plan->t[i];
  P.nv = plan->nv; P.nv_pad = plan->nv_pad; P.nslots = plan->nslots; P.nlevels = plan->nlevels;
  const int n = plan->nv, words = (n + 31) / 32, nw = (plan->block + 31) / 32;
  static const bool simple_only = [] {
    const char *e = std::getenv("IMHIP_SPARSE_KERNEL");
    return e && std::strcmp(e, "simple") == 0;
  }();
  if (plan->tile_index && !simple_only) {
    im::SparseWave A;
    A.P = P;
    for (int i = 0; i < im::kStaged; ++i) A.staged[i] = (int)(plan->t[i] - plan->t[0]);
    const size_t staged = (size_t)(plan->t[im::kStaged] - plan->t[0]);  // tables are padded to 16 bytes
    A.staged_words = (int)staged;
    A.tile_index = plan->tile_index;
    A.staged_rows = 0;  // (the update stage's)
    A.solve_words = 0;
    A.block = plan->block;
    A.nM = plan->nM;
    // per world: the factor's arrays and the list of contributing constraint rows (weight and number)
    const size_t per_world = (((size_t)plan->nslots + n + 2 * nw + 3) & ~(size_t)3) + 2 * (((size_t)njmax + 3) & ~(size_t)3);
    const size_t wave_lds = 4 * (((staged + 3) & ~(size_t)3) + 4 * per_world);
    if (wave_lds <= 64 * 1024 && staged <= 8192 && ldM >= plan->nM) {
      const dim3 grid((unsigned)((nworld + 3) / 4)), wg(256);
      const hipStream_t st = (hipStream_t)stream;
#define IM_SPARSE_WAVE(NT)                                                                            \
  hipLaunchKernelGGL(im::sparse_init_mfma_kernel<NT>, grid, wg, wave_lds, st, A, done, nefc, J, njmax, D, \
                     state, quad, M, ldM, grad, ldg, hfactor, search, search_dot, decrement, nworld)
      switch ((n + 15) / 16) {
        case 1: IM_SPARSE_WAVE(1); break;
        case 2: IM_SPARSE_WAVE(2); break;
        case 3: IM_SPARSE_WAVE(3); break;
        default: IM_SPARSE_WAVE(4); break;
      }
#undef IM_SPARSE_WAVE
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
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
  if (!plan || nworld < 0 || ld_ids < 0 || njmax <= 0) return IM_ERR_ARG;
  if (!plan->device_ready || plan->path != IM_SPARSE_FUSED) return IM_ERR_UNSUPPORTED;
  if (nworld == 0) return IM_OK;
  if (!state_changes || !changes || !ids || !J || !D || !state || !grad || !hfactor || !dof_union || !search ||
      !search_dot || !decrement)
    return IM_ERR_ARG;
  if (ldg < plan->nv) return IM_ERR_STRIDE;
  im::SparseDev P;
  for (int i = 0; i < im::NHOST; ++i) P.t[i] = plan->t[i];
  P.nv = plan->nv; P.nv_pad = plan->nv_pad; P.nslots = plan->nslots; P.nlevels = plan->nlevels;
  const int n = plan->nv, nw = (plan->block + 31) / 32;
  static const bool simple_only = [] {
    const char *e = std::getenv("IMHIP_SPARSE_KERNEL");
    return e && std::strcmp(e, "simple") == 0;
  }();
  if (n <= 64 && !simple_only) {
    im::SparseWave A;
    A.P = P;
    for (int i = 0; i < im::kStaged; ++i) A.staged[i] = (int)(plan->t[i] - plan->t[0]);
    const size_t staged = (size_t)(plan->t[im::kStaged] - plan->t[0]);
    A.staged_words = (int)staged;
    A.tile_index = nullptr;
    A.block = plan->block;
    A.nM = 0;
    const int32_t *solve_end = plan->t[im::RK] + ((plan->sizes[im::RK] + 3) & ~3);
    const size_t solve_words = (size_t)(solve_end - plan->t[im::FL]);
    // 32 staged rows where a CU still holds sixteen worlds with them, else 16
    A.staged_rows =
        4 * (staged + solve_words + 16 * (size_t)im::update_world_words(plan->nslots, n, plan->block, 32)) <= 160 * 1024 ? 32 : 16;
    const size_t per_world = (size_t)im::update_world_words(plan->nslots, n, plan->block, A.staged_rows);
    for (int i = 0; i < 5; ++i) A.solve[i] = (int)(plan->t[im::FL + i] - plan->t[im::FL]);
    A.solve_words = (int)solve_words;
    const size_t wave_lds = 4 * (staged + solve_words + 4 * per_world);
    if (wave_lds <= 64 * 1024 && staged <= 8192 && solve_words <= 4096) {
      // Worlds per workgroup: every workgroup stages the tables for itself, so larger workgroups
      // leave more of a CU's 160 KB to the worlds.  The count that keeps the most worlds on a CU
      // (at most 32 wavefronts of 57 registers) is taken, the smallest on a tie and where four
      // per workgroup already hold the whole batch.
      constexpr size_t kCuLds = 160 * 1024;
      int waves = 4;
      int64_t best = 0;
      for (int cand = 4; cand <= 16; cand *= 2) {
        const size_t bytes = 4 * (staged + solve_words + (size_t)cand * per_world);
        int64_t held = (int64_t)(kCuLds / bytes) * cand;
        held = held < 32 ? held : 32;
        if (held > best && (cand == 4 || (int64_t)nworld > best * 256)) best = held, waves = cand;
      }
      const size_t lds_bytes = 4 * (staged + solve_words + (size_t)waves * per_world);
      const dim3 grid((unsigned)((nworld + waves - 1) / waves)), wg(64 * waves);
#define IM_UPDATE_WAVE(W)                                                                                     \
  do {                                                                                                        \
    if (lds_bytes > 64 * 1024)                                                                                \
      IM_HIP_CHECK(hipFuncSetAttribute((const void *)im::sparse_update_wave_kernel<W>,                        \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));          \
    hipLaunchKernelGGL(im::sparse_update_wave_kernel<W>, grid, wg, lds_bytes, (hipStream_t)stream, A, done,   \
                       state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, hfactor,     \
                       dof_union, search, search_dot, decrement, nworld);                                     \
  } while (0)
      if (waves == 16) IM_UPDATE_WAVE(16);
      else if (waves == 8) IM_UPDATE_WAVE(8);
      else IM_UPDATE_WAVE(4);
#undef IM_UPDATE_WAVE
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
  const size_t lds_bytes = 4 * ((size_t)plan->nslots + n + 2 * nw + n + 4 * n + 2 + ((size_t)plan->nfac + 1) / 2);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::sparse_update_kernel, dim3(nworld), dim3(plan->block), lds_bytes, (hipStream_t)stream, P,
                     done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, hfactor,
                     dof_union, search, search_dot, decrement);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_newton_solve_sparse(const im_sparse_plan *plan, const im_newton_args *p, float *hfactor, int32_t *dof_union,
                           void *stream) {
  if (!plan || !p || !hfactor || !dof_union || p->nworld < 0) return IM_ERR_ARG;
  if (!plan->device_ready || plan->path != IM_SPARSE_FUSED || plan->nv > 64) return IM_ERR_UNSUPPORTED;
  if (p->nworld == 0) return IM_OK;
  const int n = plan->nv, njmax = p->njmax;
  const int nM = plan->nM;
  if (nM <= 0) return IM_ERR_UNSUPPORTED;
  im::resident::NewtonArgs a{};
  const int bad = im::resident::convert_args(*p, n, nM, a);
  if (bad != IM_OK) return bad;
  if (p->block != plan->block) return IM_ERR_ARG;
  im::SparseWave A;
  for (int i = 0; i < im::NHOST; ++i) A.P.t[i] = plan->t[i];
  A.P.nv = plan->nv; A.P.nv_pad = plan->nv_pad; A.P.nslots = plan->nslots; A.P.nlevels = plan->nlevels;
  for (int i = 0; i < im::kStaged; ++i) A.staged[i] = (int)(plan->t[i] - plan->t[0]);
  const size_t staged = (size_t)(plan->t[im::kStaged] - plan->t[0]);
  A.staged_words = (int)staged;
  A.tile_index = nullptr;
  A.block = plan->block;
  A.nM = 0;
  const int32_t *solve_end = plan->t[im::RK] + ((plan->sizes[im::RK] + 3) & ~3);
  const size_t solve_words = (size_t)(solve_end - plan->t[im::FL]);
  for (int i = 0; i < 5; ++i) A.solve[i] = (int)(plan->t[im::FL + i] - plan->t[im::FL]);
  A.solve_words = (int)solve_words;
  if (staged > 8192 || solve_words > 4096) return IM_ERR_UNSUPPORTED;
  const size_t shared = staged + solve_words + (size_t)p->nterm + n + 1;
  auto wave_words = [&](int staged_rows) {
    return (size_t)im::resident_area_words(plan->nslots, n, plan->block, njmax, staged_rows) + im::resident::kept_words(n, njmax, 0);
  };
  // the most worlds per workgroup (one workgroup per CU) that 160 KB of LDS admit and whose kernel
  // keeps to registers
  struct Variant {
    int waves, held;
    const void *fn;
  };
  // the line search keeps a lane's two rows in registers up to 64 rows and reads them from LDS beyond
  // (four rows a lane up to 128 rows was measured slower here: 997 against 930 us per loop at g1)
  static const Variant variants[] = {{16, 2, (const void *)im::newton_sparse_resident_kernel<16, 2>},
                                     {12, 2, (const void *)im::newton_sparse_resident_kernel<12, 2>},
                                     {8, 2, (const void *)im::newton_sparse_resident_kernel<8, 2>},
                                     {4, 2, (const void *)im::newton_sparse_resident_kernel<4, 2>},
                                     {16, 0, (const void *)im::newton_sparse_resident_kernel<16, 0>},
                                     {12, 0, (const void *)im::newton_sparse_resident_kernel<12, 0>},
                                     {8, 0, (const void *)im::newton_sparse_resident_kernel<8, 0>},
                                     {4, 0, (const void *)im::newton_sparse_resident_kernel<4, 0>}};
  constexpr int kVariants = 8;
  static bool usable[kVariants] = {};
  static bool probed = false;
  if (!probed) {  // once per process: register spills and the grant of the large dynamic LDS
    for (int i = 0; i < kVariants; ++i) {
      hipFuncAttributes fa{};
      // (a variant that parks more than a few values of its prologue in memory is left out)
      usable[i] = hipFuncGetAttributes(&fa, variants[i].fn) == hipSuccess && fa.localSizeBytes <= 16 &&
                  hipFuncSetAttribute(variants[i].fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      160 * 1024 - (int)fa.sharedSizeBytes) == hipSuccess;
      (void)hipGetLastError();
    }
    probed = true;
  }
  for (int i = 0; i < kVariants; ++i) {
    if (!usable[i] || variants[i].held != (njmax <= 64 ? 2 : 0)) continue;
    // 32 staged rows where the workgroup still fits with them (they cost a CU no world then), else 16
    // (snu: 32 rows with eight worlds per CU instead of twelve was measured slower, 1344 against 1283 us per loop)
    A.staged_rows = 4 * (shared + (size_t)variants[i].waves * wave_words(32)) <= 158 * 1024 ? 32 : 16;
    const size_t lds = 4 * (shared + (size_t)variants[i].waves * wave_words(A.staged_rows));
    if (lds > 158 * 1024) continue;
    const int waves = variants[i].waves;
    // as many workgroups as stay resident at once (LDS, and sixteen wavefronts of up to 128 registers
    // per CU); the others' worlds are taken up by the wavefronts that finish
    static int ncu = 0;
    if (!ncu) {
      int dev = 0;
      IM_HIP_CHECK(hipGetDevice(&dev));
      IM_HIP_CHECK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
    }
    const int per_cu = std::max(1, std::min((int)(160 * 1024 / lds), 16 / waves));
    const int needed = (p->nworld + waves - 1) / waves;
    const int grid = std::min(needed, std::max(ncu, 1) * per_cu);
    int *counter = plan->next_world;
    hipLaunchKernelGGL(im::set_counter_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, counter, grid * waves);
    void *args[] = {&A, &a, &hfactor, &dof_union, &counter};
    IM_HIP_CHECK(hipLaunchKernel(variants[i].fn, dim3((unsigned)grid), dim3(64 * waves), args, lds, (hipStream_t)stream));
    return IM_OK;
  }
  return IM_ERR_UNSUPPORTED;
}

int im_sparse_dense_factor(const im_sparse_plan *plan, const uint8_t *done, const float *grad, int ldg,
                           const float *H, int64_t ldH, const int32_t *quad_changed,
                           const int32_t *state_changed, int skip_unchanged, int skip_noflip, float *hfactor,
                           float *search, int ld_search, float *search_dot, float *decrement, int nworld,
                           void *stream) {
  if (!plan || nworld < 0) return IM_ERR_ARG;
  if (!plan->device_ready || plan->sizes[im::GAT] == 0) return IM_ERR_UNSUPPORTED;  // a plan of the fused path
  if (nworld == 0) return IM_OK;
  if (!grad || !H || !hfactor || !search || !search_dot || !decrement) return IM_ERR_ARG;
  if ((skip_unchanged && !quad_changed) || (skip_noflip && !state_changed)) return IM_ERR_ARG;
  if (ldg < plan->nv || ld_search < plan->nv || ldH < (int64_t)plan->nv_pad * plan->nv_pad) return IM_ERR_STRIDE;
  im::SparseDev P;
  for (int i = 0; i < im::NHOST; ++i) P.t[i] = plan->t[i];
  P.nv = plan->nv; P.nv_pad = plan->nv_pad; P.nslots = plan->nslots; P.nlevels = plan->nlevels;
  const int nw = (plan->block + 31) / 32;
  // the forward solve's tables, or the backward solve's (its pushes <= nfac) in the same words
  const size_t fwd_words = 4 * (size_t)plan->nv + 2 + ((size_t)plan->nfac + 1) / 2, bwd_words = (size_t)plan->nlevels + 1 + plan->nfac;
  const size_t lds_bytes = 4 * ((size_t)plan->nslots + plan->nv + 2 * nw + (fwd_words > bwd_words ? fwd_words : bwd_words));
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(im::sparse_dense_factor_kernel, dim3(nworld), dim3(plan->block), lds_bytes, (hipStream_t)stream,
                     P, done, grad, ldg, H, ldH, quad_changed, state_changed, skip_unchanged, skip_noflip, hfactor,
                     search, ld_search, search_dot, decrement);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
