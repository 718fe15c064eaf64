// Cholesky of a matrix that fits one tile (up to 64 x 64) with the solve of one right-hand side,
// nothing kept: the reference's two "no L store" tile kernels
// (src/instantmimic/utils/mjw_step_optimized.py:672-750) and the nv <= 32 branch of the Newton
// factor stage (src/instantmimic/utils/mjw_kernels/newton_stages.py:723-733), with a launch for the first
// factor of a solve in which the world's wavefront assembles H ahead of it (dense_init_tile_kernel).
//
// A group of 32 or 64 lanes owns a tile; lane i holds row i of the lower triangle in registers and
// its right-hand side entry.  Column j, once final, goes through LDS to every lane of the group
// (one store, then 16-byte reads of the same words by all lanes), which scale it by the pivot's
// reciprocal themselves and update their columns to the right (right-looking: every element sees
// the fused multiply-adds of  v = A[i][j]; for q < j: v = fma(-L[i][q], L[j][q], v)  in that
// order).  The forward substitution rides along; the factor is then laid down in LDS row by row and
// the backward substitution reads row r of it across the lanes.  No workgroup barrier anywhere.
// The arithmetic inside the reference's tile operations is Warp's (third party); this is the
// convention of the blocked factor's diagonal tiles, as the CPU restatement it is tested against.
#include <hip/hip_runtime.h>

#include <cstdint>

#include <algorithm>

#include "common.h"
#include "jtdj_wave.h"
#include "newton_wave.h"
#include "pivot.h"

namespace im {
namespace {

using resident::wave_sync;

// LDS words of one group: the column being handed round, the right-hand side entries, the pivots'
// reciprocals, and the tile itself (staged in, later the factor), rows NP + 1 words apart
template <int NP>
struct TileArea {
  static constexpr int kRow = NP + 1;
  static constexpr int kWords = 3 * NP + NP * kRow + 4;  // a multiple of four words: the column is read 16 bytes at a time
  float *col, *rhs, *rinv, *tile;
  __device__ explicit TileArea(float *base) : col(base), rhs(base + NP), rinv(base + 2 * NP), tile(base + 3 * NP) {}
};

// value of lane `src` of the caller's group of LG lanes
template <int LG>
__device__ __forceinline__ float group_bcast(float v, int src) {
  return __shfl(v, src, LG);
}

// a[c], c <= i: row i of the lower triangle (lanes at or past n and columns at or past n: zero);
// s: the right-hand side entry.  Returns the solution entry of lane i (lanes at or past n: 0).
template <int NP, int LG>
__device__ __forceinline__ float tile_factor_solve(float (&a)[NP], float s, int i, int n, const TileArea<NP> &T) {
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    if (j < n) {  // the same for every lane of the launch
      if (i < NP) {  // a group has more lanes than the tile has rows
        T.col[i] = a[j];
        T.rhs[i] = s;
      }
      wave_sync();
      // the column from its pivot on, 16 bytes per read, the same words for every lane
      float cv[NP];
#pragma unroll
      for (int q = j / 4; q < NP / 4; ++q) {
        const float4 v = ((const float4 *)T.col)[q];
        cv[4 * q] = v.x, cv[4 * q + 1] = v.y, cv[4 * q + 2] = v.z, cv[4 * q + 3] = v.w;
      }
      float d, rinv;
      pivot_sqrt_rcp(cv[j], true, d, rinv);
      const float lj = a[j] * rinv;  // rows below the diagonal; what the others compute is not read
      const float z = T.rhs[j] * rinv;
#pragma unroll
      for (int c = j + 1; c < NP; ++c) a[c] = fma_(-lj, cv[c] * rinv, a[c]);
      s = i > j ? fma_(-lj, z, s) : (i == j ? z : s);
      a[j] = i == j ? d : lj;
      if (i == j) T.rinv[j] = rinv;
      wave_sync();  // the column's words are read before the next column is written over them
    }
  }
  // the factor, row by row; the backward substitution then reads row r across the lanes:
  // x[r] = s[r] / L[r][r], s[t] = fma(-L[r][t], x[r], s[t]) for t < r, r descending
#pragma unroll
  for (int c = 0; c < NP; ++c)
    if (c <= i && i < NP) T.tile[i * TileArea<NP>::kRow + c] = a[c];
  wave_sync();
  float l_next = n > 0 ? T.tile[(n - 1) * TileArea<NP>::kRow + (i < NP ? i : 0)] : 0.0f;
  for (int r = n - 1; r >= 0; --r) {
    const float l_r = l_next;
    if (r > 0) l_next = T.tile[(r - 1) * TileArea<NP>::kRow + (i < NP ? i : 0)];
    const float xr = group_bcast<LG>(s, r) * T.rinv[r];
    s = i < r ? fma_(-l_r, xr, s) : (i == r ? xr : s);
  }
  return s;
}

// The same factor and solve by a whole wavefront on one tile of up to 32 rows: lane i of either half
// holds row i, the lower half its even columns and the upper half the odd ones (a2[k] = element
// (i, 2 k + half)), so a column's update of the columns to its right is shared between the two.
// Every element sees the same operations in the same order as above; s and the backward
// substitution run in both halves alike.
template <int NP>
__device__ __forceinline__ float tile_factor_solve_halves(float (&a2)[NP / 2], float s, int i, int half, int n,
                                                          const TileArea<NP> &T) {
  static_assert(NP % 2 == 0 && NP <= 32, "two columns a step, a row a lane of a half");
  const int ic = i < NP ? i : 0;
  const float *colh = T.col + half;
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    if (j < n) {  // the same for every lane of the launch
      const int kj = j >> 1, hj = j & 1;
      if (half == hj && i < NP) {
        T.col[i] = a2[kj];
        T.rhs[i] = s;
      }
      wave_sync();
      const float aj = i < NP ? T.col[ic] : 0.0f, pv = T.col[j];  // (a half has more lanes than a small tile has rows)
      float cv[NP / 2];
#pragma unroll
      for (int k = (j + 1) >> 1; k < NP / 2; ++k) cv[k] = colh[2 * k];  // column 2 k + half
      float d, rinv;
      pivot_sqrt_rcp(pv, true, d, rinv);
      const float lj = aj * rinv;  // rows below the diagonal; what the others compute is not read
      const float z = T.rhs[j] * rinv;
#pragma unroll
      for (int k = (j + 1) >> 1; k < NP / 2; ++k) {
        const float v = fma_(-lj, cv[k] * rinv, a2[k]);
        a2[k] = (2 * k > j || half == 1) ? v : a2[k];  // column 2 k + half lies right of column j
      }
      s = i > j ? fma_(-lj, z, s) : (i == j ? z : s);
      a2[kj] = half == hj ? (i == j ? d : lj) : a2[kj];
      if (i == j && half == hj) T.rinv[j] = rinv;
      wave_sync();  // the column's words are read before the next column is written over them
    }
  }
#pragma unroll
  for (int k = 0; k < NP / 2; ++k)
    if (2 * k + half <= i && i < NP) T.tile[i * TileArea<NP>::kRow + 2 * k + half] = a2[k];
  wave_sync();
  float l_next = n > 0 ? T.tile[(n - 1) * TileArea<NP>::kRow + ic] : 0.0f;
  for (int r = n - 1; r >= 0; --r) {
    const float l_r = l_next;
    if (r > 0) l_next = T.tile[(r - 1) * TileArea<NP>::kRow + ic];
    const float xr = group_bcast<32>(s, r) * T.rinv[r];
    s = i < r ? fma_(-l_r, xr, s) : (i == r ? xr : s);
  }
  return s;
}

// One tile per group of LG lanes, 256 / LG tiles per workgroup.  elemid == nullptr: M is dense
// with ld_world floats per world and ld_row per row, tile t the diagonal block at adr[t] (lower
// triangle read); else M holds nM values per world and tile t's element (r, c) is
// M[elemid[(t size + r) size + c]] (upper triangle read).
template <int NP, int LG>
__global__ __launch_bounds__(256) void tile_cholesky_solve_kernel(
    const float *__restrict__ M, int64_t ld_world, int64_t ld_row, const int32_t *__restrict__ adr, int ntile,
    int size, const int32_t *__restrict__ elemid, int nM, const float *__restrict__ y, int64_t ldy,
    float *__restrict__ x, int64_t ldx, int64_t ntotal) {
  extern __shared__ float lds[];
  constexpr int kRow = TileArea<NP>::kRow;
  const int group = threadIdx.x / LG, i = threadIdx.x % LG;
  const int64_t item = (int64_t)blockIdx.x * (256 / LG) + group;
  if (item >= ntotal) return;  // whole groups; nothing below waits for another group
  const int64_t w = item / ntile;
  const int t = (int)(item - w * ntile);
  const TileArea<NP> T(lds + group * TileArea<NP>::kWords);
  const float *Mw = M + w * ld_world;
  const int a0 = adr[t];
  // the tile comes in with consecutive lanes on consecutive words of its rows
  const int area = size * size;
  for (int e0 = i; e0 < area; e0 += 4 * LG) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int e = e0 + k * LG < area ? e0 + k * LG : area - 1;
      const int r = e / size, c = e - r * size;
      if (elemid) {
        const int id = elemid[(size_t)t * area + e];
        v[k] = id < nM ? Mw[id < nM ? id : 0] : 0.0f;
      } else {
        v[k] = Mw[(int64_t)(a0 + r) * ld_row + a0 + c];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int e = e0 + k * LG;
      if (e < area) {
        const int r = e / size;
        T.tile[r * kRow + e - r * size] = v[k];
      }
    }
  }
  float s = i < size ? y[w * ldy + a0 + i] : 0.0f;
  wave_sync();
  float a[NP];
#pragma unroll
  for (int c = 0; c < NP; ++c) {
    const bool mine = i < size && c <= i;
    // lower read: element (i, c); upper read: element (c, i)
    a[c] = mine ? T.tile[elemid ? c * kRow + i : i * kRow + c] : 0.0f;
  }
  wave_sync();
  s = tile_factor_solve<NP, LG>(a, s, i, size, T);
  if (i < size) x[w * ldx + a0 + i] = s;
}

// The Newton factor stage up to 32 dofs: dofs touched by the changed rows, incremental update of
// H's upper triangle (in memory and in the staged copy), then H factored as one tile and solved
// for the gradient, at every call; U is not used.  search = -x, search_dot = x.x,
// decrement = grad.x.  A wavefront per world: the rows on 32 lanes, the two halves sharing the work.
constexpr int kTileStagedRows = 16;
// LDS words of one group's stage: the tile's area, the dof union (36), the staged rows, their weights and the dofs' masks
template <int NP>
__host__ __device__ constexpr int dense_tile_stage_words() {
  return TileArea<NP>::kWords + 36 + (kTileStagedRows + 1) * NP + kTileStagedRows + NP;
}

// One world's stage on a group of 32 lanes (lane i of the group).  WHOLE: both groups of the
// wavefront work on this world: they share H's load, the pairs of the update and the columns of
// the factor between them and write the same values to the same places otherwise.
template <int NP, bool WHOLE = false>
__device__ __forceinline__ void dense_tile_world(const TileArea<NP> &T, int *ul, float *Hw, const float *Jw, const float *Dw,
                                                 const float *gw, const int32_t *sw, const int32_t *idw, int count, int quad,
                                                 int32_t *uni, float *search_w, float *search_dot_w, float *decrement_w,
                                                 int nv, int pad, int i) {
  constexpr int LG = 32, kRow = TileArea<NP>::kRow;
  // H's rows into LDS (both triangles as they lie there; only the upper one is read)
  const float inv_nv = 1.0f / (float)nv;
  constexpr int LW = WHOLE ? 64 : LG;                       // lanes that share a loop over the world's elements
  const int iw = WHOLE ? (int)(threadIdx.x & 63) : i;       // this lane among them
  const int half = WHOLE ? (int)((threadIdx.x >> 5) & 1) : 0;
  for (int e0 = iw; e0 < nv * nv; e0 += 4 * LW) {  // four loads in flight per lane
    float v[4];
    int at[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int e = e0 + k * LW < nv * nv ? e0 + k * LW : nv * nv - 1;
      const int r = (int)(((float)e + 0.5f) * inv_nv), c = e - r * nv;  // e / nv, exact for these sizes
      v[k] = Hw[(size_t)r * pad + c];
      at[k] = r * kRow + c;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (e0 + k * LW < nv * nv) T.tile[at[k]] = v[k];
  }
  // The changed rows of J come into LDS dof-major (a dof's elements of up to kTileStagedRows rows
  // side by side, 17 words a dof) with a mask per dof of the rows that are nonzero there; more
  // changed rows than that are read from memory pair by pair.
  const bool staged = count <= kTileStagedRows;
  const bool masked = !staged && count <= 128 && 2 * count + 4 * nv <= (kTileStagedRows + 1) * NP;
  float *jr = (float *)(ul + 36);             // [nv][kTileStagedRows + 1]
  float *sd = jr + (kTileStagedRows + 1) * NP;  // [kTileStagedRows] D of the row, negated for a row that left the quadratic state
  unsigned *mkl = (unsigned *)(sd + kTileStagedRows);  // [nv]
  int hit = 0;
  if (staged && count > 0) {
    const int tq = i < count ? i : count - 1;
    const int rq = idw[tq];
    const float dq = Dw[rq];
    const int sq = sw[rq];
    float rowv[kTileStagedRows];
#pragma unroll
    for (int t = 0; t < kTileStagedRows; ++t) {
      const int r = __shfl(rq, t < count ? t : 0, LG);
      rowv[t] = Jw[(size_t)r * nv + (i < nv ? i : nv - 1)];
    }
    if (i < kTileStagedRows) sd[i] = sq == quad ? dq : -dq;
    if (i < nv) {
      unsigned mk = 0u;
#pragma unroll
      for (int t = 0; t < kTileStagedRows; ++t) {
        if (t < count) {
          jr[i * (kTileStagedRows + 1) + t] = rowv[t];
          mk |= (unsigned)(rowv[t] != 0.0f) << t;
        }
      }
      mkl[i] = mk;
      hit = mk != 0u;
    }
  } else if (masked) {
    // more rows than the staged capacity: their numbers, their weights and a mask of up to 128 rows per
    // dof go where the staged rows would lie; J's elements then come from memory, but only those of
    // the rows that a pair's two dofs share
    int *rid = (int *)jr;                          // [count]
    float *sdv = jr + count;                       // [count]
    unsigned *mk4 = (unsigned *)(jr + 2 * count);  // [nv][4]
    for (int t = i; t < count; t += LG) {
      const int r = idw[t];
      rid[t] = r;
      sdv[t] = sw[r] == quad ? Dw[r] : -Dw[r];
    }
    unsigned any = 0u;
#pragma unroll
    for (int word = 0; word < 4; ++word) {
      unsigned mw = 0u;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int t0 = 32 * word + 16 * half;
        if (t0 < count) {  // (a group's count: the two groups of a wavefront may differ)
          float rowv[16];
#pragma unroll
          for (int t = 0; t < 16; ++t)
            rowv[t] = Jw[(size_t)idw[t0 + t < count ? t0 + t : count - 1] * nv + (i < nv ? i : nv - 1)];
#pragma unroll
          for (int t = 0; t < 16; ++t)
            if (t0 + t < count) mw |= (unsigned)(rowv[t] != 0.0f) << (16 * half + t);
        }
      }
      if (i < nv) mk4[4 * i + word] = mw;
      any |= mw;
    }
    hit = i < nv && any != 0u;
  } else if (i < nv) {
    for (int t = 0; t < count && !hit; ++t) hit = Jw[(size_t)idw[t] * nv + i] != 0.0f;
  }
  // dof union, ascending: lane d looks at dof d
  const unsigned long long both = __ballot(hit);
  const unsigned mask = (unsigned)(both >> (threadIdx.x & 32));
  const int nu = __popc(mask);
  if (hit) {
    const int at = __popc(mask & ((1u << i) - 1u));
    ul[at] = i;
    uni[at] = i;
  }
  if (i == 0) uni[nv] = nu;
  wave_sync();
  for (int e = iw; e < nu * (nu + 1) / 2; e += LW) {
    int cj = (int)((sqrtf((float)(8 * e + 1)) - 1.0f) * 0.5f);
    while ((cj + 1) * (cj + 2) / 2 <= e) ++cj;
    while (cj * (cj + 1) / 2 > e) --cj;
    const int row = ul[e - cj * (cj + 1) / 2], col = ul[cj];
    float delta = 0.0f;
    if (staged) {  // the rows in which both dofs are nonzero, ascending
      const float *jrow = jr + row * (kTileStagedRows + 1), *jcol = jr + col * (kTileStagedRows + 1);
      for (unsigned mm = mkl[row] & mkl[col]; mm; mm &= mm - 1u) {
        const int t = __builtin_ctz(mm);
        delta = fma_(sd[t] * jrow[t], jcol[t], delta);
      }
    } else if (masked) {
      const int *rid = (const int *)jr;
      const float *sdv = jr + count;
      const unsigned *mk4 = (const unsigned *)(jr + 2 * count);
#pragma unroll
      for (int word = 0; word < 4; ++word) {
        if (32 * word < count) {
          for (unsigned mm = mk4[4 * row + word] & mk4[4 * col + word]; mm; mm &= mm - 1u) {
            const int t = 32 * word + __builtin_ctz(mm);
            const int r = rid[t];
            delta = fma_(sdv[t] * Jw[(size_t)r * nv + row], Jw[(size_t)r * nv + col], delta);
          }
        }
      }
    } else {
      for (int t = 0; t < count; ++t) {
        const int r = idw[t];
        const float av = Jw[(size_t)r * nv + row], bv = Jw[(size_t)r * nv + col];
        float da = Dw[r] * av;
        if (sw[r] != quad) da = -da;
        if (av != 0.0f && bv != 0.0f) delta = fma_(da, bv, delta);
      }
    }
    if (delta != 0.0f) {
      const float h = T.tile[row * kRow + col] + delta;
      T.tile[row * kRow + col] = h;
      Hw[(size_t)row * pad + col] = h;
    }
  }
  float s = i < nv ? gw[i] : 0.0f;
  const float g = s;
  wave_sync();
  if constexpr (WHOLE) {
    float a2[NP / 2];
#pragma unroll
    for (int k = 0; k < NP / 2; ++k) a2[k] = (i < nv && 2 * k + half <= i) ? T.tile[(2 * k + half) * kRow + i] : 0.0f;
    wave_sync();
    s = tile_factor_solve_halves<NP>(a2, s, i, half, nv, T);
  } else {
    float a[NP];
#pragma unroll
    for (int c = 0; c < NP; ++c) a[c] = (i < nv && c <= i) ? T.tile[c * kRow + i] : 0.0f;  // upper triangle: element (c, i)
    wave_sync();
    s = tile_factor_solve<NP, LG>(a, s, i, nv, T);
  }
  if (i < nv) search_w[i] = -s;
  // as 64 lanes striding the dofs would sum them: one term per lane, the upper 32 lanes' zeros change nothing
  float s0 = fma_(s, s, 0.0f), s1 = fma_(g, s, 0.0f);
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    s0 = s0 + __shfl_down(s0, off, LG);
    s1 = s1 + __shfl_down(s1, off, LG);
  }
  if (i == 0) {
    *search_dot_w = s0;
    *decrement_w = s1;
  }
}

template <int NP>
__global__ __launch_bounds__(256) void dense_update_tile_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ state_changes,
    const int32_t *__restrict__ changes, const int32_t *__restrict__ ids, int ld_ids,
    const float *__restrict__ J, int njmax, const float *__restrict__ D, const int32_t *__restrict__ state,
    int quad, const float *__restrict__ grad, int64_t ldg, float *H_, int32_t *__restrict__ uni_,
    float *__restrict__ search, int64_t ld_search, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int pad, int nworld) {
  extern __shared__ float lds[];
  // a wavefront per world, its two halves sharing the work
  const int group = threadIdx.x >> 6, i = threadIdx.x & 31;
  const int64_t w = (int64_t)blockIdx.x * 4 + group;
  if (w >= nworld) return;
  if ((done && done[w]) || state_changes[w] == 0) return;
  const TileArea<NP> T(lds + group * dense_tile_stage_words<NP>());
  int *ul = (int *)(lds + group * dense_tile_stage_words<NP>() + TileArea<NP>::kWords);  // [nv + 1], the staged rows behind it
  int count = changes[w];
  count = count < 0 ? 0 : (count < ld_ids ? count : ld_ids);
  dense_tile_world<NP, true>(T, ul, H_ + w * (int64_t)pad * pad, J + w * (int64_t)njmax * nv, D + w * njmax, grad + w * ldg,
                       state + w * njmax, ids + w * ld_ids, count, quad, uni_ + w * (nv + 1), search + w * ld_search,
                       search_dot + w, decrement + w, nv, pad, i);
}

// The first Hessian and its factor in one launch, a wavefront per world: H = M + J' D_act J on the
// wavefront's matrix cores (jtdj_wave.h), stored, then the stage above without changed rows for the
// worlds that are not done (both halves of the wavefront run it on the same world).
template <int NP>
__global__ __launch_bounds__(256) void dense_init_tile_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ nefc_p, const float *__restrict__ J, int njmax,
    const float *__restrict__ D, const int32_t *__restrict__ state, int quad, const float *__restrict__ M, int64_t ldM,
    const int32_t *__restrict__ elemid, const float *__restrict__ grad, int64_t ldg, float *H_,
    int32_t *__restrict__ uni_, float *__restrict__ search, int64_t ld_search, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int pad, int nworld) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t w = (int64_t)blockIdx.x * 4 + wv;
  if (w >= nworld) return;
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  float *Hw = H_ + w * (int64_t)pad * pad;
  const float *Jw = J + w * (int64_t)njmax * nv;
  jtdj_wave<(NP + 15) / 16>(M + w * ldM, elemid, Jw, D + w * njmax, state + w * njmax, nefc, quad, nv, Hw, pad,
                            (pad & 3) == 0, lane);
  if (done && done[w]) return;
  // the lanes read back one another's stores (one CU: its vector cache sees them once they are issued and waited for)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  float *mine = lds + wv * dense_tile_stage_words<NP>();
  const TileArea<NP> T(mine);
  dense_tile_world<NP, true>(T, (int *)(mine + TileArea<NP>::kWords), Hw, Jw, D + w * njmax, grad + w * ldg, state + w * njmax,
                       nullptr, 0, quad, uni_ + w * (nv + 1), search + w * ld_search, search_dot + w, decrement + w, nv, pad,
                       lane & 31);
}

// The resident Newton loop (newton_wave.h) with this stage: a wavefront per world from the first
// line search to convergence, WAVES worlds per workgroup.  Both halves of the wavefront run the
// stage on the wavefront's world.  Per wavefront in LDS: what the loop keeps from round to round
// and one area that the staged tile of J, the gradient's row list and the stage's tile use one
// after the other.
template <int NP>
__host__ __device__ inline int dense_resident_area_words(int nv, int njmax) {
  int words = dense_tile_stage_words<NP>();
  const int tile = 64 * 17, grad = 2 * njmax + nv;
  words = words > tile ? words : tile;
  words = words > grad ? words : grad;
  return (words + 3) & ~3;
}
__host__ __device__ inline int dense_resident_shared_words(int nterm, int nv) { return (nterm + nv + 1 + 3) & ~3; }

template <int NP, int WAVES, int HELD>
__global__ __launch_bounds__(64 * WAVES, 16 / WAVES) void newton_dense_tile_resident_kernel(
    resident::NewtonArgs a, float *__restrict__ H_, int32_t *__restrict__ uni_, int pad, int *__restrict__ next_world) {
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nv = a.nv, njmax = a.njmax, nworld = a.nworld;
  uint32_t *term = (uint32_t *)lds;
  int *radr = (int *)(term + a.nterm);
  const int area = dense_resident_area_words<NP>(nv, njmax);
  float *mine = lds + dense_resident_shared_words(a.nterm, nv) + wv * (area + resident::kept_words(nv, njmax, 0));
  resident::LoopLds L;
  L.votes = nullptr;
  L.worlds = nullptr;
  L.term = term, L.radr = radr;
  L.rows = mine;  // the shared area: tile of J, then the gradient's lists, then the stage's tile
  L.f = mine;
  L.rowl = (int *)(mine + njmax);
  L.gl = mine + 2 * njmax;
  L.m_lds = nullptr;  // M is read from memory by the round's one product with it
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
  int64_t w = (int64_t)blockIdx.x * WAVES + wv;
  auto stage = [&]() __attribute__((always_inline)) {
    const resident::NewtonArgs &b = resident::kernel_args(0);  // the kernel's first parameter
    int lane = threadIdx.x & 31;
    asm volatile("" : "+v"(lane));  // (nothing formed from it is kept in registers from round to round)
    const TileArea<NP> T(mine);
    int count = b.quad_count[w];
    count = count < 0 ? 0 : (count < b.ld_ids ? count : b.ld_ids);
    dense_tile_world<NP, true>(T, (int *)(mine + TileArea<NP>::kWords), H_ + w * (int64_t)pad * pad,
                         b.J + w * (int64_t)b.njmax * b.nv, b.D + w * b.njmax, b.grad + w * b.ld_grad,
                         b.state + w * b.njmax, b.ids + w * (int64_t)b.ld_ids, count, b.quad, uni_ + w * (b.nv + 1),
                         b.search + w * b.nv, b.search_dot + w, b.decrement + w, b.nv, pad, lane);
  };
  // as many wavefronts as the chip keeps resident; one whose world is done takes the next world
  // nobody has started (a counter in memory that only grows: every wavefront reaches the end)
  while (w < nworld) {
    resident::newton_loop<HELD, -2, false, false>(0, L, w, stage);
    int next = 0;
    if ((threadIdx.x & 63) == 0) next = atomicAdd(next_world, 1);
    w = __builtin_amdgcn_readfirstlane(next);
  }
}

__global__ void set_dense_counter_kernel(int *counter, int value) { *counter = value; }

template <int NP, int LG>
int launch_tiles(const float *M, int64_t ld_world, int64_t ld_row, const int32_t *adr, int ntile, int size,
                 const int32_t *elemid, int nM, const float *y, int64_t ldy, float *x, int64_t ldx, int nworld,
                 hipStream_t stream) {
  const int64_t ntotal = (int64_t)nworld * ntile;
  constexpr int per = 256 / LG;
  const size_t lds = sizeof(float) * per * TileArea<NP>::kWords;
  auto fn = tile_cholesky_solve_kernel<NP, LG>;
  if (lds > 64 * 1024) IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(fn, dim3((unsigned)((ntotal + per - 1) / per)), dim3(256), lds, stream, M, ld_world, ld_row, adr, ntile,
                     size, elemid, nM, y, ldy, x, ldx, ntotal);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int dispatch_tiles(const float *M, int64_t ld_world, int64_t ld_row, const int32_t *adr, int ntile, int size,
                   const int32_t *elemid, int nM, const float *y, int64_t ldy, float *x, int64_t ldx, int nworld,
                   void *stream) {
  hipStream_t st = (hipStream_t)stream;
#define IM_TILE_CASE(NP, LG) \
  if (size <= NP) return launch_tiles<NP, LG>(M, ld_world, ld_row, adr, ntile, size, elemid, nM, y, ldy, x, ldx, nworld, st);
  IM_TILE_CASE(8, 32) IM_TILE_CASE(16, 32) IM_TILE_CASE(24, 32) IM_TILE_CASE(32, 32)
  IM_TILE_CASE(40, 64) IM_TILE_CASE(48, 64) IM_TILE_CASE(56, 64) IM_TILE_CASE(64, 64)
#undef IM_TILE_CASE
  return IM_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace im

extern "C" {

int im_tile_cholesky_solve(const float *M, int64_t ld_world, int64_t ld_row, const int32_t *tile_adr, int ntile,
                           int tile_size, const float *y, int64_t ldy, float *x, int64_t ldx, int nworld, void *stream) {
  if (nworld < 0 || ntile < 0 || tile_size <= 0) return IM_ERR_ARG;
  if (nworld == 0 || ntile == 0) return IM_OK;
  if (!M || !tile_adr || !y || !x) return IM_ERR_ARG;
  if (ld_row < tile_size || ld_world < ld_row * tile_size || ldy < tile_size || ldx < tile_size) return IM_ERR_STRIDE;
  if (tile_size > 64) return IM_ERR_UNSUPPORTED;
  return im::dispatch_tiles(M, ld_world, ld_row, tile_adr, ntile, tile_size, nullptr, 0, y, ldy, x, ldx, nworld, stream);
}

int im_tile_cholesky_solve_m(const float *M, int64_t ldM, int nM, const int32_t *block_elemid, const int32_t *block_dof,
                             int nblock, int tile_size, const float *y, int64_t ldy, float *x, int64_t ldx, int nworld,
                             void *stream) {
  if (nworld < 0 || nblock < 0 || tile_size <= 0 || nM <= 0) return IM_ERR_ARG;
  if (nworld == 0 || nblock == 0) return IM_OK;
  if (!M || !block_elemid || !block_dof || !y || !x) return IM_ERR_ARG;
  if (ldM < nM || ldy < tile_size || ldx < tile_size) return IM_ERR_STRIDE;
  if (tile_size > 64) return IM_ERR_UNSUPPORTED;
  return im::dispatch_tiles(M, ldM, 0, block_dof, nblock, tile_size, block_elemid, nM, y, ldy, x, ldx, nworld, stream);
}

// the Newton factor stage up to 32 dofs; im_dense_update_factor hands such shapes here
int im_dense_update_tile(const uint8_t *done, const int32_t *state_changes, const int32_t *changes, const int32_t *ids,
                         int ld_ids, const float *J, int njmax, const float *D, const int32_t *state, int quad,
                         const float *grad, int64_t ldg, float *H, int nv, int nv_pad, int32_t *dof_union, float *search,
                         int64_t ld_search, float *search_dot, float *decrement, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv > 32 || nv_pad < nv || ld_ids < 0 || njmax <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!state_changes || !changes || !ids || !J || !D || !state || !grad || !H || !dof_union || !search || !search_dot ||
      !decrement)
    return IM_ERR_ARG;
  if (ldg < nv || ld_search < nv) return IM_ERR_STRIDE;
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)((nworld + 3) / 4);
#define IM_STAGE_CASE(NP)                                                                                            \
  if (nv <= NP) {                                                                                                    \
    const size_t lds = sizeof(float) * 4 * im::dense_tile_stage_words<NP>();                                         \
    hipLaunchKernelGGL(im::dense_update_tile_kernel<NP>, dim3(grid), dim3(256), lds, st, done, state_changes, changes, \
                       ids, ld_ids, J, njmax, D, state, quad, grad, ldg, H, dof_union, search, ld_search, search_dot, \
                       decrement, nv, nv_pad, nworld);                                                               \
    IM_HIP_CHECK(hipGetLastError());                                                                                 \
    return IM_OK;                                                                                                    \
  }
  IM_STAGE_CASE(8) IM_STAGE_CASE(16) IM_STAGE_CASE(24) IM_STAGE_CASE(32)
#undef IM_STAGE_CASE
  return IM_ERR_UNSUPPORTED;
}

// the first Hessian and factor of a dense solve up to 32 dofs; im_dense_init_factor hands such shapes here
int im_dense_init_tile(const uint8_t *done, const int32_t *nefc, const float *J, int njmax, const float *D,
                       const int32_t *state, int quad, const float *M, int64_t ldM, const int32_t *elemid, const float *grad,
                       int64_t ldg, float *H, int nv, int nv_pad, int32_t *dof_union, float *search, int64_t ld_search,
                       float *search_dot, float *decrement, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv > 32 || nv_pad < nv || njmax <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!J || !D || !state || !M || !elemid || !grad || !H || !dof_union || !search || !search_dot || !decrement)
    return IM_ERR_ARG;
  if (ldg < nv || ld_search < nv || ((uintptr_t)H & 15) != 0) return IM_ERR_STRIDE;
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)((nworld + 3) / 4);
#define IM_INIT_CASE(NP)                                                                                              \
  if (nv <= NP) {                                                                                                     \
    const size_t lds = sizeof(float) * 4 * im::dense_tile_stage_words<NP>();                                          \
    hipLaunchKernelGGL(im::dense_init_tile_kernel<NP>, dim3(grid), dim3(256), lds, st, done, nefc, J, njmax, D, state, \
                       quad, M, ldM, elemid, grad, ldg, H, dof_union, search, ld_search, search_dot, decrement, nv,   \
                       nv_pad, nworld);                                                                               \
    IM_HIP_CHECK(hipGetLastError());                                                                                  \
    return IM_OK;                                                                                                     \
  }
  IM_INIT_CASE(8) IM_INIT_CASE(16) IM_INIT_CASE(24) IM_INIT_CASE(32)
#undef IM_INIT_CASE
  return IM_ERR_UNSUPPORTED;
}

int im_newton_solve_dense_tile(const im_newton_args *p, float *H, int32_t *dof_union, int nv, int nv_pad, int nM,
                               int32_t *next_world, void *stream) {
  if (!p || !H || !dof_union || !next_world || p->nworld < 0 || nv <= 0 || nv_pad < nv || nM <= 0) return IM_ERR_ARG;
  if (nv > 32) return IM_ERR_UNSUPPORTED;
  if (p->nworld == 0) return IM_OK;
  im::resident::NewtonArgs a{};
  const int bad = im::resident::convert_args(*p, nv, nM, a);
  if (bad != IM_OK) return bad;
  const int njmax = p->njmax;
  struct Variant {
    int np, waves, held;
    const void *fn;
  };
#define IM_DENSE_VARIANT(NP, WAVES, HELD) {NP, WAVES, HELD, (const void *)im::newton_dense_tile_resident_kernel<NP, WAVES, HELD>}
  // tile of 16 or 32 dofs; sixteen or eight worlds per workgroup; the line search keeps a lane's two
  // rows in registers up to 64 rows and reads them from LDS beyond
  static const Variant variants[] = {IM_DENSE_VARIANT(16, 16, 2), IM_DENSE_VARIANT(16, 8, 2), IM_DENSE_VARIANT(16, 16, 0),
                                     IM_DENSE_VARIANT(16, 8, 0),  IM_DENSE_VARIANT(32, 16, 2), IM_DENSE_VARIANT(32, 8, 2),
                                     IM_DENSE_VARIANT(32, 16, 0), IM_DENSE_VARIANT(32, 8, 0)};
#undef IM_DENSE_VARIANT
  constexpr int kVariants = 8;
  static bool usable[kVariants] = {};
  static bool probed = false;
  if (!probed) {  // once per process: a variant that spills registers is left out; the large dynamic LDS is asked for
    for (int i = 0; i < kVariants; ++i) {
      hipFuncAttributes fa{};
      // (a variant that parks more than a register or two in memory is left out)
      usable[i] = hipFuncGetAttributes(&fa, variants[i].fn) == hipSuccess && fa.localSizeBytes <= 16 &&
                  hipFuncSetAttribute(variants[i].fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      160 * 1024 - (int)fa.sharedSizeBytes) == hipSuccess;
      (void)hipGetLastError();
    }
    probed = true;
  }
  const int np = nv <= 16 ? 16 : 32;
  for (int i = 0; i < kVariants; ++i) {
    const Variant &v = variants[i];
    if (!usable[i] || v.np != np || v.held != (njmax <= 64 ? 2 : 0)) continue;
    const int area = np == 16 ? im::dense_resident_area_words<16>(nv, njmax) : im::dense_resident_area_words<32>(nv, njmax);
    const size_t per_wave = (size_t)area + im::resident::kept_words(nv, njmax, 0);
    const size_t lds = 4 * ((size_t)im::dense_resident_shared_words(p->nterm, nv) + v.waves * per_wave);
    if (lds > 158 * 1024) continue;
    static int ncu = 0;
    if (!ncu) {
      int dev = 0;
      IM_HIP_CHECK(hipGetDevice(&dev));
      IM_HIP_CHECK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
    }
    // as many workgroups as stay resident at once (LDS, and sixteen wavefronts of up to 128 registers per CU)
    const int per_cu = std::max(1, std::min((int)(160 * 1024 / lds), 16 / v.waves));
    const int needed = (p->nworld + v.waves - 1) / v.waves;
    const int grid = std::min(needed, std::max(ncu, 1) * per_cu);
    hipLaunchKernelGGL(im::set_dense_counter_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, next_world, grid * v.waves);
    void *args[] = {&a, &H, &dof_union, &nv_pad, &next_world};
    IM_HIP_CHECK(hipLaunchKernel(v.fn, dim3((unsigned)grid), dim3(64 * v.waves), args, lds, (hipStream_t)stream));
    return IM_OK;
  }
  return IM_ERR_UNSUPPORTED;
}

}  // extern "C"
