// Cholesky of a matrix that fits one tile (up to 64 x 64) with the solve of one right-hand side,
// nothing kept: the reference's two "no L store" tile kernels
// (src/instantmimic/utils/mjw_step_optimized.py:672-750) and the nv <= 32 branch of the Newton
// factor stage (src/instantmimic/utils/mjw_kernels/newton_stages.py:723-733).
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

#include "common.h"
#include "pivot.h"

namespace im {
namespace {

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

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
// decrement = grad.x.  Two worlds per wavefront, 32 lanes each.
template <int NP>
__global__ __launch_bounds__(256) void dense_update_tile_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ state_changes,
    const int32_t *__restrict__ changes, const int32_t *__restrict__ ids, int ld_ids,
    const float *__restrict__ J, int njmax, const float *__restrict__ D, const int32_t *__restrict__ state,
    int quad, const float *__restrict__ grad, int64_t ldg, float *H_, int32_t *__restrict__ uni_,
    float *__restrict__ search, int64_t ld_search, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int pad, int nworld) {
  extern __shared__ float lds[];
  constexpr int LG = 32, kRow = TileArea<NP>::kRow;
  const int group = threadIdx.x / LG, i = threadIdx.x % LG;
  const int64_t w = (int64_t)blockIdx.x * (256 / LG) + group;
  if (w >= nworld) return;
  if ((done && done[w]) || state_changes[w] == 0) return;
  const TileArea<NP> T(lds + group * (TileArea<NP>::kWords + 36));
  int *ul = (int *)(lds + group * (TileArea<NP>::kWords + 36) + TileArea<NP>::kWords);  // [nv + 1]
  float *Hw = H_ + w * (int64_t)pad * pad;
  const float *Jw = J + w * (int64_t)njmax * nv, *Dw = D + w * njmax, *gw = grad + w * ldg;
  const int32_t *sw = state + w * njmax, *idw = ids + w * ld_ids;
  int count = changes[w];
  count = count < 0 ? 0 : (count < ld_ids ? count : ld_ids);
  // H's rows into LDS (both triangles as they lie there; only the upper one is read)
  for (int e = i; e < nv * nv; e += LG) {
    const int r = e / nv, c = e - r * nv;
    T.tile[r * kRow + c] = Hw[(size_t)r * pad + c];
  }
  // dof union, ascending: lane d looks at dof d
  int hit = 0;
  if (i < nv)
    for (int t = 0; t < count && !hit; ++t) hit = Jw[(size_t)idw[t] * nv + i] != 0.0f;
  const unsigned long long both = __ballot(hit);
  const unsigned mask = (unsigned)(both >> (threadIdx.x & 32));
  const int nu = __popc(mask);
  if (hit) {
    const int at = __popc(mask & ((1u << i) - 1u));
    ul[at] = i;
    uni_[w * (nv + 1) + at] = i;
  }
  if (i == 0) uni_[w * (nv + 1) + nv] = nu;
  wave_sync();
  for (int e = i; e < nu * (nu + 1) / 2; e += LG) {
    int cj = (int)((sqrtf((float)(8 * e + 1)) - 1.0f) * 0.5f);
    while ((cj + 1) * (cj + 2) / 2 <= e) ++cj;
    while (cj * (cj + 1) / 2 > e) --cj;
    const int row = ul[e - cj * (cj + 1) / 2], col = ul[cj];
    float delta = 0.0f;
    for (int t = 0; t < count; ++t) {
      const int r = idw[t];
      const float av = Jw[(size_t)r * nv + row], bv = Jw[(size_t)r * nv + col];
      float da = Dw[r] * av;
      if (sw[r] != quad) da = -da;
      if (av != 0.0f && bv != 0.0f) delta = fma_(da, bv, delta);
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
  float a[NP];
#pragma unroll
  for (int c = 0; c < NP; ++c) a[c] = (i < nv && c <= i) ? T.tile[c * kRow + i] : 0.0f;  // upper triangle: element (c, i)
  wave_sync();
  s = tile_factor_solve<NP, LG>(a, s, i, nv, T);
  if (i < nv) search[w * ld_search + i] = -s;
  // as 64 lanes striding the dofs would sum them: one term per lane, the upper 32 lanes' zeros change nothing
  float s0 = fma_(s, s, 0.0f), s1 = fma_(g, s, 0.0f);
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    s0 = s0 + __shfl_down(s0, off, LG);
    s1 = s1 + __shfl_down(s1, off, LG);
  }
  if (i == 0) {
    search_dot[w] = s0;
    decrement[w] = s1;
  }
}

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
  const unsigned grid = (unsigned)((nworld + 7) / 8);
#define IM_STAGE_CASE(NP)                                                                                            \
  if (nv <= NP) {                                                                                                    \
    const size_t lds = sizeof(float) * 8 * (im::TileArea<NP>::kWords + 36);                                          \
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

}  // extern "C"
