// Blocked dense upper Cholesky factor + solve with indexed gather of M, one workgroup
// per world, the factor resident in LDS (the reference stores and reloads every U block
// through global memory), plus the dense J'DJ Hessian on fp32 MFMA for large nv.
//
// Reference schedule: src/instantmimic/utils/mjw_kernels/indexed_factor.py:15-173
// (left-looking by block column, forward solve fused into the factor loop, backward
// solve), scratch layout src/instantmimic/utils/mjw_step_optimized.py:893-955.  The
// arithmetic inside a tile operation is Warp's tile library in the reference; here it is
// spelled out and fixed (same convention as the CPU restatement it is tested against):
//   U_jk' U_ji updates: sum over t ascending with fma from 0, then C = C - sum;
//   Cholesky by columns, s = fma(-l, l, s), L[i][j] = v * (1 / L[j][j]);
//   triangular solves column oriented (j ascending forward, r descending backward), a pivot
//   is applied as a multiplication by 1 / diagonal (the reciprocal is an exact division).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <mutex>
#include <cstring>

#include "common.h"
#include "jtdj_wave.h"
#include "pivot.h"

namespace im {
namespace {

// value of lane n (0..15) of the caller's row of 16 lanes, in every lane of that row
template <int N>
__device__ __forceinline__ float row_bcast_c(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x150 + N, 0xF, 0xF, true));
}
// n becomes a constant once the caller's loop is unrolled; the DPP control must be one
__device__ __forceinline__ float row_bcast(float v, int n) {
  switch (n) {
#define IM_BCAST_CASE(N) case N: return row_bcast_c<N>(v);
    IM_BCAST_CASE(0) IM_BCAST_CASE(1) IM_BCAST_CASE(2) IM_BCAST_CASE(3) IM_BCAST_CASE(4) IM_BCAST_CASE(5)
    IM_BCAST_CASE(6) IM_BCAST_CASE(7) IM_BCAST_CASE(8) IM_BCAST_CASE(9) IM_BCAST_CASE(10) IM_BCAST_CASE(11)
    IM_BCAST_CASE(12) IM_BCAST_CASE(13) IM_BCAST_CASE(14)
#undef IM_BCAST_CASE
    default: return row_bcast_c<15>(v);
  }
}

// a[jj] = fma(-lj, lj of lane jj, a[jj]) for the columns jj right of pivot column j, as v_fmac_f32 with the
// broadcast on its first operand and the sign on its second (one instruction per column; the compiler forms a move and a
// fused multiply-add).  A DPP operand must not be read within two cycles of the vector instruction
// that wrote it, and the compiler does not look inside these blocks: each waits on entry (lj was
// just computed) and on exit (the next pivot is read from a[j + 1] through DPP).  The first column
// has a block of its own so that the rest can be scheduled into the pivot's square root.
#define IM_TR(jj) "v_fmac_f32_dpp %[a" #jj "], %[lj], -%[lj] row_newbcast:" #jj " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
#define IM_TO(jj) [a##jj] "+v"(a[jj])
__device__ __forceinline__ void trailing_update16(float (&a)[16], float lj, int j) {
  switch (j) {
    case 0:
      asm("s_nop 1\n\t" IM_TR(1) "s_nop 1" : IM_TO(1) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(2) IM_TR(3) IM_TR(4) IM_TR(5) IM_TR(6) IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) "s_nop 1" : IM_TO(2), IM_TO(3), IM_TO(4), IM_TO(5), IM_TO(6), IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 1:
      asm("s_nop 1\n\t" IM_TR(2) "s_nop 1" : IM_TO(2) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(3) IM_TR(4) IM_TR(5) IM_TR(6) IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) "s_nop 1" : IM_TO(3), IM_TO(4), IM_TO(5), IM_TO(6), IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 2:
      asm("s_nop 1\n\t" IM_TR(3) "s_nop 1" : IM_TO(3) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(4) IM_TR(5) IM_TR(6) IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) "s_nop 1" : IM_TO(4), IM_TO(5), IM_TO(6), IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 3:
      asm("s_nop 1\n\t" IM_TR(4) "s_nop 1" : IM_TO(4) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(5) IM_TR(6) IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) "s_nop 1" : IM_TO(5), IM_TO(6), IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(15) "s_nop 1" : IM_TO(15) : [lj] "v"(lj));
      break;
    case 4:
      asm("s_nop 1\n\t" IM_TR(5) "s_nop 1" : IM_TO(5) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(6) IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(6), IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 5:
      asm("s_nop 1\n\t" IM_TR(6) "s_nop 1" : IM_TO(6) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(7) IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(7), IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 6:
      asm("s_nop 1\n\t" IM_TR(7) "s_nop 1" : IM_TO(7) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(8) IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(8), IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 7:
      asm("s_nop 1\n\t" IM_TR(8) "s_nop 1" : IM_TO(8) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(9) IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(9), IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 8:
      asm("s_nop 1\n\t" IM_TR(9) "s_nop 1" : IM_TO(9) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(10) IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(10), IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 9:
      asm("s_nop 1\n\t" IM_TR(10) "s_nop 1" : IM_TO(10) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(11) IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(11), IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 10:
      asm("s_nop 1\n\t" IM_TR(11) "s_nop 1" : IM_TO(11) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(12) IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(12), IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 11:
      asm("s_nop 1\n\t" IM_TR(12) "s_nop 1" : IM_TO(12) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(13) IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(13), IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 12:
      asm("s_nop 1\n\t" IM_TR(13) "s_nop 1" : IM_TO(13) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(14) IM_TR(15) "s_nop 1" : IM_TO(14), IM_TO(15) : [lj] "v"(lj));
      break;
    case 13:
      asm("s_nop 1\n\t" IM_TR(14) "s_nop 1" : IM_TO(14) : [lj] "v"(lj));
      asm("s_nop 1\n\t" IM_TR(15) "s_nop 1" : IM_TO(15) : [lj] "v"(lj));
      break;
    case 14:
      asm("s_nop 1\n\t" IM_TR(15) "s_nop 1" : IM_TO(15) : [lj] "v"(lj));
      break;
    default: break;
  }
}
#undef IM_TR
#undef IM_TO

// Cholesky of a B x B diagonal tile with the forward solve of the right-hand side riding along:
// lane i of a row of DPP lanes holds row i of the tile in a[] and the row's right-hand side in s.
// Column j's updates are applied to the columns to its right as soon as it is final
// (right-looking), which gives every element the same fused multiply-adds in the same order
// (q ascending) as the column-wise form  v = A[i][j]; for q < j: v = fma(-L[i][q], L[j][q], v)
// while the next pivot waits for one of them only.  Nothing is stored inside the loop: column j of
// the factor replaces a[j], lane j keeps the solved right-hand side entry and the pivot's
// reciprocal.  FAST: the short forms of the square root and the reciprocal; lo / hi receive the
// smallest and largest bit pattern among the pivots, for the caller to check against the range
// the short forms are exact in (the check is off the chain from one pivot to the next that way).
template <int B, bool FAST>
__device__ __forceinline__ void diag_tile(float (&a)[B], float &s, int i, float &my_z, float &my_rinv, uint32_t &lo,
                                          uint32_t &hi) {
#pragma unroll
  for (int j = 0; j < B; ++j) {
    const float x = row_bcast(a[j], j);
    float d, rinv;
    if constexpr (FAST) {
      const uint32_t bits = __builtin_bit_cast(uint32_t, x);
      lo = bits < lo ? bits : lo;
      hi = bits > hi ? bits : hi;
      pivot_sqrt_rcp_fast(x, d, rinv);
    } else {
      d = sqrtf(x);
      rinv = 1.0f / d;
    }
    // rows below the diagonal; the pivot's own lane gets d further down, and what it and the lanes
    // above it compute in the meantime is never read
    const float lj = a[j] * rinv;
    const float z = row_bcast(s, j) * rinv;
    my_z = i == j ? z : my_z;
    my_rinv = i == j ? rinv : my_rinv;
    s = fma_(-lj, z, s);  // meaningful for i > j
    if constexpr (FAST && B == 16) {
      trailing_update16(a, lj, j);
    } else {
#pragma unroll
      for (int jj = j + 1; jj < B; ++jj) a[jj] = fma_(-lj, row_bcast(lj, jj), a[jj]);
    }
    a[j] = i == j ? d : lj;
  }
}
constexpr uint32_t kPivotBitsLo = 0x0F800000u;  // 2^-96
constexpr uint32_t kPivotBitsHi = 0x7F800000u;  // +inf: negative numbers and NaNs lie above as unsigned patterns

// The factor's LDS array: U is upper triangular, so the rows of block row t keep the columns from
// t * B on and follow one another (a staircase by tiles: 46 KB at pad 144 where the square takes
// 83 KB, which is what lets two workgroups share a CU there).  Diagonal tiles are held in full.
template <int B>
struct Stair {
  int pad;
  // words in front of block row t
  __device__ __host__ __forceinline__ int band(int t) const { return B * t * pad - (B * B / 2) * t * (t - 1); }
  // row r of block row t, column col >= t * B
  __device__ __forceinline__ int in_band(int t, int r, int col) const { return band(t) + r * (pad - t * B) + col - t * B; }
  __device__ __forceinline__ int at(int row, int col) const { return in_band(row / B, row % B, col); }
  __device__ __host__ __forceinline__ int words() const { return band(pad / B); }
};

// Where a tile element comes from.
// Dense: the upper triangle of a row-major (pad, pad) matrix (the lower one is never read);
// rows and columns >= nv are the identity whatever the buffer holds there.
template <int B>
struct DenseSrc {
  const float *H;
  int nv, pad;
  __device__ __forceinline__ float load(int kb, int ib, int, int r, int c) const {
    const int row = kb * B + r, col = ib * B + c;
    // only the upper triangle is kept up to date: mirror it inside a diagonal tile
    if (row < nv && col < nv) return row <= col ? H[(size_t)row * pad + col] : H[(size_t)col * pad + row];
    return row == col ? 1.0f : 0.0f;
  }
};

// In place: the matrix already sits in the LDS array the factor is written to (upper triangle
// valid, everything else zero); block row kb is read before the factor overwrites it.
template <int B>
struct LdsSrc {
  const float *U;
  int nv, pad;
  __device__ __forceinline__ float load(int kb, int ib, int, int r, int c) const {
    const Stair<B> S{pad};
    // a tile right of the diagonal and inside the dofs (the same test for a whole tile) is read as it lies
    if (ib != kb && (ib + 1) * B <= nv) return U[S.in_band(kb, r, ib * B + c)];
    const int row = kb * B + r, col = ib * B + c;
    if (row < nv && col < nv) return row <= col ? U[S.at(row, col)] : U[S.at(col, row)];
    return row == col ? 1.0f : 0.0f;
  }
};

// The tiles were gathered into the LDS array of the factor beforehand, diagonal tiles in full.
template <int B>
struct GatheredSrc {
  const float *U;
  int pad;
  __device__ __forceinline__ float load(int kb, int ib, int, int r, int c) const {
    return U[Stair<B>{pad}.in_band(kb, r, ib * B + c)];
  }
};

// Indexed gather of every tile on or above the diagonal into U: ids >= nM
// read as zero, padded diagonal entries get +1 (mjw_step_optimized.py:932-941).  A wavefront
// takes every (number of wavefronts)-th tile and keeps eight or nine tiles' loads in flight.
// Every word of the staircase belongs to one of these tiles, so U needs no clearing first.
template <int B>
__device__ __forceinline__ void gather_tiles(const float *__restrict__ Mw, const int32_t *__restrict__ block_idx,
                                             int nM, int nv, int pad, float *U, int tid, int nt) {
  constexpr int BB = B * B, PER = BB / 64 > 0 ? BB / 64 : 1, G = B == 16 ? 9 : 8;  // 36 tiles at pad 128: one round for four wavefronts
  const int nblk = pad / B, lane = tid & 63, nwv = nt >> 6;
  int kb = 0, ib = 0;  // cursor over the upper tiles, row by row
  auto advance = [&](int n) {
    for (int s_ = 0; s_ < n && kb < nblk; ++s_)
      if (++ib == nblk) { ++kb; ib = kb; }
  };
  advance(tid >> 6);
  while (kb < nblk) {
    int tk[G], ti[G], idx[G][PER];
    float v[G][PER];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      tk[g] = kb < nblk ? kb : -1;
      ti[g] = ib;
      advance(nwv);
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int e = u * 64 + lane;
        const bool use = tk[g] >= 0 && e < BB;
        idx[g][u] = block_idx[use ? (size_t)(tk[g] * nblk + ti[g]) * BB + e : 0];
        if (!use) idx[g][u] = nM;
      }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int u = 0; u < PER; ++u) v[g][u] = Mw[idx[g][u] < nM ? idx[g][u] : 0];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int e = u * 64 + lane;
        if (tk[g] >= 0 && e < BB) {
          const int r = e / B, c = e - r * B;
          float x = idx[g][u] < nM ? v[g][u] : 0.0f;
          if (ti[g] == tk[g] && (tk[g] + 1) * B > nv && r == c && (nblk - 1) * B + r >= nv) x = x + 1.0f;
          U[Stair<B>{pad}.in_band(tk[g], r, ti[g] * B + c)] = x;
        }
      }
  }
}

// Left-looking upper Cholesky by block column with the forward solve of rhs fused into the
// loop; U (the staircase of pad) and rhs (pad) in LDS.
template <int B, class Src>
__device__ __forceinline__ void factor_forward(const Src &src, float *U, float *rhs, float *L, int pad, int tid,
                                               int nt) {
  const int nblk = pad / B;
  constexpr int BB = B * B;
  const Stair<B> S{pad};
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  // v -= the sums over the finished block rows jb0 .. jb1 - 1 for the 16 x 16 tile at columns i0 of
  // the block row at columns k0, in the block rows' order.  One wavefront, the sums on the matrix
  // cores: v_mfma_f32_16x16x4_f32 adds its four products to the accumulator one after the other,
  // each with a fused multiply-add, so four of them chained from zero are the sum over
  // t = 0..15 ascending of the scalar form.  Two block rows at a time: their sums are
  // independent chains on the matrix cores (four at a time measured the same).
  auto schur = [&](f32x4 &v, int k0, int i0, int jb0, int jb1) {
    const int lane = tid & 63, p = lane & 15, kq = lane >> 4;
    int jb = jb0;
    for (; jb + 1 < jb1; jb += 2) {
      f32x4 sum0 = {0.0f, 0.0f, 0.0f, 0.0f}, sum1 = sum0;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const int at0 = S.in_band(jb, 4 * s4 + kq, p), at1 = S.in_band(jb + 1, 4 * s4 + kq, p);
        const float a0 = U[at0 + k0], b0 = U[at0 + i0], a1 = U[at1 + k0], b1 = U[at1 + i0];
        sum0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, sum0, 0, 0, 0);
        sum1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1, sum1, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (v[i] - sum0[i]) - sum1[i];
    }
    if (jb < jb1) {
      f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const int at = S.in_band(jb, 4 * s4 + kq, p);
        const float a = U[at + k0], b = U[at + i0];
        sum = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, sum, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = v[i] - sum[i];
    }
  };
  // look-ahead: while wavefront 0 factors a diagonal tile, the others prepare the next block row
  const bool ahead = B == 16 && nt > 64;
  for (int kb = 0; kb < nblk; ++kb) {
    const int k = kb * B;
    // the whole block row kb..nblk-1 minus the finished block rows above, in place: a tile's
    // elements are read (from U itself or from the source) before the same wavefront or thread
    // writes them, and the block rows above are final
    const int ntile = nblk - kb;
    if constexpr (B == 16) {
      // One wavefront per 16 x 16 tile.
      // With more than one wavefront, the sums over the block rows above the last finished one were
      // subtracted while that one's diagonal tile was factored (below), and what is left here is
      // the last block row's sum.
      const int lane = tid & 63, p = lane & 15, kq = lane >> 4;
      for (int tb = tid >> 6; tb < ntile; tb += nt >> 6) {
        const int ib = kb + tb, i0 = ib * B;
        f32x4 v;
        if (ahead && kb > 0) {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = U[S.in_band(kb, 4 * kq + i, i0 + p)];
          schur(v, k, i0, kb - 1, kb);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = src.load(kb, ib, (4 * kq + i) * B + p, 4 * kq + i, p);
          schur(v, k, i0, 0, kb);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) U[S.in_band(kb, 4 * kq + i, i0 + p)] = v[i];
      }
    } else {
      for (int q = tid; q < ntile * BB; q += nt) {
        const int tb = q / BB, e = q - tb * BB, r = e / B, c = e - r * B;
        const int ib = kb + tb, i0 = ib * B;
        float v = src.load(kb, ib, e, r, c);
        for (int jb = 0; jb < kb; ++jb) {
          const int j = jb * B;
          float sum = 0.0f;
#pragma unroll
          for (int t = 0; t < B; ++t) sum = fma_(U[S.in_band(jb, t, k + r)], U[S.in_band(jb, t, i0 + c)], sum);
          v = v - sum;
        }
        U[S.in_band(kb, r, i0 + c)] = v;
      }
    }
    // the right-hand side: every row below the block row that was finished last subtracts that
    // block row's sum (a chain of B terms from zero); a row has seen the block rows above it in
    // ascending order when its own turn comes
    if (kb > 0)
      for (int r = k + tid; r < pad; r += nt) {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(U[S.in_band(kb - 1, t, r)], rhs[k - B + t], sum);
        rhs[r] = rhs[r] - sum;
      }
    __syncthreads();
    // Cholesky of the diagonal tile and the forward solve of the right-hand side: the first B
    // lanes of wave 0, lane i holding row i in registers; values of other rows come through DPP
    // row broadcasts.  The short forms first; a pivot outside their range (not seen with a positive
    // definite matrix of ordinary scale) repeats the tile with the library forms.
    if (tid < 64) {
      const int i = tid;
      float a[B];
#pragma unroll
      for (int j = 0; j < B; ++j) a[j] = U[S.in_band(kb, i < B ? i : 0, k + j)];
      float s = rhs[k + (i < B ? i : 0)];
      float my_z = 0.0f, my_rinv = 0.0f;
      uint32_t lo = kPivotBitsLo, hi = kPivotBitsLo;
      diag_tile<B, true>(a, s, i, my_z, my_rinv, lo, hi);
      if (__builtin_expect(__any(i < B && (lo < kPivotBitsLo || hi >= kPivotBitsHi)), 0)) {
#pragma unroll
        for (int j = 0; j < B; ++j) a[j] = U[S.in_band(kb, i < B ? i : 0, k + j)];
        s = rhs[k + (i < B ? i : 0)];
        diag_tile<B, false>(a, s, i, my_z, my_rinv, lo, hi);
      }
      if (i < B) {
#pragma unroll
        for (int j = 0; j < B; ++j) L[j * B + i] = a[j];  // column j of the factor in a row of L; entries above the diagonal are never read
        rhs[k + i] = my_z;
        L[B * B + i] = my_rinv;  // reciprocals of the pivots, behind the tile
      }
    } else if (ahead && kb + 1 < nblk) {
      // Meanwhile the other wavefronts prepare the next block row: its tiles minus the sums over
      // the block rows above this one, which are final.  This block row's own sum follows when it
      // is finished, so every element still sees its subtractions in ascending order.
      const int lane = tid & 63, p = lane & 15, kq = lane >> 4;
      for (int tb = (tid >> 6) - 1; tb < ntile - 1; tb += (nt >> 6) - 1) {
        const int ib = kb + 1 + tb, i0 = ib * B;
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = src.load(kb + 1, ib, (4 * kq + i) * B + p, 4 * kq + i, p);
        schur(v, k + B, i0, 0, kb);
#pragma unroll
        for (int i = 0; i < 4; ++i) U[S.in_band(kb + 1, 4 * kq + i, i0 + p)] = v[i];
      }
    }
    __syncthreads();
    // U_kk = L', and U_ki = L^-1 A_ki column by column
    for (int e = tid; e < BB; e += nt) {
      const int r = e / B, c = e - r * B;
      U[S.in_band(kb, r, k + c)] = c >= r ? L[r * B + c] : 0.0f;  // a gathered tile may have sat there
    }
    for (int q = tid; q < (ntile - 1) * B; q += nt) {
      const int tb = 1 + q / B, c = q - (tb - 1) * B;
      const int i0 = (kb + tb) * B;
      float col[B];
#pragma unroll
      for (int r = 0; r < B; ++r) col[r] = U[S.in_band(kb, r, i0 + c)];
      // column j of the factor is a row of L here: 16 bytes at a time (the same words for every lane)
      const float4 *L4 = (const float4 *)L;
      float rinv[B];
#pragma unroll
      for (int q4 = 0; q4 < B / 4; ++q4) {
        const float4 t4 = L4[B * B / 4 + q4];
        rinv[4 * q4] = t4.x, rinv[4 * q4 + 1] = t4.y, rinv[4 * q4 + 2] = t4.z, rinv[4 * q4 + 3] = t4.w;
      }
      // the entries of L for step j + 1 are asked for before step j's chain of multiply-adds
      float lt[2][B];
      auto fetch = [&](int j, float *to) {
#pragma unroll
        for (int q4 = (j + 1) / 4; q4 < B / 4; ++q4) {
          const float4 t4 = L4[j * (B / 4) + q4];
          to[4 * q4] = t4.x, to[4 * q4 + 1] = t4.y, to[4 * q4 + 2] = t4.z, to[4 * q4 + 3] = t4.w;
        }
      };
      fetch(0, lt[0]);
#pragma unroll
      for (int j = 0; j < B; ++j) {
        if (j + 1 < B) fetch(j + 1, lt[(j + 1) & 1]);
        const float z = col[j] * rinv[j];
        col[j] = z;
#pragma unroll
        for (int i = j + 1; i < B; ++i) col[i] = fma_(-lt[j & 1][i], z, col[i]);
      }
#pragma unroll
      for (int r = 0; r < B; ++r) U[S.in_band(kb, r, i0 + c)] = col[r];
    }
    __syncthreads();
  }
}

// rhs <- U^-1 rhs, block rows from the bottom.  Row r's value before its block's substitution is
//   s = rhs[r]; for j = r's block + 1 .. last block: s = s - sum_j,  sum_j = U[r][block j] . x[block j]
// with each sum_j a chain of B fused multiply-adds from zero.  The sums do not depend on s, so thread r
// forms sum_j as soon as block j is solved (every row above it at once) and keeps it in a register; when
// its own block's turn comes the subtractions run in ascending j as written above and the block's B lanes
// (one row of 16 DPP lanes, or half of one) substitute with row broadcasts.  One dependent chain of B
// terms per block row instead of one over all the columns to the right.
// Needs a thread per row and at most kBackBlocks block rows; backward_solve_serial covers the rest.
constexpr int kBackBlocks = 16;

template <int B>
__device__ __forceinline__ void backward_solve_serial(const float *U, float *rhs, int pad, int tid) {
  const Stair<B> S{pad};
  for (int i0 = pad - B; i0 >= 0; i0 -= B) {
    if (tid < 64) {
      const int r = tid < B ? tid : 0;
      float s = rhs[i0 + r];
      float urow[B];
      const float *Ur = U + S.in_band(i0 / B, r, 0);  // row i0 + r, indexed by column
#pragma unroll
      for (int c = 0; c < B; ++c) urow[c] = Ur[i0 + c];
      const float rinv = 1.0f / Ur[i0 + r];
      for (int j = i0 + B; j < pad; j += B) {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(Ur[j + t], rhs[j + t], sum);
        s = s - sum;
      }
      float my_x = 0.0f;
#pragma unroll
      for (int c = B - 1; c >= 0; --c) {
        const float x = row_bcast(s * rinv, c);
        my_x = tid == c ? x : my_x;
        s = fma_(-urow[c], x, s);  // meaningful for rows above c
      }
      if (tid < B) rhs[i0 + tid] = my_x;
    }
    __syncthreads();
  }
}

template <int B>
__device__ __forceinline__ void backward_solve(const float *U, float *rhs, int pad, int tid, int nt) {
  const int nblk = pad / B;
  if (nblk > kBackBlocks || pad > nt) {  // uniform
    backward_solve_serial<B>(U, rhs, pad, tid);
    return;
  }
  const Stair<B> S{pad};
  const bool has_row = tid < pad;
  const int r = has_row ? tid : 0, b = r / B, ri = r - b * B;
  const float *Ur = U + S.in_band(b, ri, 0);  // row r, indexed by column
  float urow[B];
#pragma unroll
  for (int c = 0; c < B; ++c) urow[c] = Ur[b * B + c];
  const float rinv = 1.0f / Ur[r];
  float part[kBackBlocks];
#pragma unroll
  for (int jb = kBackBlocks - 1; jb >= 0; --jb) {
    if (jb < nblk) {  // uniform
      if (has_row && b == jb) {
        float s = rhs[r];
#pragma unroll
        for (int j = jb + 1; j < kBackBlocks; ++j)
          if (j < nblk) s = s - part[j];
        constexpr int kRow = 16 / B;            // blocks per row of 16 DPP lanes
        const int off = (jb % kRow) * B;        // where this block's lanes start in their DPP row
        float my_x = 0.0f;
#pragma unroll
        for (int c = B - 1; c >= 0; --c) {
          const float x = row_bcast(s * rinv, off + c);
          my_x = ri == c ? x : my_x;
          s = fma_(-urow[c], x, s);  // meaningful for rows above c
        }
        rhs[r] = my_x;
      }
      __syncthreads();
      float sum = 0.0f;
      if (has_row && b < jb) {
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(Ur[jb * B + t], rhs[jb * B + t], sum);
      }
      part[jb] = sum;
    }
  }
}

// rhs <- U'^-1 rhs with a finished factor (the forward half of a solve-only step): the same
// operations on rhs as inside factor_forward.  Thread r keeps row r's value in a register; once a
// block is solved every row below it subtracts that block's sum (a chain of B terms from zero),
// blocks ascending.
template <int B>
__device__ __forceinline__ void forward_solve_serial(const float *U, float *rhs, int pad, int tid) {
  const Stair<B> S{pad};
  for (int k = 0; k < pad; k += B) {
    if (tid < 64) {
      const int i = tid < B ? tid : 0;
      float s = rhs[k + i];
      float ucol[B];
#pragma unroll
      for (int j = 0; j < B; ++j) ucol[j] = U[S.in_band(k / B, j, k + i)];
      const float rinv = 1.0f / U[S.in_band(k / B, i, k + i)];
      for (int j = 0; j < k; j += B) {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(U[S.in_band(j / B, t, k + i)], rhs[j + t], sum);
        s = s - sum;
      }
      float my_z = 0.0f;
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const float z = row_bcast(s * rinv, j);
        my_z = tid == j ? z : my_z;
        s = fma_(-ucol[j], z, s);  // meaningful for rows below j
      }
      if (tid < B) rhs[k + tid] = my_z;
    }
    __syncthreads();
  }
}

template <int B>
__device__ __forceinline__ void forward_solve(const float *U, float *rhs, int pad, int tid, int nt) {
  if (pad > nt) {  // uniform
    forward_solve_serial<B>(U, rhs, pad, tid);
    return;
  }
  const Stair<B> S{pad};
  const int nblk = pad / B;
  const bool has_row = tid < pad;
  const int r = has_row ? tid : 0, b = r / B, ri = r - b * B;
  float ucol[B];
#pragma unroll
  for (int j = 0; j < B; ++j) ucol[j] = U[S.in_band(b, j, r)];
  const float rinv = 1.0f / U[S.in_band(b, ri, r)];
  float s = rhs[r];
  for (int kb = 0; kb < nblk; ++kb) {
    if (has_row && b == kb) {
      constexpr int kRow = 16 / B;
      const int off = (kb % kRow) * B;
      float my_z = 0.0f;
      if (off == 0) {
#pragma unroll
        for (int j = 0; j < B; ++j) {
          const float z = row_bcast(s * rinv, j);
          my_z = ri == j ? z : my_z;
          s = fma_(-ucol[j], z, s);  // meaningful for rows below j
        }
      } else {
#pragma unroll
        for (int j = 0; j < B; ++j) {
          const float z = row_bcast(s * rinv, (16 - B) % 16 + j);
          my_z = ri == j ? z : my_z;
          s = fma_(-ucol[j], z, s);
        }
      }
      rhs[r] = my_z;
    }
    __syncthreads();
    if (has_row && b > kb) {
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < B; ++t) sum = fma_(U[S.in_band(kb, t, r)], rhs[kb * B + t], sum);
      s = s - sum;
    }
  }
}

// Compiled for four wavefronts per SIMD (128 registers a lane): four workgroups of 256 share a CU
// at pad 128, where the LDS admits them.
template <int B>
__global__ __launch_bounds__(256, 4) void blocked_factor_solve_kernel(
    const float *__restrict__ M, int64_t ldM, int nM, const int32_t *__restrict__ block_idx,
    const float *__restrict__ y, int64_t ldy, float *__restrict__ Uout, float *__restrict__ x,
    int64_t ldx, int nv, int pad, const int32_t *__restrict__ active) {
  extern __shared__ float lds[];
  if (active && active[blockIdx.x] == 0) return;  // the whole workgroup: nothing of this world is touched
  const Stair<B> S{pad};
  const int nU = S.words();
  float *U = lds;             // [nU] the factor, block row by block row
  float *rhs = U + nU;        // [pad]
  float *L = rhs + pad;       // [B * B + B] Cholesky factor of the diagonal block (column j in row j), 1 / pivots
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t w = blockIdx.x;
  for (int i = tid; i < pad; i += nt) rhs[i] = (y && i < nv) ? y[w * ldy + i] : 0.0f;  // factor only: no y, no x
  gather_tiles<B>(M + w * ldM, block_idx, nM, nv, pad, U, tid, nt);
  __syncthreads();
  const GatheredSrc<B> src{U, pad};
  factor_forward<B>(src, U, rhs, L, pad, tid, nt);
  backward_solve<B>(U, rhs, pad, tid, nt);
  if (x)
    for (int i = tid; i < nv; i += nt) x[w * ldx + i] = rhs[i];
  if (Uout)
    for (int i = tid; i < pad * pad / 4; i += nt) {  // pad is a multiple of B >= 8: a float4 stays in a tile
      const int r = 4 * i / pad, c = 4 * i - r * pad;
      // the tiles below the block diagonal are left as the caller has them (the reference's kernel
      // stores the tiles on and right of the diagonal only, indexed_factor.py:115, 141)
      if (c >= r / B * B) ((float4 *)(Uout + w * (int64_t)pad * pad))[i] = *(const float4 *)(U + S.at(r, c));
    }
}

// ---- matrices up to 64 x 64: four worlds per wavefront ----------------------------------------
// With a wavefront per world most of the factor runs on 8 or 16 of 64 lanes (the pivots of a tile,
// its triangular solves, the right-hand side), and the SIMDs spend their issue slots on idle
// lanes.  Here a world has a DPP row of 16 lanes and a wavefront carries four worlds through
// the same instructions; the only synchronisation is within the wavefront.  U keeps the tiles
// on or above the diagonal only, tile (bi, bj) at B B (bi nblk - bi (bi - 1) / 2 + bj - bi).
// Every element sees the operations of blocked_factor_solve_kernel<B> in the same order.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__host__ __device__ inline int quad_tiles_before(int bi, int nblk) { return bi * nblk - bi * (bi - 1) / 2; }
// floats of LDS per world: tiles (a block row is updated in place), right-hand side, the
// diagonal tile's lower factor and reciprocal pivots; rounded so that the four worlds start 8 banks apart
__host__ __device__ inline int quad_world_floats(int pad, int B) {
  const int nblk = pad / B;
  const int need = B * B * quad_tiles_before(nblk, nblk) + pad + B * B + B;
  return (need + 31) / 32 * 32 + 8;
}

template <int B>
__global__ __launch_bounds__(64) void blocked_factor_solve_quad_kernel(
    const float *__restrict__ M, int64_t ldM, int nM, const int32_t *__restrict__ block_idx,
    const float *__restrict__ y, int64_t ldy, float *__restrict__ Uout, float *__restrict__ x,
    int64_t ldx, int nv, int pad, int nworld, const int32_t *__restrict__ active) {
  extern __shared__ float lds[];
  constexpr int BB = B * B, PER = BB / 16;  // a lane's elements of a tile: e = l + 16 u
  const int lane = threadIdx.x, l = lane & 15, q = lane >> 4;
  const int nblk = pad / B, ntiles = quad_tiles_before(nblk, nblk);
  const int64_t w_raw = (int64_t)blockIdx.x * 4 + q;
  // an inactive world rides along like a spare row: computed, nothing stored
  const bool live = w_raw < nworld && (!active || active[w_raw] != 0);
  const int64_t w = w_raw < nworld ? w_raw : (int64_t)nworld - 1;  // a spare row repeats the last world and stores nothing
  const int world_floats = quad_world_floats(pad, B);
  float *U = lds + q * world_floats;
  float *rhs = U + BB * ntiles;  // [pad]
  float *L = rhs + pad;          // [BB + B]
  auto tile = [&](int bi, int bj) { return U + BB * (quad_tiles_before(bi, nblk) + bj - bi); };
  const float *Mw = M + w * ldM;
  {
    // indexed gather, four tiles in flight
    int kb = 0, ib = 0;
    for (int t0 = 0; t0 < ntiles; t0 += 4) {
      int tk[4], ti[4], idx[4][PER];
      float v[4][PER];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        tk[g] = kb < nblk ? kb : -1;
        ti[g] = ib;
        if (kb < nblk && ++ib == nblk) { ++kb; ib = kb; }
      }
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int u = 0; u < PER; ++u) {
          const int e = l + 16 * u;
          idx[g][u] = block_idx[tk[g] >= 0 ? (size_t)(tk[g] * nblk + ti[g]) * BB + e : 0];
          if (tk[g] < 0) idx[g][u] = nM;
        }
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int u = 0; u < PER; ++u) v[g][u] = Mw[idx[g][u] < nM ? idx[g][u] : 0];
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int u = 0; u < PER; ++u)
          if (tk[g] >= 0) {
            const int e = l + 16 * u, r = e / B, c = e % B;
            float xv = idx[g][u] < nM ? v[g][u] : 0.0f;
            if (ti[g] == tk[g] && (tk[g] + 1) * B > nv && r == c && (nblk - 1) * B + r >= nv) xv = xv + 1.0f;
            U[BB * (t0 + g) + e] = xv;
          }
    }
  }
  for (int i = l; i < pad; i += 16) rhs[i] = (y && i < nv) ? y[w * ldy + i] : 0.0f;
  wave_sync();
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  const int m4 = l & 3, qr = l >> 3, qc = (l >> 2) & 1;  // B = 8: the lane within quadrant (qr, qc) of a tile
  for (int kb = 0; kb < nblk; ++kb) {
    const int k = kb * B, ntile = nblk - kb;
    // The sums over a finished block row on the matrix cores, with instructions that do one
    // fused multiply-add per element and step: chained from zero over t ascending they are
    // the scalar sums bit for bit.
    for (int tb = 0; tb < ntile; ++tb) {
      const int ib = kb + tb;
      if constexpr (B == 8) {
        // v_mfma_f32_4x4x1_16b_f32: sixteen independent 4 x 4 blocks, the four quadrants of one
        // 8 x 8 tile of each of the four worlds
        float *Tv = tile(kb, ib) + (4 * qr) * B + 4 * qc + m4;  // rows 4 qr + 0..3 of column 4 qc + m4
        f32x4 v;
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = Tv[u * B];
        for (int jb = 0; jb < kb; ++jb) {
          const float *Tk = tile(jb, kb) + 4 * qr + m4, *Ti = tile(jb, ib) + 4 * qc + m4;
          f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int t = 0; t < B; ++t) sum = __builtin_amdgcn_mfma_f32_4x4x1f32(Tk[t * B], Ti[t * B], sum, 0, 0, 0);
#pragma unroll
          for (int u = 0; u < 4; ++u) v[u] = v[u] - sum[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) Tv[u * B] = v[u];  // in place: nothing else reads this tile before
      } else {
        // v_mfma_f32_16x16x1_4b_f32: four independent 16 x 16 blocks, one per world.  Block b takes
        // its operands from the lanes of world b and leaves its result in registers 4 b .. 4 b + 3
        // of every lane: rows 4 (lane / 16) + 0..3 of column lane % 16.
        const int toff = (int)(tile(kb, ib) - U) + (4 * q) * B + l;
        f32x16 v;
#pragma unroll
        for (int wb = 0; wb < 4; ++wb)
#pragma unroll
          for (int u = 0; u < 4; ++u) v[4 * wb + u] = lds[wb * world_floats + toff + u * B];
        for (int jb = 0; jb < kb; ++jb) {
          const float *Tk = tile(jb, kb) + l, *Ti = tile(jb, ib) + l;
          f32x16 sum;
#pragma unroll
          for (int u = 0; u < 16; ++u) sum[u] = 0.0f;
#pragma unroll
          for (int t = 0; t < B; ++t) sum = __builtin_amdgcn_mfma_f32_16x16x1f32(Tk[t * B], Ti[t * B], sum, 0, 0, 0);
#pragma unroll
          for (int u = 0; u < 16; ++u) v[u] = v[u] - sum[u];
        }
#pragma unroll
        for (int wb = 0; wb < 4; ++wb)
#pragma unroll
          for (int u = 0; u < 4; ++u) lds[wb * world_floats + toff + u * B] = v[4 * wb + u];
      }
    }
    if (l < B) {
      float s = rhs[k + l];
      for (int jb = 0; jb < kb; ++jb) {
        const float *Tk = tile(jb, kb);
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(Tk[t * B + l], rhs[jb * B + t], sum);
        s = s - sum;
      }
      rhs[k + l] = s;
    }
    wave_sync();
    {
      // Cholesky of the diagonal tile and the forward solve of the right-hand side, lane i of
      // the world's row holding row i (see blocked_factor_solve_kernel)
      const int i = l;
      float a[B];
#pragma unroll
      for (int j = 0; j < B; ++j) a[j] = tile(kb, kb)[(i < B ? i : 0) * B + j];
      float s = rhs[k + (i < B ? i : 0)];
#pragma unroll
      for (int j = 0; j < B; ++j) {
        float d, rinv;
        pivot_sqrt_rcp(row_bcast(a[j], j), true, d, rinv);
        const float lj = i == j ? d : a[j] * rinv;
        if (i >= j && i < B) L[i * B + j] = lj;
        const float z = row_bcast(s, j) * rinv;
        if (i == j) {
          rhs[k + j] = z;
          L[BB + j] = rinv;
        }
        s = fma_(-lj, z, s);
#pragma unroll
        for (int jj = j + 1; jj < B; ++jj) a[jj] = fma_(-lj, row_bcast(lj, jj), a[jj]);
      }
    }
    wave_sync();
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = l + 16 * u, r = e / B, c = e % B;
      tile(kb, kb)[e] = c >= r ? L[c * B + r] : 0.0f;
    }
    for (int qn = l; qn < (ntile - 1) * B; qn += 16) {
      const int tb = 1 + qn / B, cc = qn % B;
      float *Tt = tile(kb, kb + tb);
      float col[B];
#pragma unroll
      for (int r = 0; r < B; ++r) col[r] = Tt[r * B + cc];
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const float z = col[j] * L[BB + j];
        col[j] = z;
#pragma unroll
        for (int i = j + 1; i < B; ++i) col[i] = fma_(-L[i * B + j], z, col[i]);
      }
#pragma unroll
      for (int r = 0; r < B; ++r) Tt[r * B + cc] = col[r];
    }
    wave_sync();
  }
  // rhs <- U^-1 rhs, block rows from the bottom
  for (int ib = nblk - 1; ib >= 0; --ib) {
    const int i0 = ib * B, r = l < B ? l : 0;
    const float *Td = tile(ib, ib);
    float s = rhs[i0 + r];
    float urow[B];
#pragma unroll
    for (int cc = 0; cc < B; ++cc) urow[cc] = Td[r * B + cc];
    const float rinv = 1.0f / Td[r * B + r];
    for (int jb = ib + 1; jb < nblk; ++jb) {
      const float *Tj = tile(ib, jb);
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < B; ++t) sum = fma_(Tj[r * B + t], rhs[jb * B + t], sum);
      s = s - sum;
    }
#pragma unroll
    for (int cc = B - 1; cc >= 0; --cc) {
      const float xv = row_bcast(s * rinv, cc);
      if (l == cc) rhs[i0 + cc] = xv;
      s = fma_(-urow[cc], xv, s);
    }
    wave_sync();
  }
  if (live) {
    if (x)
      for (int i = l; i < nv; i += 16) x[w * ldx + i] = rhs[i];
    if (Uout) {
      float4 *dst = (float4 *)(Uout + w * (int64_t)pad * pad);
      for (int i4 = l; i4 < pad * pad / 4; i4 += 16) {
        const int row = 4 * i4 / pad, col = 4 * i4 - row * pad, bi = row / B, bj = col / B;
        if (bj >= bi) dst[i4] = *(const float4 *)(tile(bi, bj) + (row % B) * B + (col % B));  // lower tiles: not written
      }
    }
  }
}

// Per-iteration factor stage on the dense Hessian: dofs touched by the changed rows,
// incremental update of H's upper triangle, then either the augmented blocked Cholesky
// (the gradient rides as column pad - 1, corner 1e30) or, with no changed row, a solve with
// the stored factor.  Reference: src/instantmimic/utils/mjw_kernels/newton_stages.py
// :614-742 (stage), :451-470 (hessian_step), :473-611 (augmented factor).  search = -x,
// search_dot = x.x, decrement = grad.x (strided over 64 lanes, shuffle-down tree).
template <int B>
__global__ __launch_bounds__(256, 4) void dense_update_factor_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ state_changes,
    const int32_t *__restrict__ changes, const int32_t *__restrict__ ids, int ld_ids,
    const float *__restrict__ J, int njmax, const float *__restrict__ D, const int32_t *__restrict__ state,
    int quad, const float *__restrict__ grad, int64_t ldg, float *H_, float *U_,
    int32_t *__restrict__ uni_, float *__restrict__ search, int64_t lds_, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int pad, int row_cap) {
  extern __shared__ float lds[];
  // The factor proper covers the dofs rounded up to whole tiles (pf); the rows and columns from
  // there to pad are the identity with the augmented column and the corner in the last place,
  // which are written out directly: at nv = 128 the array in LDS is that of eight block rows, not
  // nine, and four worlds share a CU.
  const int pf = (nv + B - 1) / B * B;
  const Stair<B> S{pf};
  const int nU = S.words();
  float *U = lds;             // [nU] the factor, block row by block row
  float *rhs = U + nU;        // [pf]
  float *L = rhs + pf;        // [B * B + B]: factor of the diagonal tile (column j in row j), 1 / pivots
  int *ul = (int *)(L + B * B + B);  // [nv] union list, [nv] = its length
  unsigned *mkl = (unsigned *)(ul + nv + 1);  // [nv] per dof: nonzero when a changed row reaches it
  float *jr = (float *)(mkl + nv);  // [row_cap] signed weights of a batch of changed rows, [row_cap] their numbers
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t w = blockIdx.x;
  if ((done && done[w]) || state_changes[w] == 0) return;
  float *Hw = H_ + w * (int64_t)pad * pad, *Uw = U_ + w * (int64_t)pad * pad;
  const float *Jw = J + w * (int64_t)njmax * nv, *Dw = D + w * njmax, *gw = grad + w * ldg;
  const int32_t *sw = state + w * njmax, *idw = ids + w * ld_ids;
  // a negative count: H is taken as it lies in memory and factored (the first factor of a solve)
  int count = changes[w];
  const bool refactor = count != 0;
  count = count < 0 ? 0 : (count < ld_ids ? count : ld_ids);
  for (int i = tid; i < pf; i += nt) rhs[i] = i < nv ? gw[i] : 0.0f;
  if (refactor) {
    // The changed rows of J and their signed weights pass through LDS in batches that use the
    // factor's array while it is still free (up to 64 rows each), the pair sums staying in the
    // matrix cores' accumulators from one batch to the next; the sums go to H in memory, and H's
    // upper triangle is then brought into the array and factored in place.  Without room for a
    // batch of four rows the pairs are read from memory one by one.
    const bool staged = row_cap >= 4;
    float *sd = jr;  // [row_cap] signed weights of a batch
    if (staged) {
      float *jb = U;  // [row_cap][nv] a batch of changed rows
      for (int dof = tid; dof < nv; dof += nt) mkl[dof] = 0u;
      // All pair sums of a 16 x 16 tile of dofs at once on the matrix cores.  Every changed row
      // enters every pair here, also where one of the two dofs is zero in it: such a term adds
      // +-0 to a sum that started at +0, which leaves all its bits, so the sums equal the ones
      // that skip those rows.  v_mfma_f32_16x16x4_f32 adds its four products one after the
      // other with a fused multiply-add each, rows ascending; a batch holds a multiple of four
      // rows, so the chain of a pair runs through the batches as through one list.
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      constexpr int HELD = 9;  // tiles a wavefront keeps sums for at a time (36 over 4 wavefronts at nv 128: one pass over the rows); more tiles take another pass
      const int lane = tid & 63, p = lane & 15, kq = lane >> 4, wv = tid >> 6, nwv = nt >> 6;
      const int nb = (nv + 15) / 16, ntiles = nb * (nb + 1) / 2;
      // one pass holds every tile (always, with four wavefronts and up to 128 dofs)
      const bool one_pass = ntiles <= HELD * nwv;
      const bool FILLS = one_pass;  // the lanes that add the sums to H also leave the new H in the factor's array
      // thread t asks for the number and the signed weight of changed row t once, at the start: a
      // batch then finds them in registers instead of making two trips to memory of its own
      const bool ids_held = count <= nt;
      int my_row = 0;
      float my_sd = 0.0f;
      if (ids_held && tid < count) {
        my_row = idw[tid];
        my_sd = sw[my_row] == quad ? Dw[my_row] : -Dw[my_row];
      }
      for (int tile0 = 0; tile0 < ntiles; tile0 += HELD * nwv) {
        f32x4 acc[HELD];
        int ra[HELD], ca[HELD];
#pragma unroll
        for (int h = 0; h < HELD; ++h) {
          acc[h] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
          const int tile = tile0 + wv + h * nwv;
          int cb = (int)((sqrtf((float)(8 * tile + 1)) - 1.0f) * 0.5f);
          while ((cb + 1) * (cb + 2) / 2 <= tile) ++cb;
          while (cb * (cb + 1) / 2 > tile) --cb;
          const int rb = tile - cb * (cb + 1) / 2;
          ra[h] = tile < ntiles ? 16 * rb + p : -1;  // the dofs this lane feeds; -1: no such tile
          ca[h] = 16 * cb + p;
        }
        for (int c0 = 0; c0 < count; c0 += row_cap) {
          const int nrow = count - c0 < row_cap ? count - c0 : row_cap;
          __syncthreads();  // the batch before this one has been read by everyone
          // the batch's row numbers first, then every element of its rows is requested before the
          // first one is stored
          int *rowid = (int *)(sd + row_cap);
          if (ids_held) {
            if (tid >= c0 && tid < c0 + nrow) {
              rowid[tid - c0] = my_row;
              sd[tid - c0] = my_sd;
            }
          } else {
            for (int t = tid; t < nrow; t += nt) {
              const int r = idw[c0 + t];
              rowid[t] = r;
              sd[t] = sw[r] == quad ? Dw[r] : -Dw[r];
            }
          }
          __syncthreads();
          const int total = nrow * nv;
          constexpr int INFLIGHT = 16;
          for (int q0 = tid; q0 < total; q0 += INFLIGHT * nt) {
            float v[INFLIGHT];
#pragma unroll
            for (int k = 0; k < INFLIGHT; ++k) {
              const int q = q0 + k * nt < total ? q0 + k * nt : total - 1;
              const int t = q / nv;
              v[k] = Jw[(size_t)rowid[t] * nv + (q - t * nv)];
            }
#pragma unroll
            for (int k = 0; k < INFLIGHT; ++k)
              if (q0 + k * nt < total) jb[q0 + k * nt] = v[k];
          }
          __syncthreads();
          if (tile0 == 0)  // dofs some changed row reaches
            for (int dof = tid; dof < nv; dof += nt) {
              unsigned hit = mkl[dof];
              for (int t = 0; t < nrow && !hit; ++t) hit = jb[t * nv + dof] != 0.0f;
              mkl[dof] = hit;
            }
          // four rows at a time for all the held tiles: their sums are independent, so the matrix
          // cores work on one while the operands of the next arrive
          for (int t0 = 0; t0 < nrow; t0 += 4) {
            const int t = t0 + kq, tc = t < nrow ? t : nrow - 1;
            const float wgt = t < nrow ? sd[tc] : 0.0f;
            const float *row = jb + tc * nv;
#pragma unroll
            for (int h = 0; h < HELD; ++h) {
              if (ra[h] >= 0) {  // the same for the whole wavefront
                const float a = ra[h] < nv ? wgt * row[ra[h]] : 0.0f;  // -(D a) == (-D) a exactly
                const float b = (t < nrow && ca[h] < nv) ? row[ca[h]] : 0.0f;
                // operands exchanged: the lane then holds four consecutive columns of one row of H's tile
                // (16 bytes of H) instead of four rows of one column; a product's bits do not depend on the order
                acc[h] = __builtin_amdgcn_mfma_f32_16x16x4f32(b, a, acc[h], 0, 0, 0);
              }
            }
          }
        }
        // H's elements of up to five held tiles are requested before the first of their sums is added
        // (all nine at once would take the registers that let four worlds share a CU).  A lane holds
        // row ra[h] of the tile, columns 4 kq .. 4 kq + 3: right of the diagonal blocks and inside the
        // dofs that is one 16-byte request; elsewhere element by element.
        constexpr int APPLY = 5;
        const bool vec = ((uintptr_t)Hw & 15) == 0;  // pad is a multiple of 16
        if (one_pass) __syncthreads();  // the rows are done with the array: the new H goes there as well
#pragma unroll
        for (int h0 = 0; h0 < HELD; h0 += APPLY) {
          f32x4 hv[APPLY];
#pragma unroll
          for (int h = h0; h < h0 + APPLY && h < HELD; ++h) {
            const int row = ra[h], col0 = ca[h] - p + 4 * kq;
            const bool wide = vec && ra[h] >= 0 && ra[h] - p != ca[h] - p && row < nv && col0 + 3 < nv;
            const bool any = acc[h][0] != 0.0f || acc[h][1] != 0.0f || acc[h][2] != 0.0f || acc[h][3] != 0.0f;
            hv[h - h0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (wide) {
              if (any || FILLS) hv[h - h0] = *(const f32x4 *)(Hw + (size_t)row * pad + col0);
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const bool mine = ra[h] >= 0 && row <= col0 + i && col0 + i < nv && (FILLS || acc[h][i] != 0.0f);
                hv[h - h0][i] = mine ? Hw[(size_t)row * pad + col0 + i] : 0.0f;
              }
            }
          }
#pragma unroll
          for (int h = h0; h < h0 + APPLY && h < HELD; ++h) {
            const int row = ra[h], col0 = ca[h] - p + 4 * kq;
            const bool wide = vec && ra[h] >= 0 && ra[h] - p != ca[h] - p && row < nv && col0 + 3 < nv;
            const bool any = acc[h][0] != 0.0f || acc[h][1] != 0.0f || acc[h][2] != 0.0f || acc[h][3] != 0.0f;
            f32x4 hn = hv[h - h0];
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (acc[h][i] != 0.0f) hn[i] = hn[i] + acc[h][i];
            if (wide) {
              if (any) *(f32x4 *)(Hw + (size_t)row * pad + col0) = hn;
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (ra[h] >= 0 && row <= col0 + i && col0 + i < nv && acc[h][i] != 0.0f) Hw[(size_t)row * pad + col0 + i] = hn[i];
            }
            if (FILLS && ra[h] >= 0) {  // zero below the diagonal and past the dofs
              f32x4 o;
#pragma unroll
              for (int i = 0; i < 4; ++i) o[i] = (row <= col0 + i && col0 + i < nv) ? hn[i] : 0.0f;
              *(f32x4 *)(U + S.at(row, col0)) = o;
            }
          }
        }
      }
      __syncthreads();  // the rows are done with the array; this workgroup's writes to H are read back below
      // 16 bytes per lane and four requests in flight; the tiles below the diagonal are not read
      const int nvec = FILLS ? 0 : pf * pf / 4, last = (pf - 1) * (pad / 4) + pf / 4 - 1;  // pf is a multiple of 16
      for (int i0 = tid; i0 < nvec; i0 += 4 * nt) {
        float4 v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int i = i0 + k * nt < nvec ? i0 + k * nt : nvec - 1;
          const int r = 4 * i / pf, c = 4 * i - r * pf;
          v[k] = ((const float4 *)Hw)[c >= r / B * B ? r * (pad / 4) + c / 4 : last];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int i = i0 + k * nt;
          if (i < nvec) {
            const int r = 4 * i / pf, c = 4 * i - r * pf;
            if (c >= r / B * B) {
              float4 o;
              o.x = (r < nv && c + 0 < nv && r <= c + 0) ? v[k].x : 0.0f;
              o.y = (r < nv && c + 1 < nv && r <= c + 1) ? v[k].y : 0.0f;
              o.z = (r < nv && c + 2 < nv && r <= c + 2) ? v[k].z : 0.0f;
              o.w = (r < nv && c + 3 < nv && r <= c + 3) ? v[k].w : 0.0f;
              *(float4 *)(U + S.at(r, c)) = o;
            }
          }
        }
      }
      __syncthreads();
    }
    if (tid < 64) {
      int nu = 0;
      for (int base = 0; base < nv; base += 64) {
        const int dof = base + tid;
        bool hit = false;
        if (dof < nv) {
          if (staged) {
            hit = mkl[dof] != 0u;
          } else {
            for (int t = 0; t < count && !hit; ++t) hit = Jw[(size_t)idw[t] * nv + dof] != 0.0f;
          }
        }
        const unsigned long long mask = __ballot(hit);
        if (hit) ul[nu + __popcll(mask & ((1ull << tid) - 1ull))] = dof;
        nu += __popcll(mask);
      }
      if (tid == 0) ul[nv] = nu;
    }
    __syncthreads();
    const int nu = ul[nv];
    int32_t *uni = uni_ + w * (nv + 1);
    for (int i = tid; i < nu; i += nt) uni[i] = ul[i];
    if (tid == 0) uni[nv] = nu;
    if (!staged) {
      const int npair = nu * (nu + 1) / 2;
      for (int e = tid; e < npair; e += nt) {
        int cj = (int)((sqrtf((float)(8 * e + 1)) - 1.0f) * 0.5f);
        while ((cj + 1) * (cj + 2) / 2 <= e) ++cj;
        while (cj * (cj + 1) / 2 > e) --cj;
        const int row = ul[e - cj * (cj + 1) / 2], col = ul[cj];
        float delta = 0.0f;
        for (int t = 0; t < count; ++t) {
          const int r = idw[t];
          const float a = Jw[(size_t)r * nv + row], b = Jw[(size_t)r * nv + col];
          float da = Dw[r] * a;
          if (sw[r] != quad) da = -da;
          if (a != 0.0f && b != 0.0f) delta = fma_(da, b, delta);
        }
        if (delta != 0.0f) Hw[(size_t)row * pad + col] = Hw[(size_t)row * pad + col] + delta;
      }
    }
    if (staged) {
      __syncthreads();
      const LdsSrc<B> src{U, nv, pf};
      factor_forward<B>(src, U, rhs, L, pf, tid, nt);
    } else {
      for (int i = tid; i < nU; i += nt) U[i] = 0.0f;
      __syncthreads();  // this workgroup's own writes to H are read back below
      const DenseSrc<B> src{Hw, nv, pad};  // pad: the row stride of H in memory
      factor_forward<B>(src, U, rhs, L, pf, tid, nt);
    }
    // stored factor: the augmented column z = U'^-1 grad above the corner sqrt(1e30 - z.z)
    if (tid < 64) {
      // the chain v = fma(-z_i, z_i, v) over i ascending; the z's come 64 at a time into the
      // lanes and reach the chain through lane reads instead of one LDS round trip each
      float v = 1.0e30f;
      for (int base = 0; base < nv; base += 64) {
        const float z = base + tid < nv ? rhs[base + tid] : 0.0f;
        const int n = nv - base < 64 ? nv - base : 64;
        for (int i = 0; i < n; ++i) {
          const float zi = __shfl(z, i, 64);
          v = fma_(-zi, zi, v);
        }
      }
      if (tid == 0) L[0] = sqrtf(v);
    }
    __syncthreads();
    for (int i = tid; i < pad * pad / 4; i += nt) {  // pad is a multiple of 16: a float4 stays in a row
      const int r = 4 * i / pad, c = 4 * i - r * pad;
      float4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      if (r < pf && c < pf) {
        if (c >= r / B * B) v = *(const float4 *)(U + S.at(r, c));
      } else if (r >= pf && r - c >= 0 && r - c < 4) {  // the identity below and right of the factor
        v.x = r == c ? 1.0f : 0.0f, v.y = r == c + 1 ? 1.0f : 0.0f, v.z = r == c + 2 ? 1.0f : 0.0f, v.w = r == c + 3 ? 1.0f : 0.0f;
      }
      if (c + 3 == pad - 1) v.w = r < nv ? rhs[r] : (r == pad - 1 ? L[0] : v.w);
      if (c >= r / B * B) ((float4 *)Uw)[i] = v;  // the tiles below the block diagonal are not written
    }
    __syncthreads();  // rhs is overwritten by the backward solve
  } else {
    const int nvec = pf * pf / 4, last = (pf - 1) * (pad / 4) + pf / 4 - 1;
    for (int i0 = tid; i0 < nvec; i0 += 4 * nt) {
      float4 v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int i = i0 + k * nt < nvec ? i0 + k * nt : nvec - 1;
        const int r = 4 * i / pf, c = 4 * i - r * pf;
        v[k] = ((const float4 *)Uw)[c >= r / B * B ? r * (pad / 4) + c / 4 : last];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int i = i0 + k * nt;
        if (i < nvec) {
          const int r = 4 * i / pf, c = 4 * i - r * pf;
          if (c + 3 == pad - 1) v[k].w = r == pad - 1 ? 1.0f : 0.0f;  // drop the augmented column
          if (c >= r / B * B) *(float4 *)(U + S.at(r, c)) = v[k];
        }
      }
    }
    __syncthreads();
    forward_solve<B>(U, rhs, pf, tid, nt);
  }
  backward_solve<B>(U, rhs, pf, tid, nt);
  if (tid < 64) {
    float s0 = 0.0f, s1 = 0.0f;
    for (int i = tid; i < nv; i += 64) {
      const float v = rhs[i];
      search[w * lds_ + i] = -v;
      s0 = fma_(v, v, s0);
      s1 = fma_(gw[i], v, s1);
    }
    for (int o = 32; o > 0; o >>= 1) {
      s0 = s0 + __shfl_down(s0, o, 64);
      s1 = s1 + __shfl_down(s1, o, 64);
    }
    if (tid == 0) {
      search_dot[w] = s0;
      decrement[w] = s1;
    }
  }
}

// ---------------------------------------------------------------------------- stored factor, several right-hand sides
// x = (U'U)^-1 y for `nrhs` columns with a factor computed earlier: forward substitution with U',
// backward with U, block by block as the fused kernels do for their single right-hand side, so a
// column here sees the operations of blocked_factor_solve_kernel in the same order.
// Reference: multi_solve_indexed_cholesky_kernel and the solve half of
// factor_multi_solve_indexed_cholesky_kernel
// (src/instantmimic/utils/mjw_kernels/indexed_factor.py:394-493, 217-391).
// One wavefront per world: the upper triangle of U packed row by row in LDS, the right-hand
// sides beside it; lane (r, c) = row r of the current block, column c of a group of 64 / B columns.
__host__ __device__ inline int packed_upper_at(int r, int c, int pad) { return r * pad - r * (r - 1) / 2 + (c - r); }

template <int B>
__global__ __launch_bounds__(64) void blocked_multi_solve_kernel(
    const float *__restrict__ Uin, const float *__restrict__ y, const int32_t *__restrict__ active,
    float *__restrict__ x, int nv, int pad, int nrhs) {
  extern __shared__ float lds[];
  const int64_t w = blockIdx.x;
  if (active && active[w] == 0) return;
  float *U = lds;                          // [pad (pad + 1) / 2]
  float *rhs = U + pad * (pad + 1) / 2;    // [pad][nrhs]
  const int lane = threadIdx.x, r = lane % B, cg = lane / B;
  constexpr int CPL = 64 / B;              // columns per pass
  const float *Uw = Uin + w * (int64_t)pad * pad;
  for (int i = lane; i < pad * pad; i += 64) {
    const int row = i / pad, col = i - row * pad;
    if (col >= row) U[packed_upper_at(row, col, pad)] = Uw[i];
  }
  for (int i = lane; i < pad * nrhs; i += 64) rhs[i] = i < nv * nrhs ? y[w * (int64_t)nv * nrhs + i] : 0.0f;
  wave_sync();
  for (int c0 = 0; c0 < nrhs; c0 += CPL) {
    const int col = c0 + cg < nrhs ? c0 + cg : nrhs - 1;  // spare lanes repeat the last column
    const bool mine = c0 + cg < nrhs;
    const int base = cg * B;                              // first lane of this column's group
    // forward: z = U'^-1 y
    for (int k = 0; k < pad; k += B) {
      float s = rhs[(k + r) * nrhs + col];
      for (int j = 0; j < k; j += B) {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(U[packed_upper_at(j + t, k + r, pad)], rhs[(j + t) * nrhs + col], sum);
        s = s - sum;
      }
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const float inv = 1.0f / U[packed_upper_at(k + j, k + j, pad)];
        const float z = __shfl(s * inv, base + j);
        if (r == j) s = z;
        if (r > j) s = fma_(-U[packed_upper_at(k + j, k + r, pad)], z, s);
      }
      wave_sync();  // every lane has read this block's old values
      if (mine) rhs[(k + r) * nrhs + col] = s;
      wave_sync();
    }
    // backward: x = U^-1 z
    for (int i0 = pad - B; i0 >= 0; i0 -= B) {
      float s = rhs[(i0 + r) * nrhs + col];
      for (int j = i0 + B; j < pad; j += B) {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < B; ++t) sum = fma_(U[packed_upper_at(i0 + r, j + t, pad)], rhs[(j + t) * nrhs + col], sum);
        s = s - sum;
      }
#pragma unroll
      for (int rr = B - 1; rr >= 0; --rr) {
        const float inv = 1.0f / U[packed_upper_at(i0 + rr, i0 + rr, pad)];
        const float xv = __shfl(s * inv, base + rr);
        if (r == rr) s = xv;
        if (r < rr) s = fma_(-U[packed_upper_at(i0 + r, i0 + rr, pad)], xv, s);
      }
      wave_sync();
      if (mine) rhs[(i0 + r) * nrhs + col] = s;
      wave_sync();
    }
  }
  for (int i = lane; i < nv * nrhs; i += 64) x[w * (int64_t)nv * nrhs + i] = rhs[i];
}

// L_out[w, adr[0] + row * nv + col] = U[w, row, col] over the nv x nv corner: the blocked upper
// factor in the dense-block layout of the caller's factor array
// (_copy_dense_factor_kernel, src/instantmimic/utils/mjw_step_optimized.py:875-886).
__global__ __launch_bounds__(256) void copy_dense_factor_kernel(const float *__restrict__ U, int pad,
                                                                const int32_t *__restrict__ block_adr, int nv,
                                                                float *__restrict__ L_out, int64_t ld_out) {
  const int64_t w = blockIdx.y;
  const int slot = blockIdx.x * 256 + threadIdx.x;
  if (slot >= nv * nv) return;
  const int row = slot / nv, col = slot - row * nv;
  L_out[w * ld_out + block_adr[0] + slot] = U[(w * pad + row) * (int64_t)pad + col];
}

// ---------------------------------------------------------------------------- dense J'DJ
// H[w] = M[w] + J[w]' diag(Dc[w]) J[w], H (nv_pad, nv_pad), on v_mfma_f32_16x16x4_f32.
// One workgroup of four wavefronts per world.  The 16 x 16 output tiles on and right of the block
// diagonal are dealt to the wavefronts round robin (36 tiles at 128 dofs: nine each, where 32 x 32
// tiles left two wavefronts with two tiles against three), accumulators in registers, mirrored at
// the end.  J is staged through LDS 32 rows at a time with the row weights beside it, in two
// copies used in turn; the next 32 rows are already on their way into registers while the matrix
// cores work on the current ones, and the weighted operand (J Dc) is formed when it is fed.
// An element's sum is the chain fma(J[r][i] * Dc[r], J[r][j], .) over the rows in order, from M.

// The 36 tiles of a matrix of eight 16-column blocks, nine per wavefront, chosen so that a
// wavefront's tiles share operands: wavefronts 0 and 1 take the triangles of blocks 0-3 and 4-7
// (four blocks read per step of four rows, each also in its weighted form), wavefronts 2 and 3
// the rectangle of rows 0-1 / 2-3 against columns 4-7 (six blocks read) and, to even the count,
// one diagonal tile of a block they hold anyway.  {row block, column block}.
__device__ constexpr signed char kJtdjTile[4][9][2] = {
    {{0, 1}, {0, 2}, {0, 3}, {1, 1}, {1, 2}, {1, 3}, {2, 2}, {2, 3}, {3, 3}},
    {{4, 4}, {4, 5}, {4, 6}, {4, 7}, {5, 5}, {5, 6}, {5, 7}, {6, 6}, {6, 7}},
    {{0, 4}, {0, 5}, {0, 6}, {0, 7}, {1, 4}, {1, 5}, {1, 6}, {1, 7}, {0, 0}},
    {{2, 4}, {2, 5}, {2, 6}, {2, 7}, {3, 4}, {3, 5}, {3, 6}, {3, 7}, {7, 7}},
};
constexpr bool jtdj_role_reads(int role, int b) {  // does a wavefront of this role use block b at all
  for (int m = 0; m < 9; ++m)
    if (kJtdjTile[role][m][0] == b || kJtdjTile[role][m][1] == b) return true;
  return false;
}
constexpr bool jtdj_role_weights(int role, int b) {  // ... and in its weighted form (as a tile's row block)
  for (int m = 0; m < 9; ++m)
    if (kJtdjTile[role][m][0] == b) return true;
  return false;
}

// NVR: the staged row width when it is known at compile time (operand addresses then differ by
// constants that the LDS instructions carry themselves), 0 for any width.
// ROLE: 0..3 = this wavefront's row of kJtdjTile (eight blocks, NVR 128), -1 = tiles dealt round
// robin at run time, each with operand reads of its own.
// `out(i0, j, h, off)` receives what a lane holds of each tile: rows i0 .. i0 + 3 of column j (the
// elements with i <= j < nv are H's), and whether the tile lies right of the diagonal blocks.
template <int NVR, int ROLE, class Out>
__device__ __forceinline__ void jtdj_tiles_as(const float *__restrict__ Mdense, const float *__restrict__ J, int njmax,
                                           const float *__restrict__ D, const int32_t *__restrict__ state,
                                           const int32_t *__restrict__ nefc_p, int quad, int nv, float *lds,
                                           const Out &out) {
  const int nvr = NVR ? NVR : (nv + 31) / 32 * 32;   // staged row width
  // two copies of the staging area: the rows of the next chunk are written while wavefronts that
  // are behind still read the current one, which leaves one barrier per chunk
  const int stage_words = 32 * nvr + 32;
  float *Js = lds;                       // [32][nvr] J rows (zero past nefc and past nv)
  float *dcs = Js + 32 * nvr;            // [32] their weights
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t w = blockIdx.x;
  const int nb = (nv + 15) / 16;
  // A matrix-core operand is 16 columns of four consecutive rows, which lie a whole number of
  // bank rounds apart: the 16-column groups of a row are stored exchanged by the row's number
  // (all four ways where the width is a multiple of 64, two ways otherwise), so the four rows of
  // a request fall on different banks.
  const int swz = nvr % 64 == 0 ? 3 : 1;
  const int kq = lane >> 4, kqs = kq & swz;
  // tiles (bi <= bj) distributed over the four waves; each wave keeps its tiles' accumulators
  constexpr int MAXT = ROLE >= 0 ? 9 : 7;  // 36 tiles at eight blocks over 4 wavefronts; dealt at run time: up to seven blocks, 28 tiles
  float4v acc[MAXT];
  int tbi[MAXT], tbj[MAXT], mine = 0;
  if (ROLE >= 0) {
#pragma unroll
    for (int m = 0; m < MAXT; ++m) {
      tbi[m] = kJtdjTile[ROLE < 0 ? 0 : ROLE][m][0];
      tbj[m] = kJtdjTile[ROLE < 0 ? 0 : ROLE][m][1];
    }
    mine = MAXT;
  } else {
    int t = 0;
#pragma unroll
    for (int m = 0; m < MAXT; ++m) tbi[m] = tbj[m] = 0;
    for (int bi = 0; bi < nb; ++bi)
      for (int bj = bi; bj < nb; ++bj, ++t)
        if ((t & 3) == wave) {
#pragma unroll
          for (int m = 0; m < MAXT; ++m)
            if (mine == m) { tbi[m] = bi; tbj[m] = bj; }
          ++mine;
        }
    mine = mine < MAXT ? mine : MAXT;
  }
  // The accumulators start from M (accumulator layout of a 16x16 tile: lane l holds column
  // j = l % 16 and, in register v, row i = 4 * (l / 16) + v): every lane asks for all its elements
  // at once, with clamped indices so that no load hangs on a condition, and the answers arrive
  // while the first rows of J are staged.
  const float *Mw = Mdense + w * (int64_t)nv * nv;
#pragma unroll
  for (int m = 0; m < MAXT; ++m) {
    const int j = tbj[m] * 16 + (lane & 15), jc = j < nv ? j : nv - 1;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int i = tbi[m] * 16 + 4 * kq + v, ic = i < nv ? i : nv - 1;
      acc[m][v] = Mw[(int64_t)ic * nv + jc];
    }
  }
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  const float *Jw = J + w * (int64_t)njmax * nv;
  const float *Dw = D + w * njmax;
  const int32_t *sw = state + w * njmax;
  // a wavefront stages 8 of a chunk's 32 rows, lanes across the columns (two per lane)
  const int c0 = lane, c1 = lane + 64;
  const int c0c = c0 < nv ? c0 : nv - 1, c1c = c1 < nv ? c1 : nv - 1;
  float v0[8], v1[8], dd = 0.0f;
  int sd = 0;
  // The first 32 rows are read as they lie.  Of the rows behind them only those that contribute
  // (inside nefc, state `quad`) are read at all: every wavefront counts them by ballot, 256 rows
  // per round with the loads of a round issued together, and the wavefronts share out the writing
  // of the list of their numbers and weights, which the barrier behind the first chunk publishes.
  int *rowl = (int *)(lds + 2 * stage_words);  // [njmax rounded up to 4]
  float *dl = (float *)(rowl + ((njmax + 3) & ~3));
  {  // every load is issued whatever the row: clamped, selected later
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = wave * 8 + i, rowc = row < njmax ? row : njmax - 1;
      v0[i] = Jw[(int64_t)rowc * nv + c0c];
      v1[i] = Jw[(int64_t)rowc * nv + c1c];
    }
    const int row = wave * 8 + (lane & 7), rowc = row < njmax ? row : njmax - 1;
    dd = Dw[rowc];
    sd = sw[rowc];
  }
  int cnt = 0;
  for (int r = 32; r < njmax; r += 256) {
    int st[4];
    float dv[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = r + 64 * q + lane, rowc = row < njmax ? row : njmax - 1;
      st[q] = sw[rowc];
      dv[q] = Dw[rowc];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = r + 64 * q + lane;
      const bool act = row < nefc && st[q] == quad;
      const uint64_t mask = __ballot(act);
      if (q == wave && act) {
        const int pos = cnt + __popcll(mask & ((1ull << lane) - 1));
        rowl[pos] = row;
        dl[pos] = dv[q];
      }
      cnt += __popcll(mask);
    }
  }
  auto prefetch = [&](int p0) {  // list positions p0 .. p0 + 31
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int pos = p0 + wave * 8 + i, row = pos < cnt ? rowl[pos] : 0;
      v0[i] = Jw[(int64_t)row * nv + c0c];
      v1[i] = Jw[(int64_t)row * nv + c1c];
    }
  };
  auto stage = [&](int p0, int buf, bool listed) {
    float *Jb = Js + buf * stage_words, *db = dcs + buf * stage_words;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool in = p0 + wave * 8 + i < (listed ? cnt : nefc);
      const int x = 16 * ((wave * 8 + i) & swz);  // the row's exchange of its 16-column groups
      if (c0 < nvr) Jb[(wave * 8 + i) * nvr + (c0 ^ x)] = (in && c0 < nv) ? v0[i] : 0.0f;  // nvr is 32 for nv <= 32
      if (c1 < nvr) Jb[(wave * 8 + i) * nvr + (c1 ^ x)] = (in && c1 < nv) ? v1[i] : 0.0f;
    }
    if (lane < 8) {
      const int pos = p0 + wave * 8 + lane;
      db[wave * 8 + lane] = listed ? (pos < cnt ? dl[pos] : 0.0f) : ((pos < nefc && sd == quad) ? dd : 0.0f);
    }
  };
  stage(0, 0, false);
  __syncthreads();
  const int nchunk = nefc > 0 ? 1 + (cnt + 31) / 32 : 0;
  for (int c = 0, buf = 0; c < nchunk; ++c, buf ^= 1) {
    prefetch(32 * c);
    // v_mfma_f32_16x16x4_f32: lane l supplies A[i = l % 16][k = l / 16] and B[k = l / 16][j = l % 16]
    // the wavefront's tiles take turns inside the loop over the rows: independent accumulators
    // keep the matrix core busy while one of them waits for its previous result
    const float *Jc = Js + buf * stage_words, *dc = dcs + buf * stage_words;
    if (ROLE >= 0) {
      constexpr int R = ROLE < 0 ? 0 : ROLE;
      const float *pblk[8];
#pragma unroll
      for (int b = 0; b < 8; ++b) pblk[b] = Jc + kq * nvr + (b ^ kqs) * 16 + (lane & 15);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float dk = dc[4 * q + kq];
        float u[8], wt[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) u[b] = jtdj_role_reads(R, b) ? pblk[b][4 * q * nvr] : 0.0f;
#pragma unroll
        for (int b = 0; b < 8; ++b) wt[b] = jtdj_role_weights(R, b) ? u[b] * dk : 0.0f;
#pragma unroll
        for (int m = 0; m < MAXT; ++m)
          acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(wt[kJtdjTile[R][m][0]], u[kJtdjTile[R][m][1]], acc[m], 0, 0, 0);
      }
    } else {
      const float *pa[MAXT], *pb[MAXT];
#pragma unroll
      for (int m = 0; m < MAXT; ++m) {
        pa[m] = Jc + kq * nvr + (tbi[m] ^ kqs) * 16 + (lane & 15);
        pb[m] = Jc + kq * nvr + (tbj[m] ^ kqs) * 16 + (lane & 15);
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float dk = dc[4 * q + kq];
#pragma unroll
        for (int m = 0; m < MAXT; ++m)
          if (m < mine)
            acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[m][4 * q * nvr] * dk, pb[m][4 * q * nvr], acc[m], 0, 0, 0);
      }
    }
    // the other copy was last read one chunk ago, before the barrier that every wavefront has passed since
    stage(32 * c, buf ^ 1, true);
    __syncthreads();
  }
#pragma unroll
  for (int m = 0; m < MAXT; ++m) {
    if (m >= mine) continue;
    out(tbi[m] * 16 + 4 * kq, tbj[m] * 16 + (lane & 15), acc[m], tbi[m] != tbj[m]);
  }
}

template <int NVR, class Out>
__device__ __forceinline__ void jtdj_tiles(const float *__restrict__ Mdense, const float *__restrict__ J, int njmax,
                                           const float *__restrict__ D, const int32_t *__restrict__ state,
                                           const int32_t *__restrict__ nefc_p, int quad, int nv, float *lds,
                                           const Out &out) {
  // NVR == 128 is launched for 113 .. 128 dofs only (eight blocks): a code path per wavefront, every
  // path with the same barriers, and nothing else in the kernel -- the run-time dealing of tiles
  // needs more registers than four workgroups per CU leave, and a kernel's register and scratch
  // budget is that of its most expensive path
  if constexpr (NVR == 128) {
    switch (threadIdx.x >> 6) {
      case 0: jtdj_tiles_as<NVR, 0>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, out); break;
      case 1: jtdj_tiles_as<NVR, 1>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, out); break;
      case 2: jtdj_tiles_as<NVR, 2>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, out); break;
      default: jtdj_tiles_as<NVR, 3>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, out); break;
    }
  } else {
    jtdj_tiles_as<NVR, -1>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, out);
  }
}

// four workgroups per CU at 128 dofs (measured 0.83 -> 0.77 ms for 16384 worlds in spite of the
// spilled registers), three otherwise
template <int NVR>
__global__ __launch_bounds__(256, NVR == 128 ? 4 : 3) void jtdj_mfma_kernel(
    const float *__restrict__ Mdense, const float *__restrict__ J, int njmax,
    const float *__restrict__ D, const int32_t *__restrict__ state, const int32_t *__restrict__ nefc_p,
    int quad, float *__restrict__ H, int nv, int nv_pad) {
  extern __shared__ float lds[];
  float *Hw = H + blockIdx.x * (int64_t)nv_pad * nv_pad;
  // upper triangle from the accumulators, lower triangle mirrored: H is symmetric bit for bit
  const bool vec = (nv_pad & 3) == 0 && ((uintptr_t)H & 15) == 0;
  jtdj_tiles<NVR>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, [&](int i0, int j, float4v h, bool off) {
    store_h_mirrored(Hw, nv, nv_pad, vec, i0, j, h, off);
  });
}

// The same assembly followed, in the same workgroup, by the blocked Cholesky of H and the solve:
// H goes to memory (the per-iteration stage keeps updating it there) and into the factor's LDS
// array at once, so the factor neither gathers it from memory nor waits for another launch, and
// on a CU the matrix-core phase of one world runs beside the pivot chains of the others.  The rows
// of J are staged in the factor's array, which is free until H is complete.  Results are those of
// im_jtdj_mfma followed by im_blocked_factor_solve (B = 16) bit for bit.
template <int NVR>
__global__ __launch_bounds__(256, NVR == 128 ? 4 : 3) void jtdj_factor_solve_kernel(
    const float *__restrict__ Mdense, const float *__restrict__ J, int njmax, const float *__restrict__ D,
    const int32_t *__restrict__ state, const int32_t *__restrict__ nefc_p, int quad, float *__restrict__ H, int nv,
    int nv_pad, const float *__restrict__ y, int64_t ldy, float *__restrict__ Uout, float *__restrict__ x, int64_t ldx,
    int pad) {
  constexpr int B = 16;
  extern __shared__ float lds[];
  const Stair<B> S{pad};
  const int nU = S.words();
  const int nvr = NVR ? NVR : (nv + 31) / 32 * 32, stage_words = 2 * (32 * nvr + 32) + 2 * ((njmax + 3) & ~3);
  float *U = lds;       // first the staged rows of J (two copies) and the list of contributing rows, then [nU] H, then the factor
  float *rhs = lds + (nU > stage_words ? nU : stage_words);  // [pad]
  float *L = rhs + pad;  // [B * B + B]
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t w = blockIdx.x;
  for (int i = tid; i < pad; i += nt) rhs[i] = (y && i < nv) ? y[w * ldy + i] : 0.0f;
  float *Hw = H ? H + w * (int64_t)nv_pad * nv_pad : nullptr;
  // the assembly's last barrier is behind every wavefront when the elements come out, so they can
  // go where the rows were staged.  The factor reads the upper triangle below nv only (the rest
  // of a diagonal tile by symmetry, the padding as the identity) and writes every entry of a block
  // row before anything reads it, so the array needs no clearing.
  const bool vec = (nv_pad & 3) == 0 && ((uintptr_t)H & 15) == 0;
  jtdj_tiles<NVR>(Mdense, J, njmax, D, state, nefc_p, quad, nv, lds, [&](int i0, int j, float4v h, bool off) {
    if (Hw) store_h_mirrored(Hw, nv, nv_pad, vec, i0, j, h, off);
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (i0 + v < nv && j < nv && i0 + v <= j) U[S.at(i0 + v, j)] = h[v];
  });
  __syncthreads();
  const LdsSrc<B> src{U, nv, pad};
  factor_forward<B>(src, U, rhs, L, pad, tid, nt);
  backward_solve<B>(U, rhs, pad, tid, nt);
  if (x)
    for (int i = tid; i < nv; i += nt) x[w * ldx + i] = rhs[i];
  if (Uout)
    for (int i = tid; i < pad * pad / 4; i += nt) {
      const int r = 4 * i / pad, c = 4 * i - r * pad;
      // the tiles below the block diagonal are left as the caller has them (the reference's kernel
      // stores the tiles on and right of the diagonal only, indexed_factor.py:115, 141)
      if (c >= r / B * B) ((float4 *)(Uout + w * (int64_t)pad * pad))[i] = *(const float4 *)(U + S.at(r, c));
    }
}

// Every float whose bit pattern lies in [first, last] and that is in the pivots' range: do the
// short forms give the bits of sqrtf and of 1.0f / sqrtf?
__global__ void check_pivot_sqrt_kernel(uint32_t first, uint32_t last, unsigned long long *mismatches) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  unsigned long long bad = 0;
  for (uint64_t u = (uint64_t)first + blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; u <= last; u += stride) {
    const float x = __builtin_bit_cast(float, (uint32_t)u);
    if (!pivot_in_range(x)) continue;
    float d, rinv;
    pivot_sqrt_rcp_fast(x, d, rinv);
    const float want = sqrtf(x);
    bad += __builtin_bit_cast(uint32_t, d) != __builtin_bit_cast(uint32_t, want);
    bad += __builtin_bit_cast(uint32_t, rinv) != __builtin_bit_cast(uint32_t, 1.0f / want);
  }
  if (bad) atomicAdd(mismatches, bad);
}

}  // namespace
}  // namespace im

extern "C" {

// Factor store of im_blocked_factor_multi_solve_static: one array per GPU, held from the moment
// the library is loaded on it until the process ends.  In host code the name below is only a
// handle for hipGetSymbolAddress; kernels get the address that call returns.
static __device__ __align__(256) float scratch[IM_STATIC_SCRATCH_BYTES / sizeof(float)];

// Address of `scratch` on the current device, looked up once per device.
static int static_scratch(float **out) {
  constexpr int kMaxDevices = 64;
  static float *ptr[kMaxDevices] = {};
  static std::mutex guard;
  int dev = -1;
  IM_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return IM_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(guard);
  if (!ptr[dev]) {
    float *p = nullptr;
    IM_HIP_CHECK(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return IM_OK;
}

// factor (+ forward / backward solve when y and x are given) for every world whose `active`
// entry is nonzero (all when null)
static int launch_blocked_factor(const float *M, int64_t ldM, int nM, const int32_t *block_idx, int block_size,
                                 int nv, int pad, const float *y, int64_t ldy, float *U, float *x, int64_t ldx,
                                 const int32_t *active, int nworld, void *stream) {
  const int B = block_size;
  static const bool quad_off = [] {
    const char *e = std::getenv("IMHIP_BLOCKED_KERNEL");
    return e && std::strcmp(e, "simple") == 0;
  }();
  if (pad <= (B == 8 ? 64 : 48) && !quad_off) {
    // small matrices: four worlds per wavefront (16 x 16 tiles at pad 64 need 46 KB of LDS per
    // wavefront, three per CU, and are no faster that way)
    const size_t quad_bytes = sizeof(float) * 4 * (size_t)im::quad_world_floats(pad, B);
    auto qfn = B == 8 ? im::blocked_factor_solve_quad_kernel<8> : im::blocked_factor_solve_quad_kernel<16>;
    hipLaunchKernelGGL(qfn, dim3((unsigned)((nworld + 3) / 4)), dim3(64), quad_bytes, (hipStream_t)stream, M, ldM, nM,
                       block_idx, y, ldy, U, x, ldx, nv, pad, nworld, active);
    IM_HIP_CHECK(hipGetLastError());
    return IM_OK;
  }
  const size_t u_words = B == 8 ? im::Stair<8>{pad}.words() : im::Stair<16>{pad}.words();
  const size_t lds_bytes = sizeof(float) * (u_words + pad + B * B + B);
  if (lds_bytes > 160 * 1024) return IM_ERR_UNSUPPORTED;
  auto fn = B == 8 ? im::blocked_factor_solve_kernel<8> : im::blocked_factor_solve_kernel<16>;
  if (lds_bytes > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  // The pivots of a tile, the triangular solves and the right-hand side are one wavefront's work
  // whatever the workgroup size, and the other wavefronts wait at the barriers meanwhile: what
  // counts is how many worlds are resident on a CU.  Small workgroups leave the registers for more
  // of them (measured on g1, snu and the 128-dof stress shape: 64 threads up to pad 48, 128 for
  // 16 x 16 tiles at pad 64, 256 beyond; at pad 128 four workgroups of 38 KB share a CU and the
  // launch takes 1.30 ms for 16384 worlds where two of 512 threads took 1.90).
  const int threads = pad <= 48 ? 64 : (pad <= 64 && B == 16) ? 128 : 256;
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(threads), lds_bytes, (hipStream_t)stream, M, ldM, nM, block_idx, y,
                     ldy, U, x, ldx, nv, pad, active);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

static int check_blocked_shape(int block_size, int nv, int pad) {
  if (nv <= 0 || pad < nv) return IM_ERR_ARG;
  if (block_size != 8 && block_size != 16) return IM_ERR_UNSUPPORTED;
  if (pad % block_size || pad - nv >= block_size) return IM_ERR_ARG;
  return IM_OK;
}

static int launch_multi_solve(const float *U, int block_size, int nv, int pad, const float *y, int nrhs,
                              const int32_t *active, float *x, int nworld, void *stream) {
  const size_t lds_bytes = sizeof(float) * ((size_t)pad * (pad + 1) / 2 + (size_t)pad * nrhs);
  if (lds_bytes > 160 * 1024) return IM_ERR_UNSUPPORTED;
  auto fn = block_size == 8 ? im::blocked_multi_solve_kernel<8> : im::blocked_multi_solve_kernel<16>;
  if (lds_bytes > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(64), lds_bytes, (hipStream_t)stream, U, y, active, x, nv, pad, nrhs);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_blocked_factor_solve(const float *M, int64_t ldM, int nM, const int32_t *block_idx, int block_size,
                            int nv, int pad, const float *y, int64_t ldy, float *U, float *x, int64_t ldx,
                            int nworld, void *stream) {
  if (nworld < 0) return IM_ERR_ARG;
  if (const int st = check_blocked_shape(block_size, nv, pad)) return st;
  if (nworld == 0) return IM_OK;
  if (!M || !block_idx || !y || !x) return IM_ERR_ARG;
  if (ldy < nv || ldx < nv) return IM_ERR_STRIDE;
  if (U && ((uintptr_t)U & 15)) return IM_ERR_STRIDE;  // written 16 bytes at a time
  return launch_blocked_factor(M, ldM, nM, block_idx, block_size, nv, pad, y, ldy, U, x, ldx, nullptr, nworld, stream);
}

int im_blocked_multi_solve(const float *U, int block_size, int nv, int pad, const float *y, int rhs_count,
                           const int32_t *active, float *x, int nworld, void *stream) {
  if (nworld < 0 || rhs_count <= 0) return IM_ERR_ARG;
  if (const int st = check_blocked_shape(block_size, nv, pad)) return st;
  if (nworld == 0) return IM_OK;
  if (!U || !y || !x) return IM_ERR_ARG;
  return launch_multi_solve(U, block_size, nv, pad, y, rhs_count, active, x, nworld, stream);
}

int im_blocked_factor_multi_solve(const float *M, int64_t ldM, int nM, const int32_t *block_idx, int block_size,
                                  int nv, int pad, const float *y, int rhs_count, const int32_t *active, float *U,
                                  float *x, int nworld, void *stream) {
  if (nworld < 0 || rhs_count <= 0) return IM_ERR_ARG;
  if (const int st = check_blocked_shape(block_size, nv, pad)) return st;
  if (nworld == 0) return IM_OK;
  if (!M || !block_idx || !y || !x || !U) return IM_ERR_ARG;
  if ((uintptr_t)U & 15) return IM_ERR_STRIDE;
  const int st = launch_blocked_factor(M, ldM, nM, block_idx, block_size, nv, pad, nullptr, 0, U, nullptr, 0, active,
                                       nworld, stream);
  if (st != IM_OK) return st;
  return launch_multi_solve(U, block_size, nv, pad, y, rhs_count, active, x, nworld, stream);
}

int im_blocked_factor_multi_solve_static(const float *M, int64_t ldM, int nM, const int32_t *block_idx,
                                         int block_size, int nv, int pad, const float *y, int rhs_count,
                                         const int32_t *active, float *x, int nworld, void *stream) {
  if (nworld < 0 || rhs_count <= 0) return IM_ERR_ARG;
  if (const int st = check_blocked_shape(block_size, nv, pad)) return st;
  if ((uint64_t)nworld * pad * pad * sizeof(float) > IM_STATIC_SCRATCH_BYTES) return IM_ERR_SCRATCH;
  if (nworld == 0) return IM_OK;
  if (!M || !block_idx || !y || !x) return IM_ERR_ARG;
  float *U = nullptr;
  if (const int st = static_scratch(&U)) return st;
  // every active world's (pad, pad) slice is written whole by the factor kernel before the
  // solve reads it, and the solve skips the inactive ones: nothing has to start at zero
  const int st = launch_blocked_factor(M, ldM, nM, block_idx, block_size, nv, pad, nullptr, 0, U, nullptr, 0, active,
                                       nworld, stream);
  if (st != IM_OK) return st;
  return launch_multi_solve(U, block_size, nv, pad, y, rhs_count, active, x, nworld, stream);
}

int im_blocked_index_layout(const int32_t *elemid, int nv, int nM, int block_size, int32_t *layout,
                            float *identity) {
  if (!elemid || !layout || nv <= 0 || nM < 0 || block_size <= 0) return IM_ERR_ARG;
  const int B = block_size, nblk = (nv + B - 1) / B;
  int32_t *out = layout;
  for (int kb = 0; kb < nblk; ++kb)
    for (int ib = 0; ib < nblk; ++ib)
      for (int r = 0; r < B; ++r)
        for (int c = 0; c < B; ++c) {
          const int row = kb * B + r, col = ib * B + c;
          *out++ = (row < nv && col < nv) ? elemid[(size_t)row * nv + col] : nM;  // nM: out of range, reads as zero
        }
  if (identity)
    for (int r = 0; r < B; ++r)
      for (int c = 0; c < B; ++c) identity[r * B + c] = (r == c && (nblk - 1) * B + r >= nv) ? 1.0f : 0.0f;
  return IM_OK;
}

int im_copy_dense_factor(const float *U, int pad, const int32_t *block_adr, int nv, float *L_out, int64_t ld_out,
                         int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || pad < nv) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!U || !block_adr || !L_out) return IM_ERR_ARG;
  if (ld_out < (int64_t)nv * nv) return IM_ERR_STRIDE;
  hipLaunchKernelGGL(im::copy_dense_factor_kernel, dim3((unsigned)((nv * nv + 255) / 256), (unsigned)nworld), dim3(256),
                     0, (hipStream_t)stream, U, pad, block_adr, nv, L_out, ld_out);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_jtdj_mfma(const float *Mdense, const float *J, int njmax, const float *D, const int32_t *state,
                 const int32_t *nefc, int quad, float *H, int nv, int nv_pad, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv_pad < nv || njmax <= 0) return IM_ERR_ARG;  // rows are clamped to njmax - 1
  if (nworld == 0) return IM_OK;
  if (!Mdense || !J || !D || !state || !H) return IM_ERR_ARG;
  if (nv > 128) return IM_ERR_UNSUPPORTED;
  const int nvr = (nv + 31) / 32 * 32;
  // two copies of the staged rows, the list of contributing rows with their weights
  const size_t lds_bytes = sizeof(float) * (2 * (32 * (size_t)nvr + 32) + 2 * (size_t)((njmax + 3) & ~3));
  if (lds_bytes > 160 * 1024) return IM_ERR_UNSUPPORTED;
  auto fn = nv > 112 ? im::jtdj_mfma_kernel<128> : im::jtdj_mfma_kernel<0>;
  if (lds_bytes > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(256), lds_bytes, (hipStream_t)stream, Mdense, J, njmax, D, state, nefc,
                     quad, H, nv, nv_pad);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_jtdj_factor_solve(const float *Mdense, const float *J, int njmax, const float *D, const int32_t *state,
                         const int32_t *nefc, int quad, float *H, int nv, int nv_pad, const float *y, int64_t ldy,
                         float *U, int pad, float *x, int64_t ldx, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || njmax <= 0 || (H && nv_pad < nv)) return IM_ERR_ARG;
  if (check_blocked_shape(16, nv, pad) != IM_OK) return check_blocked_shape(16, nv, pad);
  if (nworld == 0) return IM_OK;
  if (!Mdense || !J || !D || !state || (x && !y)) return IM_ERR_ARG;
  if (nv > 128) return IM_ERR_UNSUPPORTED;
  if ((y && ldy < nv) || (x && ldx < nv)) return IM_ERR_STRIDE;
  if (U && ((uintptr_t)U & 15)) return IM_ERR_STRIDE;
  const int nvr = (nv + 31) / 32 * 32;
  const size_t stage_words = 2 * (32 * (size_t)nvr + 32) + 2 * (size_t)((njmax + 3) & ~3), u_words = im::Stair<16>{pad}.words();
  const size_t lds_bytes = sizeof(float) * ((u_words > stage_words ? u_words : stage_words) + pad + 16 * 16 + 16);
  if (lds_bytes > 160 * 1024) return IM_ERR_UNSUPPORTED;
  auto fn = nv > 112 ? im::jtdj_factor_solve_kernel<128> : im::jtdj_factor_solve_kernel<0>;
  if (lds_bytes > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(256), lds_bytes, (hipStream_t)stream, Mdense, J, njmax, D, state, nefc, quad,
                     H, nv, nv_pad, y, ldy, U, x, ldx, pad);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_dense_update_factor(const uint8_t *done, const int32_t *state_changes, const int32_t *changes,
                           const int32_t *ids, int ld_ids, const float *J, int njmax, const float *D,
                           const int32_t *state, int quad, const float *grad, int64_t ldg, float *H, float *U,
                           int nv, int nv_pad, int32_t *dof_union, float *search, int64_t ld_search,
                           float *search_dot, float *decrement, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv_pad <= nv || ld_ids < 0 || njmax <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!state_changes || !changes || !ids || !J || !D || !state || !grad || !H || !U || !dof_union || !search ||
      !search_dot || !decrement)
    return IM_ERR_ARG;
  if (nv_pad % 16) return IM_ERR_ARG;
  if (ldg < nv || ld_search < nv) return IM_ERR_STRIDE;
  if (nv <= 32)  // no factor is kept for such a matrix: one tile, factored at every call
    return im_dense_update_tile(done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, H, nv,
                                nv_pad, dof_union, search, ld_search, search_dot, decrement, nworld, stream);
  // up to 64 columns: a wavefront per world with a lane per column (IMHIP_DENSE_STAGE=blocked keeps
  // the workgroup-per-world kernel below, which serves the larger matrices)
  static const bool column_off = [] {
    const char *e = std::getenv("IMHIP_DENSE_STAGE");
    return e && std::strcmp(e, "blocked") == 0;
  }();
  if (!column_off && (nv_pad == 48 || nv_pad == 64))
    return im_dense_update_column(done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg, H, U,
                                  nv, nv_pad, dof_union, search, ld_search, search_dot, decrement, nworld, stream);
  if (((uintptr_t)H | (uintptr_t)U) & 15) return IM_ERR_STRIDE;  // read and written 16 bytes at a time
  constexpr int B = 16;
  const int pf = (nv + B - 1) / B * B;  // the factor in LDS covers the dofs; the kernel writes the identity beyond them itself
  const size_t base_bytes =
      sizeof(float) * ((size_t)im::Stair<B>{pf}.words() + pf + B * B + B + 2 * (size_t)nv + 1);
  if (base_bytes > 160 * 1024) return IM_ERR_UNSUPPORTED;
  // a batch of changed rows uses the factor's array: up to 64 rows, a multiple of four
  int row_cap = (int)(im::Stair<B>{pf}.words() / (size_t)nv) & ~3;
  row_cap = row_cap < 64 ? row_cap : 64;
  const size_t lds_bytes = base_bytes + sizeof(float) * 128;  // the batch's weights and row numbers behind the tables
  auto fn = im::dense_update_factor_kernel<B>;
  if (lds_bytes > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  hipLaunchKernelGGL(fn, dim3(nworld), dim3(256), lds_bytes, (hipStream_t)stream, done, state_changes, changes,
                     ids, ld_ids, J, njmax, D, state, quad, grad, ldg, H, U, dof_union, search, ld_search,
                     search_dot, decrement, nv, nv_pad, row_cap);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_check_pivot_sqrt(uint32_t first_bits, uint32_t last_bits, unsigned long long *mismatches, void *stream) {
  if (!mismatches || last_bits < first_bits) return IM_ERR_ARG;
  hipLaunchKernelGGL(im::check_pivot_sqrt_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, first_bits, last_bits,
                     mismatches);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
