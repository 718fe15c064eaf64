// The dense Newton factor stage above 32 dofs on one wavefront per world, a lane per column of
// the padded matrix (nv_pad = 48 or 64): the incremental update of H's upper triangle over the
// changed rows' dof union, the augmented blocked Cholesky U'U = H (16 x 16 blocks, the gradient as
// the last column) or, without changed rows, the solve with the stored factor, the backward
// solve, search = -x and the two sums.
// Reference: src/instantmimic/utils/mjw_kernels/newton_stages.py:614-742 (stage), :473-611
// (augmented blocked factor), :451-470 and :651-701 (update over the dof union).
//
// Lane c keeps column c of the upper triangle in registers, u[r] = U[r][c].  A block row's
// elements first lose the earlier block rows' sums (for every element a sum of 16 fused
// multiply-adds started from zero per earlier block row, then one subtraction: the blocked order),
// the factor of the other column arriving inside the multiply-add (the block row's columns copied
// into every row of sixteen lanes, then a DPP row broadcast); inside the block row every lane --
// diagonal block, blocks to its right, gradient column alike -- runs
//   u[k + r] = (u[k + r] - sum_{q < r} U[k + q][k + r] * u[k + q]) / U[k + r][k + r]
// with column k + r's elements broadcast the same way, which is the diagonal tile's Cholesky and the
// triangular solves of the tiles to its right in one.  The backward solve needs rows of U across
// lanes: a 16 x 16 tile at a time is turned round through LDS.  The gradient column rides in lane
// 63 (a padding column that no other lane reads).
// The first factor of a solve has a launch of its own in which the wavefront assembles H first
// (dense_init_column_kernel; newton_fusion.py:470 of the reference calls upstream's assembly there).
// Same operations in the same order as the workgroup-per-world kernel of blocked_kernels.hip and
// the CPU restatement both are tested against.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "common.h"
#include "jtdj_wave.h"
#include "newton_wave.h"
#include "pivot.h"

namespace im {
namespace {

using resident::wave_sync;

constexpr int kColStagedRows = 32;  // the changed rows a stage keeps in LDS (a 32-bit mask per dof); beyond, up to 128 rows, their masks only
// LDS words of one world's stage: a 16 x 16 tile turned round (rows 17 words apart), the staged
// changed rows dof-major (33 words a dof), their weights, the dofs' masks
template <int NBLK>
__host__ __device__ constexpr int column_stage_words() {
  return 16 * 17 + (kColStagedRows + 1) * 16 * NBLK + kColStagedRows + 16 * NBLK;
}

// acc[r] = fma(value of lane r of the caller's row of sixteen lanes of `other`, own, acc[r]), r = 0 .. 15:
// the broadcast rides in the multiply-add (DPP).  The leading wait covers a register written just
// before: a DPP read needs two idle cycles after a vector write of its source, which the compiler
// does not see inside the block.
__device__ __forceinline__ void row_fmac16(float (&acc)[16], float other, float own) {
#define IM_ROW_FMAC(n) "v_fmac_f32_dpp %" #n ", %16, %17 row_newbcast:" #n " row_mask:0xf bank_mask:0xf\n\t"
  asm("s_nop 1\n\t" IM_ROW_FMAC(0) IM_ROW_FMAC(1) IM_ROW_FMAC(2) IM_ROW_FMAC(3) IM_ROW_FMAC(4) IM_ROW_FMAC(5) IM_ROW_FMAC(6)
          IM_ROW_FMAC(7) IM_ROW_FMAC(8) IM_ROW_FMAC(9) IM_ROW_FMAC(10) IM_ROW_FMAC(11) IM_ROW_FMAC(12) IM_ROW_FMAC(13)
              IM_ROW_FMAC(14) IM_ROW_FMAC(15)
      : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7]),
        "+v"(acc[8]), "+v"(acc[9]), "+v"(acc[10]), "+v"(acc[11]), "+v"(acc[12]), "+v"(acc[13]), "+v"(acc[14]), "+v"(acc[15])
      : "v"(other), "v"(own));
#undef IM_ROW_FMAC
}
// v = fma(value of lane r of the row of minus_row[q], own[q], v) for q = 0 .. r - 1 in order (r a
// constant after unrolling): the statements keep their order among themselves, the first one waits
__device__ __forceinline__ void row_chain(float &v, const float (&minus_row)[16], const float *own, int r) {
  asm volatile("s_nop 1");
#pragma unroll
  for (int q = 0; q < 15; ++q)
    if (q < r)
      asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(v) : "v"(minus_row[q]), "v"(own[q]), "n"(r));
}

__device__ __forceinline__ float lane_value(float v, int lane) {  // `lane` the same for the whole wavefront
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// changes_raw: the world's count of changed rows as the stage receives it (negative: factor H as it
// lies there; zero: solve with the stored factor).
template <int NBLK>
__device__ __forceinline__ void dense_column_world(float *scr, float *Hw, float *Uw, const float *Jw, const float *Dw,
                                                   const float *gw, const int32_t *sw, const int32_t *idw,
                                                   int changes_raw, int ld_ids, int quad, int32_t *uni, float *search_w,
                                                   float *search_dot_w, float *decrement_w, int nv, int lane) {
  constexpr int PAD = 16 * NBLK, RHS = 63;  // RHS: the lane of the gradient column
  float *tt = scr;                                   // [16][17]
  float *jr = tt + 16 * 17;                          // [PAD][kColStagedRows + 1]
  float *sd = jr + (kColStagedRows + 1) * PAD;       // [kColStagedRows]
  unsigned *mkl = (unsigned *)(sd + kColStagedRows);  // [PAD]
  const bool refactor = changes_raw != 0;
  const int count = changes_raw < 0 ? 0 : (changes_raw < ld_ids ? changes_raw : ld_ids);
  const float g = lane < nv ? gw[lane] : 0.0f;
  float u[PAD];
  float rdiag = 1.0f;  // 1 / U[c][c] of this lane's column
  float x = 0.0f;      // this lane's entry of the right-hand side / solution
  if (refactor) {
    // ---- the changed rows, the dof union
    const bool staged = count <= kColStagedRows;
    const bool masked = !staged && count <= 128 && 2 * count + 4 * nv <= (kColStagedRows + 1) * PAD;
    unsigned mk = 0u;
    bool hit = false;
    if (staged && count > 0) {
      const int tq = lane < count ? lane : count - 1;
      const int rq = idw[tq];
      const float dq = Dw[rq];
      const int sq = sw[rq];
      if (lane < kColStagedRows) sd[lane] = sq == quad ? dq : -dq;
      // sixteen rows at a time: their elements of this lane's dof asked for together
#pragma unroll
      for (int half = 0; half < kColStagedRows / 16; ++half) {
        if (16 * half >= count) break;  // the same for every lane
        float rowv[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          const int r = __builtin_amdgcn_readlane(rq, 16 * half + t);  // (lanes at or past count hold row count - 1)
          rowv[t] = Jw[(size_t)r * nv + (lane < nv ? lane : nv - 1)];
        }
        if (lane < nv) {
#pragma unroll
          for (int t = 0; t < 16; ++t) {
            if (16 * half + t < count) {
              jr[lane * (kColStagedRows + 1) + 16 * half + t] = rowv[t];
              mk |= (unsigned)(rowv[t] != 0.0f) << (16 * half + t);
            }
          }
        }
      }
      if (lane < nv) {
        mkl[lane] = mk;
        hit = mk != 0u;
      }
    } else if (masked) {
      // more rows than the staged capacity: their numbers, their weights and a mask of up to 128 rows per
      // dof go where the staged rows would lie; J's elements then come from memory, but only those of
      // the rows that a pair's two dofs share
      int *rid = (int *)jr;                          // [count]
      float *sdv = jr + count;                       // [count]
      unsigned *mk4 = (unsigned *)(jr + 2 * count);  // [nv][4]
      for (int t = lane; t < count; t += 64) {
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
          if (t0 >= count) break;  // the same for every lane
          float rowv[16];
#pragma unroll
          for (int t = 0; t < 16; ++t)
            rowv[t] = Jw[(size_t)idw[t0 + t < count ? t0 + t : count - 1] * nv + (lane < nv ? lane : nv - 1)];
#pragma unroll
          for (int t = 0; t < 16; ++t)
            if (t0 + t < count) mw |= (unsigned)(rowv[t] != 0.0f) << (16 * half + t);
        }
        if (lane < nv) mk4[4 * lane + word] = mw;
        any |= mw;
      }
      hit = lane < nv && any != 0u;
    } else if (lane < nv) {
      for (int t = 0; t < count && !hit; ++t) hit = Jw[(size_t)idw[t] * nv + lane] != 0.0f;
    }
    const unsigned long long umask = __ballot(hit);
    if (hit) uni[__popcll(umask & ((1ull << lane) - 1ull))] = lane;
    if (lane == 0) uni[nv] = __popcll(umask);
    if (!staged) {
      // the update in memory, a union row at a time, ahead of the column's load: lane c adds to the
      // elements of column c that it reads back itself
      wave_sync();
      for (unsigned long long rest = umask; rest; rest &= rest - 1ull) {
        const int r = __builtin_ctzll(rest);  // the same for every lane
        if (!(hit && lane >= r)) continue;
        float delta = 0.0f;
        if (masked) {
          const int *rid = (const int *)jr;
          const float *sdv = jr + count;
          const unsigned *mk4 = (const unsigned *)(jr + 2 * count);
          for (int word = 0; 32 * word < count; ++word) {
            for (unsigned mm = mk4[4 * r + word] & mk4[4 * lane + word]; mm; mm &= mm - 1u) {
              const int t = 32 * word + __builtin_ctz(mm);
              const int rr = rid[t];
              delta = fma_(sdv[t] * Jw[(size_t)rr * nv + r], Jw[(size_t)rr * nv + lane], delta);
            }
          }
        } else {
          for (int t = 0; t < count; ++t) {
            const int rr = idw[t];
            const float av = Jw[(size_t)rr * nv + r], bv = Jw[(size_t)rr * nv + lane];
            float da = Dw[rr] * av;
            if (sw[rr] != quad) da = -da;
            if (av != 0.0f && bv != 0.0f) delta = fma_(da, bv, delta);
          }
        }
        if (delta != 0.0f) Hw[(size_t)r * PAD + lane] = Hw[(size_t)r * PAD + lane] + delta;
      }
    }
    // ---- H's column: the upper triangle up to nv, the identity beyond; lane RHS takes the gradient
#pragma unroll
    for (int r = 0; r < PAD; ++r) {
      const bool rhs_lane = lane == RHS;
      const bool mine = rhs_lane ? r < nv : (r <= lane && lane < nv);
      const float *src = rhs_lane ? gw + (r < nv ? r : 0) : Hw + (size_t)r * PAD + (lane < PAD ? lane : 0);
      const float v = *src;
      u[r] = mine ? v : ((r == lane && !rhs_lane) ? 1.0f : 0.0f);
    }
    wave_sync();
    // ---- update over the pairs (row <= column) of the union from the staged rows, a union row at a time: lane c owns pair (r, c)
#pragma unroll
    for (int r = 0; r < PAD; ++r) {
      if (!staged || !((umask >> r) & 1ull)) continue;  // the same for every lane
      float delta = 0.0f;
      {
        const unsigned mk_r = (unsigned)__builtin_amdgcn_readlane((int)mk, r);
        const float *jrow = jr + r * (kColStagedRows + 1), *jcol = jr + (lane < PAD ? lane : 0) * (kColStagedRows + 1);
        for (unsigned mm = (hit && lane >= r) ? (mk_r & mk) : 0u; mm; mm &= mm - 1u) {
          const int t = __builtin_ctz(mm);
          delta = fma_(sd[t] * jrow[t], jcol[t], delta);
        }
      }
      if (delta != 0.0f) {
        u[r] = u[r] + delta;
        Hw[(size_t)r * PAD + lane] = u[r];
      }
    }
    // ---- augmented blocked factor, a block row at a time
#pragma unroll
    for (int kb = 0; kb < NBLK; ++kb) {
      const int k = 16 * kb;
      // lane L's copy of a register of lane k + (L & 15): the block row's sixteen columns side by side in
      // every row of sixteen lanes, from where one lane's value reaches its row inside the multiply-add
      // (a DPP row broadcast; the copy comes through the LDS crossbar)
      const int from_block = 4 * (k + (lane & 15));
#pragma unroll
      for (int jb = 0; jb < kb; ++jb) {
        const int j = 16 * jb;
        float sum[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) sum[r] = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          const float other = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from_block, __builtin_bit_cast(int, u[j + t])));
          row_fmac16(sum, other, u[j + t]);  // sum[r] = fma(U[j + t][k + r], u[j + t], sum[r])
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) u[k + r] = u[k + r] - sum[r];
      }
      float minus_row[16];  // minus_row[q]: minus the block copy of row k + q, once that row is final
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        if (k + r == RHS) continue;  // (a matrix of 64 columns: its last one is padding, and lane 63 holds the gradient)
        float v = u[k + r];
        row_chain(v, minus_row, &u[k], r);  // v = fma(-U[k + q][k + r], u[k + q], v) for q < r, in order
        // the pivot is lane k + r's value
        float d, inv;
        pivot_sqrt_rcp(lane_value(v, k + r), true, d, inv);
        u[k + r] = lane == k + r ? d : v * inv;
        if (lane == k + r) rdiag = inv;
        if (r < 15) {
          minus_row[r] = -__builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from_block, __builtin_bit_cast(int, u[k + r])));
          // in its register here, ahead of the next step's wait: the negation is a vector write that
          // the DPP reads of the steps to come must not follow too closely
          asm volatile("" : "+v"(minus_row[r]));
        }
      }
    }
    // ---- the corner of the augmented column, the factor out
    float corner = 1.0e30f;
#pragma unroll
    for (int i = 0; i < PAD; ++i)
      if (i < nv) corner = fma_(-u[i], u[i], corner);  // lane RHS's column is the forward-solved gradient
    corner = sqrtf(corner);
    const int out_col = lane == RHS ? PAD - 1 : lane;
    const bool out = lane == RHS || lane < PAD - 1;
#pragma unroll
    for (int r = 0; r < PAD; ++r) {
      float v = r <= lane ? u[r] : 0.0f;
      if (lane == RHS) v = r < nv ? u[r] : (r == PAD - 1 ? corner : 0.0f);
      if (out) Uw[(size_t)r * PAD + out_col] = v;
    }
    // the forward-solved gradient, an entry per lane
#pragma unroll
    for (int r = 0; r < PAD; ++r) {
      const float z = lane_value(u[r], RHS);
      x = (lane == r && r < nv) ? z : x;
    }
    if (lane == RHS) {  // from here on column RHS is the identity's (as is column PAD - 1)
#pragma unroll
      for (int r = 0; r < PAD; ++r) u[r] = r == RHS ? 1.0f : 0.0f;
      rdiag = 1.0f;
    }
  } else {
    // ---- the stored factor with the identity in place of its augmented column; forward solve
    float dg = 1.0f;
#pragma unroll
    for (int r = 0; r < PAD; ++r) {
      const float v = Uw[(size_t)r * PAD + (lane < PAD ? lane : 0)];
      u[r] = (lane < PAD - 1 && r <= lane) ? v : (r == lane ? 1.0f : 0.0f);
      dg = r == lane ? u[r] : dg;
    }
    rdiag = 1.0f / dg;
    x = g;
#pragma unroll
    for (int kb = 0; kb < NBLK; ++kb) {
      const int k = 16 * kb;
      const bool here = lane >= k && lane < k + 16;
#pragma unroll
      for (int jb = 0; jb < kb; ++jb) {
        const int j = 16 * jb;
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; ++t) sum = fma_(u[j + t], lane_value(x, j + t), sum);
        x = here ? x - sum : x;
      }
#pragma unroll
      for (int jj = 0; jj < 16; ++jj) {
        const float z = lane_value(x * rdiag, k + jj);
        x = lane == k + jj ? z : ((here && lane > k + jj) ? fma_(-u[k + jj], z, x) : x);
      }
    }
  }
  // ---- backward solve U x = z, block rows from the last; rows of U come across lanes through LDS
#pragma unroll
  for (int ib = NBLK - 1; ib >= 0; --ib) {
    const int i0 = 16 * ib;
    const bool here = lane >= i0 && lane < i0 + 16;
#pragma unroll
    for (int jb = ib + 1; jb < NBLK; ++jb) {
      const int j = 16 * jb;
      if (lane >= j && lane < j + 16) {
#pragma unroll
        for (int r = 0; r < 16; ++r) tt[(lane - j) * 17 + r] = u[i0 + r];  // tt[t][r] = U[i0 + r][j + t]
      }
      wave_sync();
      float sum = 0.0f;
      const int rr = here ? lane - i0 : 0;
#pragma unroll
      for (int t = 0; t < 16; ++t) sum = fma_(tt[t * 17 + rr], lane_value(x, j + t), sum);
      x = here ? x - sum : x;
      wave_sync();
    }
    if (here) {
#pragma unroll
      for (int r = 0; r < 16; ++r) tt[(lane - i0) * 17 + r] = u[i0 + r];  // tt[c][r] = U[i0 + r][i0 + c]
    }
    wave_sync();
#pragma unroll
    for (int r = 15; r >= 0; --r) {
      const float xv = lane_value(x * rdiag, i0 + r);
      const int tl = here ? lane - i0 : 0;
      const float urc = tt[r * 17 + tl];  // U[i0 + tl][i0 + r]
      x = lane == i0 + r ? xv : ((here && lane < i0 + r) ? fma_(-urc, xv, x) : x);
    }
    wave_sync();
  }
  // ---- search = -x, x . x and grad . x as 64 lanes striding the dofs sum them
  const float xs = lane < nv ? x : 0.0f;
  if (lane < nv) search_w[lane] = -xs;
  float s0 = fma_(xs, xs, 0.0f), s1 = fma_(g, xs, 0.0f);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s0 = s0 + __shfl_down(s0, off, 64);
    s1 = s1 + __shfl_down(s1, off, 64);
  }
  if (lane == 0) {
    *search_dot_w = s0;
    *decrement_w = s1;
  }
}

// A wavefront per world, four worlds per workgroup.
template <int NBLK>
__global__ __launch_bounds__(256) void dense_update_column_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ state_changes, const int32_t *__restrict__ changes,
    const int32_t *__restrict__ ids, int ld_ids, const float *__restrict__ J, int njmax, const float *__restrict__ D,
    const int32_t *__restrict__ state, int quad, const float *__restrict__ grad, int64_t ldg, float *H_, float *U_,
    int32_t *__restrict__ uni_, float *__restrict__ search, int64_t ld_search, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int nworld) {
  extern __shared__ float lds[];
  constexpr int PAD = 16 * NBLK;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t w = (int64_t)blockIdx.x * 4 + wv;
  if (w >= nworld) return;
  if ((done && done[w]) || state_changes[w] == 0) return;
  dense_column_world<NBLK>(lds + wv * column_stage_words<NBLK>(), H_ + w * (int64_t)PAD * PAD, U_ + w * (int64_t)PAD * PAD,
                           J + w * (int64_t)njmax * nv, D + w * njmax, grad + w * ldg, state + w * njmax, ids + w * ld_ids,
                           changes[w], ld_ids, quad, uni_ + w * (nv + 1), search + w * ld_search, search_dot + w,
                           decrement + w, nv, lane);
}

// The first Hessian and its factor in one launch: H = M + J' D_act J of every world on the matrix
// cores of its wavefront (jtdj_wave.h), stored, then the stage above on H as it lies there for the
// worlds that are not done.
template <int NBLK>
__global__ __launch_bounds__(256, NBLK == 3 ? 3 : 2) void dense_init_column_kernel(
    const uint8_t *__restrict__ done, const int32_t *__restrict__ nefc_p, const float *__restrict__ J, int njmax,
    const float *__restrict__ D, const int32_t *__restrict__ state, int quad, const float *__restrict__ M, int64_t ldM,
    const int32_t *__restrict__ elemid, const float *__restrict__ grad, int64_t ldg, float *H_, float *U_,
    int32_t *__restrict__ uni_, float *__restrict__ search, int64_t ld_search, float *__restrict__ search_dot,
    float *__restrict__ decrement, int nv, int nworld) {
  extern __shared__ float lds[];
  constexpr int PAD = 16 * NBLK;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t w = (int64_t)blockIdx.x * 4 + wv;
  if (w >= nworld) return;
  int nefc = nefc_p ? nefc_p[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  float *Hw = H_ + w * (int64_t)PAD * PAD;
  const float *Jw = J + w * (int64_t)njmax * nv;
  jtdj_wave<NBLK>(M + w * ldM, elemid, Jw, D + w * njmax, state + w * njmax, nefc, quad, nv, Hw, PAD, true, lane);
  if (done && done[w]) return;
  // the lanes read back one another's stores (one CU: its vector cache sees them once they are issued and waited for)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  dense_column_world<NBLK>(lds + wv * column_stage_words<NBLK>(), Hw, U_ + w * (int64_t)PAD * PAD, Jw, D + w * njmax,
                           grad + w * ldg, state + w * njmax, nullptr, -1, 0, quad, uni_ + w * (nv + 1),
                           search + w * ld_search, search_dot + w, decrement + w, nv, lane);
}

// The resident Newton loop (newton_wave.h) with this stage: a wavefront per world from the first
// line search to convergence, WAVES worlds per workgroup.  Per wavefront in LDS: what the loop
// keeps from round to round and one area that the staged tile of J, the gradient's row list and
// the stage use one after the other.
template <int NBLK>
__host__ __device__ inline int column_resident_area_words(int nv, int njmax) {
  int words = column_stage_words<NBLK>();
  const int tile = 64 * 17, grad = 2 * njmax + nv;
  words = words > tile ? words : tile;
  words = words > grad ? words : grad;
  return (words + 3) & ~3;
}
__host__ __device__ inline int column_resident_shared_words(int nterm, int nv) { return (nterm + nv + 1 + 3) & ~3; }

template <int NBLK, int WAVES, int HELD>
__global__ __launch_bounds__(64 * WAVES, NBLK == 3 ? 3 : 2) void newton_dense_column_resident_kernel(
    resident::NewtonArgs a, float *__restrict__ H_, float *__restrict__ U_, int32_t *__restrict__ uni_,
    int *__restrict__ next_world) {
  extern __shared__ float lds[];
  constexpr int PAD = 16 * NBLK;
  const int tid = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nv = a.nv, njmax = a.njmax, nworld = a.nworld;
  uint32_t *term = (uint32_t *)lds;
  int *radr = (int *)(term + a.nterm);
  const int area = column_resident_area_words<NBLK>(nv, njmax);
  float *mine = lds + column_resident_shared_words(a.nterm, nv) + wv * (area + resident::kept_words(nv, njmax, 0));
  resident::LoopLds L;
  L.votes = nullptr;
  L.worlds = nullptr;
  L.term = term, L.radr = radr;
  L.rows = mine;  // the shared area: tile of J, then the gradient's lists, then the stage
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
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));  // (nothing formed from it is kept in registers from round to round)
    dense_column_world<NBLK>(mine, H_ + w * (int64_t)PAD * PAD, U_ + w * (int64_t)PAD * PAD,
                             b.J + w * (int64_t)b.njmax * b.nv, b.D + w * b.njmax, b.grad + w * b.ld_grad,
                             b.state + w * b.njmax, b.ids + w * (int64_t)b.ld_ids, b.quad_count[w], b.ld_ids, b.quad,
                             uni_ + w * (b.nv + 1), b.search + w * b.nv, b.search_dot + w, b.decrement + w, b.nv, lane);
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

__global__ void set_column_counter_kernel(int *counter, int value) { *counter = value; }

struct ColumnVariant {
  int nblk, waves, held;
  const void *fn;
};

}  // namespace
}  // namespace im

extern "C" int im_newton_solve_dense_column(const im_newton_args *p, float *H, float *U, int32_t *dof_union, int nv,
                                            int nv_pad, int nM, int32_t *next_world, void *stream) {
  if (!p || !H || !U || !dof_union || !next_world || p->nworld < 0 || nv <= 0 || nv_pad <= nv || nM <= 0) return IM_ERR_ARG;
  if (nv <= 32 || (nv_pad != 48 && nv_pad != 64)) return IM_ERR_UNSUPPORTED;
  if (p->nworld == 0) return IM_OK;
  im::resident::NewtonArgs a{};
  const int bad = im::resident::convert_args(*p, nv, nM, a);
  if (bad != IM_OK) return bad;
  const int njmax = p->njmax;
#define IM_COLUMN_VARIANT(NBLK, WAVES, HELD) \
  {NBLK, WAVES, HELD, (const void *)im::newton_dense_column_resident_kernel<NBLK, WAVES, HELD>}
  // 48 or 64 columns; four or eight worlds per workgroup (a lane holds a whole column: up to 256 registers);
  // the line search keeps a lane's two rows in registers up to 64 rows and reads them from LDS beyond
  // (four first: at about 150 registers a lane a CU holds twelve wavefronts, three such workgroups or one of eight)
  static const im::ColumnVariant variants[] = {IM_COLUMN_VARIANT(3, 4, 2), IM_COLUMN_VARIANT(3, 8, 2), IM_COLUMN_VARIANT(3, 4, 0),
                                               IM_COLUMN_VARIANT(3, 8, 0), IM_COLUMN_VARIANT(4, 4, 2), IM_COLUMN_VARIANT(4, 8, 2),
                                               IM_COLUMN_VARIANT(4, 4, 0), IM_COLUMN_VARIANT(4, 8, 0)};
#undef IM_COLUMN_VARIANT
  constexpr int kVariants = 8;
  static bool usable[kVariants] = {};
  static int regs[kVariants] = {};
  static bool probed = false;
  if (!probed) {  // once per process: a variant that spills registers is left out; the large dynamic LDS is asked for
    for (int i = 0; i < kVariants; ++i) {
      hipFuncAttributes fa{};
      // (a variant that parks more than a register or two of its prologue in memory is left out)
      usable[i] = hipFuncGetAttributes(&fa, variants[i].fn) == hipSuccess && fa.localSizeBytes <= 16 &&
                  hipFuncSetAttribute(variants[i].fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      160 * 1024 - (int)fa.sharedSizeBytes) == hipSuccess;
      regs[i] = fa.numRegs;
      (void)hipGetLastError();
    }
    probed = true;
  }
  const int nblk = nv_pad / 16;
  for (int i = 0; i < kVariants; ++i) {
    const im::ColumnVariant &v = variants[i];
    if (!usable[i] || v.nblk != nblk || v.held != (njmax <= 64 ? 2 : 0)) continue;
    const int area = nblk == 3 ? im::column_resident_area_words<3>(nv, njmax) : im::column_resident_area_words<4>(nv, njmax);
    const size_t per_wave = (size_t)area + im::resident::kept_words(nv, njmax, 0);
    const size_t lds = 4 * ((size_t)im::column_resident_shared_words(p->nterm, nv) + v.waves * per_wave);
    if (lds > 158 * 1024) continue;
    static int ncu = 0;
    if (!ncu) {
      int dev = 0;
      IM_HIP_CHECK(hipGetDevice(&dev));
      IM_HIP_CHECK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
    }
    // as many workgroups as stay resident at once: by LDS and by registers
    int per_cu = 0;
    IM_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, v.fn, 64 * v.waves, lds));
    per_cu = std::max(1, per_cu);
    const int needed = (p->nworld + v.waves - 1) / v.waves;
    const int grid = std::min(needed, std::max(ncu, 1) * per_cu);
    hipLaunchKernelGGL(im::set_column_counter_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, next_world, grid * v.waves);
    void *args[] = {&a, &H, &U, &dof_union, &next_world};
    IM_HIP_CHECK(hipLaunchKernel(v.fn, dim3((unsigned)grid), dim3(64 * v.waves), args, lds, (hipStream_t)stream));
    return IM_OK;
  }
  return IM_ERR_UNSUPPORTED;
}

extern "C" int im_dense_update_column(const uint8_t *done, const int32_t *state_changes, const int32_t *changes,
                                      const int32_t *ids, int ld_ids, const float *J, int njmax, const float *D,
                                      const int32_t *state, int quad, const float *grad, int64_t ldg, float *H, float *U,
                                      int nv, int nv_pad, int32_t *dof_union, float *search, int64_t ld_search,
                                      float *search_dot, float *decrement, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv_pad <= nv || ld_ids < 0 || njmax <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!state_changes || !changes || !ids || !J || !D || !state || !grad || !H || !U || !dof_union || !search ||
      !search_dot || !decrement)
    return IM_ERR_ARG;
  if (ldg < nv || ld_search < nv) return IM_ERR_STRIDE;
  if (nv_pad != 48 && nv_pad != 64) return IM_ERR_UNSUPPORTED;
  const unsigned grid = (unsigned)((nworld + 3) / 4);
  if (nv_pad == 48) {
    hipLaunchKernelGGL(im::dense_update_column_kernel<3>, dim3(grid), dim3(256), 16 * im::column_stage_words<3>(),
                       (hipStream_t)stream, done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg,
                       H, U, dof_union, search, ld_search, search_dot, decrement, nv, nworld);
  } else {
    hipLaunchKernelGGL(im::dense_update_column_kernel<4>, dim3(grid), dim3(256), 16 * im::column_stage_words<4>(),
                       (hipStream_t)stream, done, state_changes, changes, ids, ld_ids, J, njmax, D, state, quad, grad, ldg,
                       H, U, dof_union, search, ld_search, search_dot, decrement, nv, nworld);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_dense_init_tile(const uint8_t *done, const int32_t *nefc, const float *J, int njmax, const float *D,
                                  const int32_t *state, int quad, const float *M, int64_t ldM, const int32_t *elemid,
                                  const float *grad, int64_t ldg, float *H, int nv, int nv_pad, int32_t *dof_union,
                                  float *search, int64_t ld_search, float *search_dot, float *decrement, int nworld,
                                  void *stream);

extern "C" int im_dense_init_factor(const uint8_t *done, const int32_t *nefc, const float *J, int njmax, const float *D,
                                    const int32_t *state, int quad, const float *M, int64_t ldM, const int32_t *elemid,
                                    const float *grad, int64_t ldg, float *H, float *U, int nv, int nv_pad,
                                    int32_t *dof_union, float *search, int64_t ld_search, float *search_dot,
                                    float *decrement, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || nv_pad < nv || njmax <= 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!J || !D || !state || !M || !elemid || !grad || !H || !dof_union || !search || !search_dot || !decrement)
    return IM_ERR_ARG;
  if (ldg < nv || ld_search < nv || ((uintptr_t)H & 15) != 0 || (nv_pad & 3) != 0) return IM_ERR_STRIDE;
  if (nv <= 32)
    return im_dense_init_tile(done, nefc, J, njmax, D, state, quad, M, ldM, elemid, grad, ldg, H, nv, nv_pad, dof_union,
                              search, ld_search, search_dot, decrement, nworld, stream);
  if (!U) return IM_ERR_ARG;
  if (nv_pad <= nv || (nv_pad != 48 && nv_pad != 64)) return IM_ERR_UNSUPPORTED;
  const unsigned grid = (unsigned)((nworld + 3) / 4);
  if (nv_pad == 48) {
    hipLaunchKernelGGL(im::dense_init_column_kernel<3>, dim3(grid), dim3(256), 16 * im::column_stage_words<3>(),
                       (hipStream_t)stream, done, nefc, J, njmax, D, state, quad, M, ldM, elemid, grad, ldg, H, U, dof_union,
                       search, ld_search, search_dot, decrement, nv, nworld);
  } else {
    hipLaunchKernelGGL(im::dense_init_column_kernel<4>, dim3(grid), dim3(256), 16 * im::column_stage_words<4>(),
                       (hipStream_t)stream, done, nefc, J, njmax, D, state, quad, M, ldM, elemid, grad, ldg, H, U, dof_union,
                       search, ld_search, search_dot, decrement, nv, nworld);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
