// The resident Newton loop: one wavefront per world from the first line search to convergence,
// four worlds per workgroup, as the reference keeps a world in one block for the whole loop
// (src/instantmimic/utils/mjw_kernels/newton_fusion.py:57-298).  Per iteration and world, in the
// reference kernel's order (:170-296): M search, J search, the scalar line search with the step
// and the constraints' new forces and states (newton_stages.py:79-444), the gradient (:745-798),
// the factor stage, the convergence test.  Every stage performs the operations of the per-stage
// kernels of this library in their order, so a solve gives the same bits whichever way it runs.
//
// The factor stage is handed in by the kernel that includes this file (a generated kernel for the
// model's tree: four wavefronts work on the workgroup's four worlds together), which is why the
// loop keeps the four wavefronts in step at two workgroup barriers per iteration; a world that is
// done idles through them until the workgroup's last world finishes.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/imhip.h"
#include "newton_search.h"

namespace im {
namespace resident {

struct NewtonArgs {
  // options (arrays indexed by world modulo their length)
  const float *tolerance, *ls_tolerance, *meaninertia;
  int ntolerance, nls_tolerance, nmeaninertia;
  int nv, njmax, nworld, ls_iterations, maxiter, block, quad, ls_overflow_bit, iter_overflow_bit;
  // row tables of M v: nv + 1 offsets, then per term the column and the element of M
  const int32_t *mulm_rowadr, *mulm_col, *mulm_madr;
  int nterm, nM;
  // the step's inputs
  const int32_t *ne, *nf, *nefc;
  const float *M;
  int64_t ldM;
  const float *J, *D, *frictionloss, *smooth;  // J (nworld, njmax, nv); D, frictionloss (nworld, njmax); smooth (nworld, nv)
  // solver state, rows of nv or njmax floats per world unless a stride is given
  float *qacc, *Ma, *force, *Jaref, *search, *search_dot, *mv, *jv, *alpha, *improvement, *grad, *grad_dot,
      *grad_scale, *decrement, *qfrc_constraint;
  int64_t ld_grad;
  int32_t *state, *ids, *quad_count, *state_count, *niter, *overflow, *nsolving;
  int ld_ids;
  uint8_t *done, *exhausted, *unchanged;
  int stage_lds_floats;  // dynamic LDS the factor stage uses from offset 0; the loop's own arrays follow
  // cooperative loop: a counter in memory, set to four times the grid's workgroups before the launch,
  // from which a wavefront whose world is done takes the next world nobody has started (null: a
  // workgroup keeps to its own four worlds)
  int *next_world;
  // cooperative loop: whether a wavefront keeps its world's row of M in LDS (1) or reads it from
  // memory in the round's one product with it (0: the LDS saved admits another workgroup per CU)
  int m_lds;
};

// The public argument block checked and turned into the kernels' (host side).
inline int convert_args(const im_newton_args &p, int nv, int nM, NewtonArgs &a) {
  const int njmax = p.njmax;
  if (njmax <= 0 || p.iterations < 0 || p.ls_iterations < 0 || (p.block != 32 && p.block != 64) || p.ntolerance <= 0 ||
      p.nls_tolerance <= 0 || p.nmeaninertia <= 0 || p.nterm <= 0)
    return IM_ERR_ARG;
  if (!p.opt_tolerance || !p.opt_ls_tolerance || !p.stat_meaninertia || !p.M_mulm_rowadr || !p.M_mulm_col ||
      !p.M_mulm_madr || !p.M || !p.efc_J || !p.efc_D || !p.qfrc_smooth || !p.qacc || !p.efc_Ma || !p.efc_force ||
      !p.efc_state || !p.Jaref || !p.search || !p.search_dot || !p.mv || !p.jv || !p.alpha || !p.improvement || !p.grad ||
      !p.grad_dot || !p.grad_scale || !p.newton_decrement || !p.qfrc_constraint || !p.quad_changed_ids ||
      !p.quad_changed_count || !p.state_changed_count || !p.solver_niter || !p.done || !p.ls_exhausted ||
      !p.search_unchanged || (p.nf && !p.efc_frictionloss))
    return IM_ERR_ARG;
  if (p.ldM < nM || p.ld_grad < nv || p.ld_ids < 0) return IM_ERR_STRIDE;
  if (p.nterm >= 65536 || nM >= 65536 || 64 * (int64_t)nv >= (1 << 20)) return IM_ERR_UNSUPPORTED;
  a.tolerance = p.opt_tolerance, a.ls_tolerance = p.opt_ls_tolerance, a.meaninertia = p.stat_meaninertia;
  a.ntolerance = p.ntolerance, a.nls_tolerance = p.nls_tolerance, a.nmeaninertia = p.nmeaninertia;
  a.nv = nv, a.njmax = njmax, a.nworld = p.nworld, a.ls_iterations = p.ls_iterations, a.maxiter = p.iterations;
  a.block = p.block, a.quad = p.quad, a.ls_overflow_bit = p.ls_overflow_bit;
  a.iter_overflow_bit = p.iterations_overflow_bit;
  a.mulm_rowadr = p.M_mulm_rowadr, a.mulm_col = p.M_mulm_col, a.mulm_madr = p.M_mulm_madr;
  a.nterm = p.nterm, a.nM = nM;
  a.ne = p.ne, a.nf = p.nf, a.nefc = p.nefc, a.M = p.M, a.ldM = p.ldM, a.J = p.efc_J, a.D = p.efc_D;
  a.frictionloss = p.efc_frictionloss, a.smooth = p.qfrc_smooth;
  a.qacc = p.qacc, a.Ma = p.efc_Ma, a.force = p.efc_force, a.Jaref = p.Jaref, a.search = p.search;
  a.search_dot = p.search_dot, a.mv = p.mv, a.jv = p.jv, a.alpha = p.alpha, a.improvement = p.improvement;
  a.grad = p.grad, a.grad_dot = p.grad_dot, a.grad_scale = p.grad_scale, a.decrement = p.newton_decrement;
  a.qfrc_constraint = p.qfrc_constraint, a.ld_grad = p.ld_grad;
  a.state = p.efc_state, a.ids = p.quad_changed_ids, a.quad_count = p.quad_changed_count;
  a.state_count = p.state_changed_count, a.niter = p.solver_niter, a.overflow = p.overflow, a.nsolving = p.nsolving;
  a.ld_ids = p.ld_ids, a.done = p.done, a.exhausted = p.ls_exhausted, a.unchanged = p.search_unchanged;
  a.stage_lds_floats = 0;
  a.next_world = nullptr;
  a.m_lds = 1;
  return IM_OK;
}

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
// a value every lane holds alike, as a scalar (so that it occupies no vector register while it waits)
__device__ __forceinline__ float uniform(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// orders this wavefront's writes (LDS and memory) before its later reads: the stages hand their
// results on through memory, written by some lanes and read by others
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void block_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// words of LDS of the loop's own arrays behind the factor stage's area: four flags, the row tables of M v
// (one word per term, nv + 1 offsets), then per wavefront the world's row of M, the search
// direction, Ma, mv, Jaref, jv, D and the friction losses, the gradient's list of rows with a force
// (value and row number) and its copy of the gradient.  The factor stage's area must also hold four wavefronts'
// staged tiles of J: 4 x 64 rows x 16 dofs, a row 17 words.
// words a wavefront keeps from round to round: M, the search direction, Ma, mv, qacc; Jaref, jv, D, friction losses
__host__ __device__ inline size_t kept_words(int nv, int njmax, int nM) { return (size_t)nM + 4 * (size_t)nv + 4 * (size_t)njmax; }
__host__ __device__ inline size_t loop_lds_words(int nv, int njmax, int nM, int nterm) {
  return 8 + (size_t)nterm + nv + 1 + 4 * (kept_words(nv, njmax, nM) + 2 * (size_t)njmax + nv);
}
__host__ __device__ inline size_t staged_rows_words(int) { return 4 * 64 * 17; }  // four wavefronts' tiles of J

// ---- M search (newton_fusion.py:171-176): lane d owns dofs d, d + 64 --------------------------
__device__ __forceinline__ void mul_m_world(const NewtonArgs &a, const uint32_t *term, const int *radr, const float *m,
                                            const float *v, float *out, float *out_lds, int lane) {
  for (int dof = lane; dof < a.nv; dof += 64) {
    float value = 0.0f;
    const int end = radr[dof + 1];
    for (int k = radr[dof]; k < end; k += 4) {  // four terms' operands at a time, a term past the end dropped
      float x[4], y[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t t = term[k + u < end ? k + u : end - 1];
        x[u] = m[t >> 16];
        y[u] = v[t & 0xffffu];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) value = k + u < end ? fma_(x[u], y[u], value) : value;
    }
    out[dof] = value;
    out_lds[dof] = value;
  }
}

// ---- J search (newton_stages.py:157-178): 64 rows at a time through LDS, a lane per row --------
template <int U>
__device__ __forceinline__ void jv_world(const NewtonArgs &a, const float *Jw, int nefc, float *rows_lds,
                                         const float *sv, float *jv, float *jv_lds, int lane) {
  const int nv = a.nv, stride = nv | 1;
  const float inv_nv = 1.0f / (float)nv;
  for (int r0 = 0; r0 < nefc; r0 += 64) {
    const int rows = nefc - r0 < 64 ? nefc - r0 : 64;
    const float *src = Jw + (int64_t)r0 * nv;
    const int total = rows * nv;
    for (int i0 = lane; i0 < total; i0 += U * 64) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = src[i0 + 64 * u < total ? i0 + 64 * u : total - 1];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + 64 * u;
        if (i < total) {
          const int r = (int)(((float)i + 0.5f) * inv_nv);  // i / nv, exact while i stays below 2^20
          rows_lds[r * stride + (i - r * nv)] = v[u];
        }
      }
    }
    wave_sync();
    if (lane < rows) {
      const float *row = rows_lds + lane * stride;
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
          for (int u = 0; u < 8; ++u) p = fma_(x[u], y[u], p);
        }
        for (; i < i1; ++i) p = fma_(row[i], sv[i], p);
        return p;
      };
      float acc = 0.0f;
      if (nv > 50) {
        for (int start = 0; start < nv; start += 20) acc = acc + chain(start, start + 20 < nv ? start + 20 : nv);
      } else {
        acc = chain(0, nv);
      }
      jv[r0 + lane] = acc;
      jv_lds[r0 + lane] = acc;
    }
    wave_sync();  // the rows are read before the next 64 overwrite them
  }
}

// ---- the gradient (newton_stages.py:745-798), a lane per dof ------------------------------------
// The world's scalars that the loop carries in registers (every lane the same values); they are
// written to memory as they change.
struct Scalars {
  float search_dot, grad_dot, decrement, grad_scale, alpha, improvement;
  int niter;
};
// For a world whose states changed: qfrc_constraint = J' force over the listed rows (`cnt` rows with
// a nonzero force, ascending, in f / rowl), grad = Ma - qfrc_smooth - qfrc_constraint, grad . grad.
// Otherwise the rescaling of the three scalars.  Returns whether the search direction stays.
// AHEAD: the next rows' elements are asked for before the current ones are added (ROWS more
// registers a lane).
template <bool AHEAD>
__device__ __forceinline__ bool gradient_world(const NewtonArgs &a, int64_t w, const float *Jw, bool changed, int cnt,
                                               const float *f, const int *rowl, const float *Ma_l, float *gl, Scalars &sc,
                                               int lane) {
  if (!changed) {
    const float sigma = sc.grad_scale, new_sigma = sigma - sc.alpha;
    float ratio = 0.0f;
    if (sigma != 0.0f) ratio = new_sigma / sigma;
    const float ratio_sq = ratio * ratio;
    sc.grad_dot = uniform(sc.grad_dot * ratio_sq);
    sc.decrement = uniform(sc.decrement * ratio_sq);
    sc.grad_scale = uniform(new_sigma);
    if (lane == 0) {
      a.grad_dot[w] = sc.grad_dot;
      a.decrement[w] = sc.decrement;
      a.grad_scale[w] = sc.grad_scale;
      a.unchanged[w] = 1;
    }
    return true;
  }
  const int nv = a.nv;
#ifndef IM_GRADIENT_ROWS
#define IM_GRADIENT_ROWS 16
#endif
  constexpr int ROWS = IM_GRADIENT_ROWS;
  for (int dof = lane; dof < nv; dof += 64) {
    const float ma = Ma_l[dof], sm = a.smooth[w * nv + dof];
    float sum = 0.0f;
    // the next ROWS rows' elements are asked for before the current ones are added
    float jv[ROWS], jn[ROWS];
    auto fetch = [&](int p0, float (&v)[ROWS]) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < ROWS; ++u) v[u] = Jw[(int64_t)rowl[p0 + u < cnt ? p0 + u : cnt - 1] * nv + dof];
    };
    if (AHEAD && cnt > 0) fetch(0, jv);
    for (int p0 = 0; p0 < cnt; p0 += ROWS) {
      if (!AHEAD) fetch(p0, jv);
      if (AHEAD && p0 + ROWS < cnt) fetch(p0 + ROWS, jn);
#pragma unroll
      for (int u = 0; u < ROWS; ++u) sum = p0 + u < cnt ? fma_(jv[u], f[p0 + u], sum) : sum;
      if (AHEAD) {
#pragma unroll
        for (int u = 0; u < ROWS; ++u) jv[u] = jn[u];
      }
    }
    const float g = ma - sm - sum;
    a.qfrc_constraint[w * nv + dof] = sum;
    a.grad[w * a.ld_grad + dof] = g;
    gl[dof] = g;
  }
  wave_sync();
  // grad . grad as a block of `block` lanes sums it: lane `rank` its dofs rank, rank + block, ..,
  // 32 lanes in a shuffle-down tree, the trees in order
  float p = 0.0f;
  if (lane < a.block)
    for (int dof = lane; dof < nv; dof += a.block) p = fma_(gl[dof], gl[dof], p);
  for (int off = 16; off > 0; off >>= 1) p = p + __shfl_down(p, off, 32);
  float total = 0.0f + __shfl(p, 0, 64);
  if (a.block > 32) total = total + __shfl(p, 32, 64);
  sc.grad_dot = uniform(total);
  sc.decrement = 0.0f;
  sc.grad_scale = 1.0f;
  if (lane == 0) {
    a.grad_dot[w] = total;
    a.decrement[w] = 0.0f;
    a.grad_scale[w] = 1.0f;
    a.unchanged[w] = 0;
  }
  return false;
}

// ---- search . search and grad . x of a factor stage that leaves only the search direction -----
__device__ __forceinline__ void search_sums_world(const NewtonArgs &a, int64_t w, const float *gl, Scalars &sc, int lane) {
  float s0 = 0.0f, s1 = 0.0f;
  for (int d = lane; d < a.nv && lane < a.block; d += a.block) {
    const float v = -a.search[w * a.nv + d];
    s0 = fma_(v, v, s0);
    s1 = fma_(gl[d], v, s1);
  }
  for (int o = 16; o > 0; o >>= 1) {
    s0 = s0 + __shfl_down(s0, o, 32);
    s1 = s1 + __shfl_down(s1, o, 32);
  }
  const float a1 = __shfl(s0, 32, 64), b1 = __shfl(s1, 32, 64);
  float ra = 0.0f + __shfl(s0, 0, 64), rb = 0.0f + __shfl(s1, 0, 64);
  if (a.block > 32) ra = ra + a1, rb = rb + b1;
  sc.search_dot = uniform(ra);
  sc.decrement = uniform(rb);
  if (lane == 0) {
    a.search_dot[w] = ra;
    a.decrement[w] = rb;
  }
}

// ---- J search through a tile of 64 rows x 16 dofs (4.3 KB of LDS whatever the width of J) ------
// The same chain per row as jv_world: the dofs in order, the 20-dof partial sums of the reference's
// rule beyond 50 dofs.  A lane loads 16 elements per tile, four rows of 64 bytes per instruction.
// AHEAD: the next tile's elements are asked for while the current one is worked on (sixteen more
// registers a lane).  WIDE: a tile row's operands are read eight at a time ahead of their part of
// the chain (sixteen more again).
template <bool AHEAD, bool WIDE>
__device__ __forceinline__ void jv_world_tiled(const NewtonArgs &a, const float *Jw, int nefc, float *tile,
                                               const float *sv, float *jv, float *jv_lds, int lane) {
  const int nv = a.nv;
  const int c = lane & 15, rq = lane >> 4;
  const bool split = nv > 50;
  // the 16 elements of a lane for the tile at (r0, c0); the next tile's are asked for while the
  // current one is worked on, so the trips to memory of all but the first tile are hidden
  auto fetch = [&](int r0, int c0, float (&v)[16]) __attribute__((always_inline)) {
    const int rows = nefc - r0 < 64 ? nefc - r0 : 64, cw = nv - c0 < 16 ? nv - c0 : 16;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int r = rq + 4 * k;
      v[k] = Jw[(int64_t)(r0 + (r < rows ? r : rows - 1)) * nv + c0 + (c < cw ? c : cw - 1)];
    }
  };
  float v[16];
  if (AHEAD && nefc > 0) fetch(0, 0, v);
  for (int r0 = 0; r0 < nefc; r0 += 64) {
    const int rows = nefc - r0 < 64 ? nefc - r0 : 64;
    float acc = 0.0f, p = 0.0f;
    for (int c0 = 0; c0 < nv; c0 += 16) {
      const int cw = nv - c0 < 16 ? nv - c0 : 16;
      if (!AHEAD) fetch(r0, c0, v);
#pragma unroll
      for (int k = 0; k < 16; ++k) tile[(rq + 4 * k) * 17 + c] = v[k];
      wave_sync();
      const bool more_columns = c0 + 16 < nv;
      const int next_r0 = more_columns ? r0 : r0 + 64, next_c0 = more_columns ? c0 + 16 : 0;
      if (AHEAD && next_r0 < nefc) fetch(next_r0, next_c0, v);
      if (lane < rows) {
        // a tile row's operands are read eight at a time before their part of the chain (two waits
        // per tile, not sixteen)
        const float *row = tile + lane * 17;
        if constexpr (!WIDE) {  // the short form, for a kernel without registers to spare
          for (int i = 0; i < cw; ++i) {
            if (split && (c0 + i) % 20 == 0 && c0 + i > 0) {
              acc = acc + p;
              p = 0.0f;
            }
            p = fma_(row[i], sv[c0 + i], p);
          }
        } else
#pragma unroll
        for (int h = 0; h < 16; h += 8) {
          float x[8], y[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            x[i] = row[h + i];
            y[i] = sv[c0 + (h + i < cw ? h + i : 0)];
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            if (h + i < cw) {  // the same for every lane
              if (split && (c0 + h + i) % 20 == 0 && c0 + h + i > 0) {
                acc = acc + p;
                p = 0.0f;
              }
              p = fma_(x[i], y[i], p);
            }
          }
        }
      }
      wave_sync();  // the tile is read before the next one overwrites it
    }
    if (lane < rows) {
      const float out = split ? acc + p : p;
      if (jv) jv[r0 + lane] = out;
      jv_lds[r0 + lane] = out;
    }
  }
}

// ---- the loop ------------------------------------------------------------------------------------
// Where the loop's arrays lie in LDS (set up by the kernel around it).
struct LoopLds {
  int *votes;            // [4] cooperative stage only
  int *worlds;           // [4] cooperative stage only: the world of each wavefront (nworld: none), read by the stage
  const uint32_t *term;  // [nterm] col | madr << 16, shared by the workgroup
  const int *radr;       // [nv + 1]
  // per wavefront, kept from round to round:
  float *m_lds;          // [nM] the world's row of M
  float *sv;             // [nv] the search direction
  float *Ma, *mv, *qacc; // [nv] each
  float *Jaref, *jv;     // [njmax] each
  float *D, *fl;         // [njmax] each: the rows' weights and friction losses (read at every step of the line search)
  // per wavefront, used within a round (may share one area with the factor stage's own arrays):
  float *f;              // [njmax] forces of the listed rows
  int *rowl;             // [njmax] their numbers
  float *gl;             // [nv] the gradient (a cooperative stage's loop reads it again after the stage)
  float *rows;           // staged rows of J: 64 x (nv | 1), or the 64 x 17 tile
};

// A world's vectors stay in LDS and its scalars in registers from round to round; memory receives
// every value as it is produced (the arrays end as after the stage launches) and is read again only
// for what another wavefront or the factor stage has written there.
// HELD: rows of a world a lane keeps in registers during the line search (0: read from LDS at every
// evaluation); JU: loads in flight per lane while rows of J are staged, 0 for the tiled staging
// with the next tile asked for ahead and a tile row's operands read eight at a time, -2 with the
// first of the two only, -1 with neither (each costs sixteen registers a lane).
// COOP: `stage()` works on the workgroup's four worlds together (every wavefront calls it in step,
// between two workgroup barriers; it takes the worlds' numbers from L.worlds and skips the worlds
// whose `unchanged` byte is set).  A wavefront whose world is done takes the next world from the
// counter a.next_world (or, without one, idles through the barriers); the workgroup leaves when all
// four are idle.  Otherwise
// `stage()` is the wavefront's own world's stage (it leaves search_dot and newton_decrement in
// memory itself), called only when that world needs it, and a wavefront leaves as soon as its world
// is done.  `w_raw`: the wavefront's world.
//
// `kernarg_offset`: where the kernel's NewtonArgs parameter lies in its kernel-argument segment.  The
// loop reads the arguments from there, through a pointer it launders once per round: about sixty
// pointers cannot stay in scalar registers across the stages (held, they are spilled to vector
// lanes and read back one by one), and from the segment each is one scalar load next to its use.
typedef const NewtonArgs __attribute__((address_space(4))) KernelNewtonArgs;
__device__ __forceinline__ const NewtonArgs &kernel_args(int kernarg_offset) {
  const char __attribute__((address_space(4))) *seg =
      (const char __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr();
  KernelNewtonArgs *ap = (KernelNewtonArgs *)(seg + kernarg_offset);
  asm volatile("" : "+s"(ap));
  return *(const NewtonArgs *)ap;
}

// MLDS: the world's row of M is kept in LDS (where L.m_lds is not null); otherwise `M search` reads it from memory
// every round, which leaves the LDS to more worlds per CU.
template <int HELD, int JU, bool COOP, bool MLDS = true, class Stage>
__device__ __forceinline__ void newton_loop(int kernarg_offset, const LoopLds &L, int64_t w_raw, Stage &&stage) {
  const NewtonArgs &a0 = kernel_args(kernarg_offset);
  const NewtonArgs &a = a0;
  const int lane_fixed = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int nv = a.nv, njmax = a.njmax;
  // what belongs to the wavefront's current world
  int64_t w = 0;
  bool live = false, done = true, unchanged = false;
  int nefc = 0, ne = 0, nf = 0, budget = 0;
  const float *Jw = a.J;
  float tolerance = 0.0f, ls_tolerance = 0.0f, meaninertia = 1.0f;
  Scalars sc{};
  auto enter = [&](int64_t w_raw) __attribute__((always_inline)) {
    const NewtonArgs &a = kernel_args(kernarg_offset);
    // the world's number as a scalar: every address below is a scalar base plus a lane offset
    const int w_lo = __builtin_amdgcn_readfirstlane((int)(w_raw & 0xffffffff)), w_hi = __builtin_amdgcn_readfirstlane((int)(w_raw >> 32));
    const int64_t w_uniform = ((int64_t)w_hi << 32) | (uint32_t)w_lo;
    live = w_uniform < a.nworld;
    w = live ? w_uniform : (int64_t)a.nworld - 1;
    done = !live || a.done[w] != 0;
    if (live && done && lane_fixed == 0) a.unchanged[w] = 1;  // the factor stage leaves such a world alone
    unchanged = !done && a.unchanged[w] != 0;
    nefc = a.nefc ? a.nefc[w] : njmax;
    nefc = __builtin_amdgcn_readfirstlane(nefc < njmax ? nefc : njmax);
    ne = __builtin_amdgcn_readfirstlane(a.ne ? a.ne[w] : 0), nf = __builtin_amdgcn_readfirstlane(a.nf ? a.nf[w] : 0);
    Jw = a.J + w * (int64_t)njmax * nv;
    tolerance = a.tolerance[w % a.ntolerance], ls_tolerance = a.ls_tolerance[w % a.nls_tolerance];
    meaninertia = a.meaninertia[w % a.nmeaninertia];
    sc = Scalars{uniform(a.search_dot[w]), uniform(a.grad_dot[w]), uniform(a.decrement[w]), uniform(a.grad_scale[w]),
                 uniform(a.alpha[w]), uniform(a.improvement[w]), __builtin_amdgcn_readfirstlane(a.niter[w])};
    budget = a.maxiter;  // rounds this wavefront gives the world, whatever the data
    if (done) return;
    // what the loop keeps: M, Ma, Jaref into LDS (mv and jv are formed before they are read: a world
    // enters with a new search direction unless it is done) and qacc
    if constexpr (MLDS)
      if (L.m_lds)
        for (int k = lane_fixed; k < a.nM; k += 64) L.m_lds[k] = a.M[w * a.ldM + k];
    for (int k = lane_fixed; k < nv; k += 64) {
      L.Ma[k] = a.Ma[w * nv + k];
      L.mv[k] = a.mv[w * nv + k];
      L.qacc[k] = a.qacc[w * nv + k];
    }
    for (int r = lane_fixed; r < njmax; r += 64) {
      L.Jaref[r] = a.Jaref[w * njmax + r];
      L.jv[r] = a.jv[w * njmax + r];
      L.D[r] = a.D[w * njmax + r];
      L.fl[r] = a.frictionloss ? a.frictionloss[w * njmax + r] : 0.0f;
    }
    wave_sync();
  };
  enter(w_raw);
  bool queue_empty = !(COOP && a0.next_world);
#ifdef IM_NEWTON_STAMPS  // development aid: time per phase, summed over the rounds, left in the world's row of jv
  long long t_phase[8] = {0, 0, 0, 0, 0, 0, 0, 0}, t_last = wall_clock64();
#define IM_STAMP(k) do { const long long t_now = wall_clock64(); t_phase[k] += t_now - t_last; t_last = t_now; } while (0)
#else
#define IM_STAMP(k) do {} while (0)
#endif
  // Every world gets at most maxiter rounds of its wavefront, whatever the data, and the counter of
  // worlds only grows: every wavefront leaves the loop.
  for (;;) {
    const NewtonArgs &a = kernel_args(kernarg_offset);  // read afresh in every round
    if (COOP) {
      // a wavefront without a world to work on takes the next one nobody has started; the other
      // wavefronts' worlds go on with their own rounds beside it (the stage does not care which
      // iteration a world is in)
      while (done && !queue_empty) {
        int next = 0;
        if (lane_fixed == 0) next = atomicAdd(a.next_world, 1);
        next = __builtin_amdgcn_readfirstlane(next);
        if (next < a.nworld)
          enter(next);
        else
          queue_empty = true;
      }
      if (lane_fixed == 0) {
        L.votes[wv] = done ? 0 : 1;
        L.worlds[wv] = done ? a.nworld : (int)w;
      }
      block_sync();
      if (!(L.votes[0] | L.votes[1] | L.votes[2] | L.votes[3])) break;  // the workgroup's four worlds are done
    } else if (done) {
      break;
    }
    // the lane number as a value the compiler cannot see through, new in every round: nothing a
    // stage derives from it is kept in registers across the other stages
    int lane = lane_fixed;
    asm volatile("" : "+v"(lane));
    IM_STAMP(0);
    if (!done) {
      if (!unchanged) {
        for (int k = lane; k < nv; k += 64) L.sv[k] = a.search[w * nv + k];
        wave_sync();
        mul_m_world(a, L.term, L.radr, (MLDS && L.m_lds) ? (const float *)L.m_lds : a.M + w * a.ldM, L.sv, a.mv + w * nv, L.mv, lane);
        if constexpr (JU > 0)
          jv_world<(JU > 0 ? JU : 1)>(a, Jw, nefc, L.rows, L.sv, a.jv + w * njmax, L.jv, lane);
        else
          jv_world_tiled<(JU == 0 || JU == -2), (JU == 0)>(a, Jw, nefc, L.rows, L.sv, a.jv + w * njmax, L.jv, lane);
        wave_sync();
      }
      IM_STAMP(1);
      // (the force list and the row list of the gradient are free until the step is taken)
      const search::LsWorld lw{a.smooth + w * nv, L.D, L.fl, L.Jaref, L.sv, L.mv, L.jv, L.Ma, sc.search_dot, tolerance,
                               ls_tolerance, meaninertia, ne, nf, nefc, nv, a.ls_iterations, L.f, (float *)L.rowl};
      const search::LsResult ls = search::linesearch_rows<HELD, true>(lw, lane & 31);  // both halves on this world
      sc.alpha = uniform(ls.alpha), sc.improvement = uniform(ls.improvement);
      if (lane == 0) {
        a.alpha[w] = ls.alpha;
        a.improvement[w] = ls.improvement;
        a.exhausted[w] = ls.exhausted ? 1 : 0;
        if (!ls.converged && a.overflow) a.overflow[w] = a.overflow[w] | a.ls_overflow_bit;
      }
      IM_STAMP(2);
      // the step (newton_stages.py:373-381), then force and state of every row from the new Jaref, the
      // rows whose being quadratic flipped (ascending) and the two counts (:385-444); the rows with a
      // force are listed for the gradient as they are formed
      const float al = ls.alpha;
      for (int i = lane; i < nv; i += 64) {
        const float q = fma_(al, L.sv[i], L.qacc[i]), v = fma_(al, L.mv[i], L.Ma[i]);
        L.qacc[i] = q;
        L.Ma[i] = v;
        a.qacc[w * nv + i] = q;
        a.Ma[w * nv + i] = v;
      }
      int nquad = 0, nstate = 0, cnt = 0;
      for (int base = 0; base < nefc; base += 64) {
        const int r = base + lane;
        bool quad_flip = false, changed = false;
        float f = 0.0f;
        if (r < nefc) {
          const float x = L.Jaref[r] + al * L.jv[r], d = L.D[r];
          L.Jaref[r] = x;
          a.Jaref[w * njmax + r] = x;
          f = -d * x;
          int st = 1;
          if (r >= ne && r < ne + nf) {
            const float fr = L.fl[r], rf = search::safe_div(fr, d);
            if (x <= -rf) f = fr, st = 2;
            else if (x >= rf) f = -fr, st = 3;
          } else if (r >= ne && x >= 0.0f) {
            f = 0.0f, st = 0;
          }
          const int old = a.state[w * njmax + r];
          a.force[w * njmax + r] = f;
          a.state[w * njmax + r] = st;
          quad_flip = (old == 1) != (st == 1);
          changed = old != st;
        }
        const unsigned long long below = (1ull << lane) - 1ull;
        const unsigned long long m = __ballot(quad_flip);
        if (quad_flip) {
          const int slot = nquad + __popcll(m & below);
          if (slot < a.ld_ids) a.ids[w * (int64_t)a.ld_ids + slot] = r;
        }
        nquad += __popcll(m);
        nstate += __popcll(__ballot(changed));
        const unsigned long long mf = __ballot(f != 0.0f);
        if (f != 0.0f) {
          const int pos = cnt + __popcll(mf & below);
          L.f[pos] = f;
          L.rowl[pos] = r;
        }
        cnt += __popcll(mf);
      }
      nstate += ls.exhausted ? 1 : 0;
      if (lane == 0) {
        a.quad_count[w] = nquad;
        a.state_count[w] = nstate;
      }
      wave_sync();
      IM_STAMP(3);
      unchanged = gradient_world<(JU == 0 || JU == -2)>(a, w, Jw, nstate != 0, cnt, L.f, L.rowl, L.Ma, L.gl, sc, lane);
      IM_STAMP(4);
    }
    if (COOP) {
      block_sync();  // gradients, states and the `unchanged` bytes of the four worlds are in place; the rows of J are done with
      IM_STAMP(5);
      stage();
      block_sync();  // the four search directions are complete
    } else {
      wave_sync();
      if (!done && !unchanged) stage();
      wave_sync();
    }
    IM_STAMP(6);
    lane = lane_fixed;
    asm volatile("" : "+v"(lane));  // no address from before the stage is kept through it
    if (!done) {
      const NewtonArgs &a = kernel_args(kernarg_offset);
      if (!unchanged) {
        if (COOP) {
          search_sums_world(a, w, L.gl, sc, lane);
        } else {  // the stage has left the two sums in memory
          sc.search_dot = uniform(a.search_dot[w]);
          sc.decrement = uniform(a.decrement[w]);
        }
      }
      // newton_fusion.py:265-296
      sc.niter += 1;
      const float scale = meaninertia * (float)nv;
      const bool converged = sc.alpha == 0.0f || (sc.improvement > 0.0f && sc.improvement / scale < tolerance) ||
                             sqrtf(sc.grad_dot) / scale < tolerance || 0.5f * sc.decrement / scale < tolerance;
      const bool finished = converged || sc.niter == a.maxiter;
      if (lane == 0) {
        a.niter[w] = sc.niter;
        if (finished) {
          if (!converged && a.overflow) a.overflow[w] = a.overflow[w] | a.iter_overflow_bit;
          a.done[w] = 1;
          a.unchanged[w] = 1;
          if (a.nsolving) atomicAdd(a.nsolving, -1);
        }
      }
      budget -= 1;
      done = finished || budget <= 0;
    }
    IM_STAMP(7);
  }
#ifdef IM_NEWTON_STAMPS
  if (live && lane_fixed < 8) a0.jv[w * njmax + lane_fixed] = (float)t_phase[lane_fixed];
#endif
#undef IM_STAMP
}

// The layout behind a cooperative stage's area of `a.stage_lds_floats` words (the staged rows of J
// use that area between two stages): four flags, the row tables of M v, then each of the four
// wavefronts' own arrays.  Fills the tables; the caller synchronises the workgroup before the loop.
__device__ __forceinline__ LoopLds coop_layout(const NewtonArgs &a, float *lds) {
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int nv = a.nv, njmax = a.njmax, nM = a.m_lds ? a.nM : 0;
  LoopLds L;
  L.votes = (int *)(lds + a.stage_lds_floats);
  L.worlds = L.votes + 4;
  uint32_t *term = (uint32_t *)(L.worlds + 4);
  int *radr = (int *)(term + a.nterm);
  float *mine = (float *)(radr + nv + 1) + wv * (kept_words(nv, njmax, nM) + 2 * njmax + nv);
  L.term = term, L.radr = radr;
  L.m_lds = a.m_lds ? mine : nullptr;
  L.sv = mine + nM;
  L.Ma = L.sv + nv;
  L.mv = L.Ma + nv;
  L.qacc = L.mv + nv;
  L.Jaref = L.qacc + nv;
  L.jv = L.Jaref + njmax;
  L.D = L.jv + njmax;
  L.fl = L.D + njmax;
  L.f = L.fl + njmax;
  L.rowl = (int *)(L.f + njmax);
  L.gl = (float *)(L.rowl + njmax);
  L.rows = lds + wv * (64 * 17);
  for (int k = threadIdx.x; k < a.nterm; k += blockDim.x) term[k] = (uint32_t)a.mulm_col[k] | (uint32_t)a.mulm_madr[k] << 16;
  for (int k = threadIdx.x; k <= nv; k += blockDim.x) radr[k] = a.mulm_rowadr[k];
  return L;
}

}  // namespace resident
}  // namespace im
