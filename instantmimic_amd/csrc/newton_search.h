// The scalar line search of a Newton iteration and the re-evaluation of the constraints after the
// step, for one world: the two parts of the reference's line-search stage
// (src/instantmimic/utils/mjw_kernels/newton_stages.py:79-444) that sit between J v and the
// gradient.  The stage's control flow, reductions (32 lanes, shuffle-down tree, lane 0 broadcast)
// and tolerances are the reference's; the per-row cost model it calls
// (solver._compute_efc_eval_pt_*_pyramidal, _eval_pt, _in_bracket, _eval_constraint, safe_div) is
// upstream mujoco_warp code that is not in the reference tree and is restated here from MuJoCo's
// published primal line search: for x = Jaref + alpha jv a row costs
//   equality:      D x^2 / 2                                  (summed with the Gauss term)
//   friction loss: D x^2 / 2 inside |x| < f / D, else f (|x| - f / (2 D))
//   other rows:    D x^2 / 2 where x < 0, else 0              (pyramidal cones, limits)
// and a point is (cost - cost at alpha 0, first derivative, second derivative).
// Shared by the per-stage kernels and the resident Newton kernel.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace im {
namespace search {


constexpr float kMinVal = 1.0e-15f;        // MuJoCo's mjMINVAL
constexpr float kMaxVal = 1.0e10f;         // MuJoCo's mjMAXVAL
constexpr float kAlphaNoise = 0x1p-20f;    // relative noise of a summed first derivative (this library's choice)

struct Pt {
  float c, g, h;  // cost (relative to alpha 0), d / d alpha, d2 / d alpha2
};
__device__ __forceinline__ Pt operator+(Pt a, Pt b) { return {a.c + b.c, a.g + b.g, a.h + b.h}; }
__device__ __forceinline__ float safe_div(float x, float y) { return x / (y != 0.0f ? y : kMinVal); }
// a quadratic (q0, q1, q2) at alpha
__device__ __forceinline__ Pt eval_pt(Pt q, float a) { return {a * a * q.h + a * q.g + q.c, 2.0f * a * q.h + q.g, 2.0f * q.h}; }
__device__ __forceinline__ bool in_bracket(Pt x, Pt y) { return (x.g < y.g && y.g < 0.0f) || (x.g > y.g && y.g > 0.0f); }

// The quadratic a row follows at position x: its own where it is in the quadratic zone, the linear
// pieces of the friction-loss cost outside, nothing for a satisfied inequality.
// (rf: the friction row's f / D, which does not change during a search: formed once per row)
__device__ __forceinline__ Pt row_quad(bool friction, float D, float f, float rf, float jaref, float jv, float x) {
  const Pt quad = {0.5f * jaref * jaref * D, jv * jaref * D, 0.5f * jv * jv * D};
  if (friction) {
    if (x <= -rf) return {f * (-0.5f * rf - jaref), -f * jv, 0.0f};
    if (x >= rf) return {f * (-0.5f * rf + jaref), f * jv, 0.0f};
    return quad;
  }
  if (x < 0.0f) return quad;
  return {0.0f, 0.0f, 0.0f};
}
// point of a row at alpha, cost relative to alpha 0, with the row's cost at alpha 0 computed beforehand (row_quad(..., jaref).c)
__device__ __forceinline__ Pt row_point_from(bool friction, float D, float f, float rf, float jaref, float jv, float c0, float alpha) {
  Pt p = eval_pt(row_quad(friction, D, f, rf, jaref, jv, jaref + alpha * jv), alpha);
  p.c = p.c - c0;
  return p;
}
// point of a row at alpha 0 with its cost itself
__device__ __forceinline__ Pt row_point_zero(bool friction, float D, float f, float rf, float jaref, float jv) {
  const Pt q = row_quad(friction, D, f, rf, jaref, jv, jaref);
  return {q.c, q.g, 2.0f * q.h};
}

// sum over the 32 lanes of a world: shuffle-down tree, lane 0's value to all, then the +0 of the
// later warps' empty partials (newton_stages.py:36-52).  The tree's first step crosses the two
// rows of 16 lanes of a world (v_permlane16_swap_b32 hands every even row the odd row behind it),
// the others stay inside a row (DPP shifts); what a lane receives from beyond its row or world
// never reaches lane 0, whose sum has the association of the 32-lane shuffle-down tree.  Lane 0's
// (lane 32's) value then goes to its world through a lane read.  A world's 32 lanes are active or
// inactive together.
template <int N>
__device__ __forceinline__ float row_shl(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + N, 0xF, 0xF, true));
}
__device__ __forceinline__ float lanes_sum(float s) {
  // v_permlane16_swap_b32 a, b: the odd rows of a change places with the even rows of b.  Written
  // out, with its wait states: the compiler's builtin returns the first result twice when both
  // operands hold the same value.
  unsigned upper = __builtin_bit_cast(unsigned, s), lower = upper;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lower), "+v"(upper));
  s = s + __builtin_bit_cast(float, upper);  // lane i of an even row: lane i + 16
  s = s + row_shl<8>(s);
  s = s + row_shl<4>(s);
  s = s + row_shl<2>(s);
  s = s + row_shl<1>(s);
  const float first = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 0));
  const float second = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 32));
  s = (threadIdx.x & 32) ? second : first;
  return s + 0.0f;
}
__device__ __forceinline__ Pt lanes_sum(Pt p) { return {lanes_sum(p.c), lanes_sum(p.g), lanes_sum(p.h)}; }
// The same tree with the sums of both halves of the wavefront handed to every lane: `lower` that of
// lanes 0 - 31, `upper` that of lanes 32 - 63 (for a wavefront whose halves sum different things).
__device__ __forceinline__ void lanes_sum_halves(float s, float &lower_sum, float &upper_sum) {
  unsigned upper = __builtin_bit_cast(unsigned, s), lower = upper;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lower), "+v"(upper));
  s = s + __builtin_bit_cast(float, upper);
  s = s + row_shl<8>(s);
  s = s + row_shl<4>(s);
  s = s + row_shl<2>(s);
  s = s + row_shl<1>(s);
  lower_sum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 0)) + 0.0f;
  upper_sum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 32)) + 0.0f;
}
__device__ __forceinline__ void lanes_sum_halves(Pt p, Pt &lower_sum, Pt &upper_sum) {
  lanes_sum_halves(p.c, lower_sum.c, upper_sum.c);
  lanes_sum_halves(p.g, lower_sum.g, upper_sum.g);
  lanes_sum_halves(p.h, lower_sum.h, upper_sum.h);
}

struct SearchArgs {
  const float *tolerance, *ls_tolerance, *meaninertia;
  int ntolerance, nls_tolerance, nmeaninertia;
  const int32_t *ne, *nf, *nefc;
  const float *smooth, *D, *frictionloss, *Jaref, *search, *search_dot, *mv, *jv, *Ma;
  int64_t ld_smooth, ld_D, ld_floss, ld_Jaref, ld_search, ld_mv, ld_jv, ld_Ma;
  const uint8_t *done;
  float *alpha, *improvement;
  uint8_t *exhausted;
  int32_t *overflow;
  int overflow_bit, nv, njmax, ls_iterations, nworld;
};

// One world's rows and scalars as the line search reads them (the rows may lie in memory or in LDS).
struct LsWorld {
  const float *smooth, *D, *frictionloss, *Jaref, *search, *mv, *jv, *Ma;  // frictionloss may be null
  float search_dot, tolerance, ls_tolerance, meaninertia;
  int ne, nf, nefc, nv, ls_iterations;
  // optional, two arrays of nefc floats each that the search may use for what it forms once per row
  // (a friction row's f / D, the row's cost at step 0) when it does not hold the rows in registers
  float *row_scratch0 = nullptr, *row_scratch1 = nullptr;
};
struct LsResult {
  float alpha, improvement;
  bool exhausted, converged;
};

// 32 lanes per world (the reference's reduction width), two such groups per wavefront.  HELD: rows
// of the world a lane keeps in registers (weight, friction loss, Jaref, jv and the cost at alpha 0)
// -- every candidate step evaluates every row, three candidates per round; 0: more rows than that,
// read at every evaluation.  Every lane of the group returns the same result.
// SPLIT: both halves of the wavefront work on the same world (each with `lane` = 0 .. 31): of a
// round's three candidate steps the lower half evaluates the first and the upper half the second
// (each sum is still one group's 32-lane tree), both evaluate the third.
template <int HELD, bool SPLIT = false>
__device__ __forceinline__ LsResult linesearch_rows(const LsWorld &wd, int lane) {
  const int nv = wd.nv, ne = wd.ne, nf = wd.nf, nefc = wd.nefc;
  const float *D = wd.D, *fl = wd.frictionloss, *Jaref = wd.Jaref, *jv = wd.jv;
  const float tolerance = wd.tolerance, ls_tolerance = wd.ls_tolerance;
  const float snorm = sqrtf(wd.search_dot);
  const float scale = wd.meaninertia * (float)nv;
  const float gtol = fmaxf(tolerance * ls_tolerance * snorm * scale, 1.0e-6f);
  // Gauss term and equality rows: one quadratic (0, g1, g2)
  float g1 = 0.0f, g2 = 0.0f;
  for (int dof = lane; dof < nv; dof += 32) {
    const float s = wd.search[dof];
    g1 = g1 + s * (wd.Ma[dof] - wd.smooth[dof]);
    g2 = g2 + 0.5f * s * wd.mv[dof];
  }
  for (int r = lane; r < ne; r += 32) {
    const float jvD = jv[r] * D[r];
    g1 = g1 + jvD * Jaref[r];
    g2 = g2 + 0.5f * jv[r] * jvD;
  }
  const Pt gauss = {0.0f, lanes_sum(g1), lanes_sum(g2)};
  // this lane's rows ne + lane, ne + lane + 32, ...
  constexpr int NH = HELD > 0 ? HELD : 1;
  float hd[NH], hf[NH], hrf[NH], hja[NH], hv[NH], hc0[NH];
  if constexpr (HELD > 0) {
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      const int r = ne + lane + 32 * k, rc = r < nefc ? r : (nefc > 0 ? nefc - 1 : 0);
      const bool in = r < nefc, fr = r < ne + nf;
      hd[k] = in ? D[rc] : 0.0f;
      hf[k] = (in && fl) ? fl[rc] : 0.0f;
      hja[k] = in ? Jaref[rc] : 0.0f;
      hv[k] = in ? jv[rc] : 0.0f;
      hrf[k] = (in && fr) ? safe_div(hf[k], hd[k]) : 0.0f;
      hc0[k] = row_quad(fr, hd[k], hf[k], hrf[k], hja[k], hv[k], hja[k]).c;
    }
  }
  // sum over this lane's rows of the rows' points at one or three step lengths
  auto rows_sum = [&](auto point) {
    if constexpr (HELD > 0) {
#pragma unroll
      for (int k = 0; k < HELD; ++k) {
        const int r = ne + lane + 32 * k;
        if (r < nefc) point(r < ne + nf, hd[k], hf[k], hrf[k], hja[k], hv[k], hc0[k]);
      }
    } else if (wd.row_scratch0) {
      for (int r = ne + lane; r < nefc; r += 32)
        point(r < ne + nf, D[r], fl ? fl[r] : 0.0f, wd.row_scratch0[r], Jaref[r], jv[r], wd.row_scratch1[r]);
    } else {
      for (int r = ne + lane; r < nefc; r += 32) {
        const bool fr = r < ne + nf;
        const float d = D[r], f = fl ? fl[r] : 0.0f, ja = Jaref[r], v = jv[r];
        const float rf = fr ? safe_div(f, d) : 0.0f;
        point(fr, d, f, rf, ja, v, row_quad(fr, d, f, rf, ja, v, ja).c);
      }
    }
  };
  if (HELD == 0 && wd.row_scratch0) {
    // a lane writes and later reads its own rows only (a wavefront's two halves write the same values)
    for (int r = ne + lane; r < nefc; r += 32) {
      const bool fr = r < ne + nf;
      const float d = D[r], f = fl ? fl[r] : 0.0f, ja = Jaref[r], v = jv[r];
      const float rf = fr ? safe_div(f, d) : 0.0f;
      wd.row_scratch0[r] = rf;
      wd.row_scratch1[r] = row_quad(fr, d, f, rf, ja, v, ja).c;
    }
  }
  auto rows_at = [&](float alpha) {
    Pt s = {0.0f, 0.0f, 0.0f};
    rows_sum([&](bool fr, float d, float f, float rf, float ja, float v, float c0) { s = s + row_point_from(fr, d, f, rf, ja, v, c0, alpha); });
    return lanes_sum(s);
  };
  Pt z = {0.0f, 0.0f, 0.0f};
  rows_sum([&](bool fr, float d, float f, float rf, float ja, float v, float) { z = z + row_point_zero(fr, d, f, rf, ja, v); });
  const Pt rows0 = lanes_sum(z);
  const Pt p0 = {gauss.c + rows0.c, gauss.g + rows0.g, 2.0f * gauss.h + rows0.h};
  const Pt p0_delta = {0.0f, p0.g, p0.h};
  const float q1_abs = sqrtf(2.0f * fmaxf(rows0.c, 0.0f) * fmaxf(rows0.h, 0.0f)) + fabsf(gauss.g);
  const float gtol_accept = fmaxf(gtol, kAlphaNoise * q1_abs);
  const float noise_floor = kAlphaNoise * fmaxf(1.0f, safe_div(q1_abs, p0.h));
  float alpha = 0.0f, improvement = 0.0f;
  bool converged = fabsf(p0.g) < kAlphaNoise * q1_abs;
  const float lo_alpha_in = -safe_div(p0.g, p0.h);
  Pt lo_in = {0.0f, 0.0f, 0.0f};
  if (!converged) {
    lo_in = eval_pt(gauss, lo_alpha_in) + rows_at(lo_alpha_in);
    if (fabsf(lo_in.g) < gtol_accept && lo_in.c < 0.0f) {
      converged = true;
      alpha = lo_alpha_in;
      improvement = -lo_in.c;
    }
  }
  if (!converged) {
    const bool lo_less = lo_in.g < p0.g;
    Pt lo = lo_less ? lo_in : p0_delta, hi = lo_less ? p0_delta : lo_in;
    float lo_alpha = lo_less ? lo_alpha_in : 0.0f, hi_alpha = lo_less ? 0.0f : lo_alpha_in;
    for (int it = 0; it < wd.ls_iterations; ++it) {
      const float lo_next_alpha = lo_alpha - safe_div(lo.g, lo.h);
      const float hi_next_alpha = hi_alpha - safe_div(hi.g, hi.h);
      const float mid_alpha = 0.5f * (lo_alpha + hi_alpha);
      Pt s_lo = {0.0f, 0.0f, 0.0f}, s_hi = s_lo, s_mid = s_lo;
      Pt lo_next, hi_next, mid;
      if constexpr (SPLIT) {
        const float mine_alpha = (threadIdx.x & 32) ? hi_next_alpha : lo_next_alpha;
        rows_sum([&](bool fr, float d, float f, float rf, float ja, float v, float c0) {
          s_lo = s_lo + row_point_from(fr, d, f, rf, ja, v, c0, mine_alpha);
          s_mid = s_mid + row_point_from(fr, d, f, rf, ja, v, c0, mid_alpha);
        });
        Pt rows_lo, rows_hi, rows_mid, same;
        lanes_sum_halves(s_lo, rows_lo, rows_hi);
        lanes_sum_halves(s_mid, rows_mid, same);
        lo_next = eval_pt(gauss, lo_next_alpha) + rows_lo;
        hi_next = eval_pt(gauss, hi_next_alpha) + rows_hi;
        mid = eval_pt(gauss, mid_alpha) + rows_mid;
      } else {
        rows_sum([&](bool fr, float d, float f, float rf, float ja, float v, float c0) {
          s_lo = s_lo + row_point_from(fr, d, f, rf, ja, v, c0, lo_next_alpha);
          s_hi = s_hi + row_point_from(fr, d, f, rf, ja, v, c0, hi_next_alpha);
          s_mid = s_mid + row_point_from(fr, d, f, rf, ja, v, c0, mid_alpha);
        });
        lo_next = eval_pt(gauss, lo_next_alpha) + lanes_sum(s_lo);
        hi_next = eval_pt(gauss, hi_next_alpha) + lanes_sum(s_hi);
        mid = eval_pt(gauss, mid_alpha) + lanes_sum(s_mid);
      }
      const bool conv_lo = fabsf(lo_next.g) < gtol_accept && lo_next.c < 0.0f;
      const bool conv_hi = fabsf(hi_next.g) < gtol_accept && hi_next.c < 0.0f;
      const bool conv_mid = fabsf(mid.g) < gtol_accept && mid.c < 0.0f;
      const bool conv = conv_lo || conv_hi || conv_mid;
      bool swap_lo = false, swap_hi = false;
      if (conv) {
        Pt best = {kMaxVal, 0.0f, 0.0f};
        float best_alpha = 0.0f;
        if (conv_lo && lo_next.c < best.c) best = lo_next, best_alpha = lo_next_alpha;
        if (conv_hi && hi_next.c < best.c) best = hi_next, best_alpha = hi_next_alpha;
        if (conv_mid && mid.c < best.c) best = mid, best_alpha = mid_alpha;
        lo = hi = best;
        lo_alpha = hi_alpha = best_alpha;
      } else {
        const bool a1 = in_bracket(lo, lo_next);
        if (a1) lo = lo_next, lo_alpha = lo_next_alpha;
        const bool a2 = in_bracket(lo, mid);
        if (a2) lo = mid, lo_alpha = mid_alpha;
        const bool a3 = in_bracket(lo, hi_next);
        if (a3) lo = hi_next, lo_alpha = hi_next_alpha;
        swap_lo = a1 || a2 || a3;
        const bool b1 = in_bracket(hi, hi_next) || (hi.g < 0.0f && hi_next.g > 0.0f);
        if (b1) hi = hi_next, hi_alpha = hi_next_alpha;
        const bool b2 = in_bracket(hi, mid);
        if (b2) hi = mid, hi_alpha = mid_alpha;
        const bool b3 = in_bracket(hi, lo_next);
        if (b3) hi = lo_next, hi_alpha = lo_next_alpha;
        swap_hi = b1 || b2 || b3;
      }
      const bool ls_done = conv || (!swap_lo && !swap_hi) || (lo.c < 0.0f && lo.g < 0.0f && lo.g > -gtol) ||
                           (hi.c < 0.0f && hi.g > 0.0f && hi.g < gtol);
      const bool improved = lo.c < 0.0f || hi.c < 0.0f;
      const bool lo_better = lo.c < hi.c;
      if (improved) {
        alpha = lo_better ? lo_alpha : hi_alpha;
        improvement = -(lo_better ? lo.c : hi.c);
      }
      if (ls_done) {
        converged = true;
        break;
      }
    }
  }
  return {alpha, improvement, fabsf(alpha) < noise_floor, converged};
}

template <int HELD, bool SPLIT = false>
__device__ __forceinline__ void linesearch_world(const SearchArgs &a, int64_t w, int lane) {
  int nefc = a.nefc ? a.nefc[w] : a.njmax;
  nefc = nefc < a.njmax ? nefc : a.njmax;
  const LsWorld r{a.smooth + w * a.ld_smooth, a.D + w * a.ld_D, a.frictionloss ? a.frictionloss + w * a.ld_floss : nullptr,
                  a.Jaref + w * a.ld_Jaref, a.search + w * a.ld_search, a.mv + w * a.ld_mv, a.jv + w * a.ld_jv,
                  a.Ma + w * a.ld_Ma, a.search_dot[w], a.tolerance[w % a.ntolerance], a.ls_tolerance[w % a.nls_tolerance],
                  a.meaninertia[w % a.nmeaninertia], a.ne ? a.ne[w] : 0, a.nf ? a.nf[w] : 0, nefc, a.nv, a.ls_iterations};
  const LsResult out = linesearch_rows<HELD, SPLIT>(r, lane);
  if (SPLIT ? (threadIdx.x & 63) == 0 : lane == 0) {
    a.alpha[w] = out.alpha;
    a.improvement[w] = out.improvement;
    a.exhausted[w] = out.exhausted ? 1 : 0;
    if (!out.converged && a.overflow) a.overflow[w] = a.overflow[w] | a.overflow_bit;
  }
}

// After the step: force and state of every row from the new Jaref, the rows whose being
// QUADRATIC flipped in ascending order, their count and the count of all state changes plus one
// for an exhausted line search (newton_stages.py:385-444).  States: 0 satisfied, 1 quadratic,
// 2 linear negative, 3 linear positive (MuJoCo's mjtConstraintState).  A wavefront per world.
__device__ __forceinline__ void eval_constraints_world(
    const float *__restrict__ Jaref, int64_t ld_Jaref, const float *__restrict__ D, int64_t ld_D,
    const float *__restrict__ frictionloss, int64_t ld_floss, const int32_t *__restrict__ ne_,
    const int32_t *__restrict__ nf_, const int32_t *__restrict__ nefc_, int njmax,
    const uint8_t *__restrict__ exhausted, float *__restrict__ force,
    int64_t ld_force, int32_t *__restrict__ state, int64_t ld_state, int32_t *__restrict__ ids, int ld_ids,
    int32_t *__restrict__ quad_count, int32_t *__restrict__ state_count, int64_t w, int lane) {
  const int ne = ne_ ? ne_[w] : 0, nf = nf_ ? nf_[w] : 0;
  int nefc = nefc_ ? nefc_[w] : njmax;
  nefc = nefc < njmax ? nefc : njmax;
  int nquad = 0, nstate = 0;
  for (int base = 0; base < nefc; base += 64) {
    const int r = base + lane;
    bool quad_flip = false, changed = false;
    if (r < nefc) {
      const float x = Jaref[w * ld_Jaref + r], d = D[w * ld_D + r];
      float f = -d * x;
      int s = 1;
      if (r >= ne && r < ne + nf) {
        const float fr = frictionloss[w * ld_floss + r], rf = safe_div(fr, d);
        if (x <= -rf) f = fr, s = 2;
        else if (x >= rf) f = -fr, s = 3;
      } else if (r >= ne && x >= 0.0f) {
        f = 0.0f, s = 0;
      }
      const int old = state[w * ld_state + r];
      force[w * ld_force + r] = f;
      state[w * ld_state + r] = s;
      quad_flip = (old == 1) != (s == 1);
      changed = old != s;
    }
    const unsigned long long m = __ballot(quad_flip);
    if (quad_flip) {
      const int slot = nquad + __popcll(m & ((1ull << lane) - 1ull));
      if (slot < ld_ids) ids[w * (int64_t)ld_ids + slot] = r;
    }
    nquad += __popcll(m);
    nstate += __popcll(__ballot(changed));
  }
  if (lane == 0) {
    quad_count[w] = nquad;
    state_count[w] = nstate + ((exhausted && exhausted[w]) ? 1 : 0);
  }
}


}  // namespace search
}  // namespace im
