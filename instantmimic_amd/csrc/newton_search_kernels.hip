// Launchers of the scalar line search and of the constraints' re-evaluation (the per-world code is
// in newton_search.h).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"
#include "newton_search.h"

namespace im {
namespace {

using namespace search;

// A wavefront per world: the sums run over 32 lanes (the reference's reduction width) and the two
// halves of the wavefront evaluate different candidate steps of a round side by side.
template <int HELD>
__global__ __launch_bounds__(64) void newton_linesearch_kernel(SearchArgs a) {
  const int lane = threadIdx.x & 31;
  const int64_t w = blockIdx.x;
  if (w >= a.nworld) return;
  if (a.done && a.done[w]) return;
  linesearch_world<HELD, true>(a, w, lane);
}

// A wavefront per world.
__global__ __launch_bounds__(256) void newton_eval_constraints_kernel(
    const float *__restrict__ Jaref, int64_t ld_Jaref, const float *__restrict__ D, int64_t ld_D,
    const float *__restrict__ frictionloss, int64_t ld_floss, const int32_t *__restrict__ ne_,
    const int32_t *__restrict__ nf_, const int32_t *__restrict__ nefc_, int njmax,
    const uint8_t *__restrict__ done, const uint8_t *__restrict__ exhausted, float *__restrict__ force,
    int64_t ld_force, int32_t *__restrict__ state, int64_t ld_state, int32_t *__restrict__ ids, int ld_ids,
    int32_t *__restrict__ quad_count, int32_t *__restrict__ state_count, int nworld) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (w >= nworld) return;
  if (lane == 0) {
    quad_count[w] = 0;
    state_count[w] = 0;
  }
  if (done && done[w]) return;
  eval_constraints_world(Jaref, ld_Jaref, D, ld_D, frictionloss, ld_floss, ne_, nf_, nefc_, njmax, exhausted, force,
                         ld_force, state, ld_state, ids, ld_ids, quad_count, state_count, w, lane);
}

}  // namespace
}  // namespace im

using namespace im;

extern "C" int im_newton_linesearch(const float *opt_tolerance, int ntolerance, const float *opt_ls_tolerance,
                                    int nls_tolerance, const float *stat_meaninertia, int nmeaninertia,
                                    const int32_t *ne, const int32_t *nf, const int32_t *nefc, int njmax,
                                    const float *qfrc_smooth, int64_t ld_smooth, const float *efc_D, int64_t ld_D,
                                    const float *efc_frictionloss, int64_t ld_frictionloss, const float *Jaref,
                                    int64_t ld_Jaref, const float *search, int64_t ld_search, const float *search_dot,
                                    const float *mv, int64_t ld_mv, const float *jv, int64_t ld_jv,
                                    const float *efc_Ma, int64_t ld_Ma, const uint8_t *done, int ls_iterations,
                                    int overflow_bit, float *alpha, float *improvement, uint8_t *ls_exhausted,
                                    int32_t *overflow, int nv, int nworld, void *stream) {
  if (nworld < 0 || nv <= 0 || njmax < 0 || ls_iterations < 0 || ntolerance <= 0 || nls_tolerance <= 0 ||
      nmeaninertia <= 0)
    return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!opt_tolerance || !opt_ls_tolerance || !stat_meaninertia || !qfrc_smooth || !search || !search_dot || !mv ||
      !efc_Ma || !alpha || !improvement || !ls_exhausted || (njmax > 0 && (!efc_D || !Jaref || !jv)))
    return IM_ERR_ARG;
  if (nf && !efc_frictionloss) return IM_ERR_ARG;
  if (ld_smooth < nv || ld_search < nv || ld_mv < nv || ld_Ma < nv || ld_D < njmax || ld_Jaref < njmax ||
      ld_jv < njmax || (efc_frictionloss && ld_frictionloss < njmax))
    return IM_ERR_STRIDE;
  SearchArgs a{opt_tolerance, opt_ls_tolerance, stat_meaninertia, ntolerance, nls_tolerance, nmeaninertia, ne, nf,
               nefc, qfrc_smooth, efc_D, efc_frictionloss, Jaref, search, search_dot, mv, jv, efc_Ma, ld_smooth, ld_D,
               ld_frictionloss, ld_Jaref, ld_search, ld_mv, ld_jv, ld_Ma, done, alpha, improvement, ls_exhausted,
               overflow, overflow_bit, nv, njmax, ls_iterations, nworld};
  // rows per lane: two up to 64 rows, four up to 128, eight up to 256
  auto fn = njmax <= 64 ? newton_linesearch_kernel<2> : njmax <= 128 ? newton_linesearch_kernel<4>
            : njmax <= 256 ? newton_linesearch_kernel<8> : newton_linesearch_kernel<0>;
  hipLaunchKernelGGL(fn, dim3((unsigned)nworld), dim3(64), 0, (hipStream_t)stream, a);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_newton_eval_constraints(const float *Jaref, int64_t ld_Jaref, const float *efc_D, int64_t ld_D,
                                          const float *efc_frictionloss, int64_t ld_frictionloss, const int32_t *ne,
                                          const int32_t *nf, const int32_t *nefc, int njmax, const uint8_t *done,
                                          const uint8_t *ls_exhausted, float *efc_force, int64_t ld_force,
                                          int32_t *efc_state, int64_t ld_state, int32_t *quad_changed_ids, int ld_ids,
                                          int32_t *quad_changed_count, int32_t *state_changed_count, int nworld,
                                          void *stream) {
  if (nworld < 0 || njmax < 0 || ld_ids < 0) return IM_ERR_ARG;
  if (nworld == 0) return IM_OK;
  if (!quad_changed_count || !state_changed_count || (njmax > 0 && (!Jaref || !efc_D || !efc_force || !efc_state || !quad_changed_ids)))
    return IM_ERR_ARG;
  if (nf && !efc_frictionloss) return IM_ERR_ARG;
  if (ld_Jaref < njmax || ld_D < njmax || ld_force < njmax || ld_state < njmax || (efc_frictionloss && ld_frictionloss < njmax))
    return IM_ERR_STRIDE;
  hipLaunchKernelGGL(newton_eval_constraints_kernel, dim3((unsigned)((nworld + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     Jaref, ld_Jaref, efc_D, ld_D, efc_frictionloss, ld_frictionloss, ne, nf, nefc, njmax, done,
                     ls_exhausted, efc_force, ld_force, efc_state, ld_state, quad_changed_ids, ld_ids,
                     quad_changed_count, state_changed_count, nworld);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
