// The start of a constraint solve up to the first gradient in one launch: what the reference's
// init_context does before its first Hessian (src/instantmimic/utils/mjw_kernels/newton_fusion.py
// :431-500) -- worlds without constraint rows finish at qacc_smooth, Jaref = J qacc - aref,
// Ma = M qacc, forces and states of every row, the first gradient.  A wavefront per world, four
// worlds per workgroup, with the per-world routines of the resident Newton loop: the same
// operations in the same order as im_newton_init_empty_worlds, im_newton_init_jaref,
// im_mul_m_sparse, im_newton_eval_constraints and im_newton_gradient one after the other, so the
// same bits, with J read from memory once (the gradient's rows come from the cache).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"
#include "newton_wave.h"

namespace im {
namespace {

// LDS words of one wavefront: the tile of J, then sv, Ma, gl (nv each), Jaref, f, rowl (njmax each)
__host__ __device__ inline size_t init_wave_words(int nv, int njmax) { return 64 * 17 + 3 * (size_t)nv + 3 * (size_t)njmax; }

__global__ __launch_bounds__(256) void newton_init_context_kernel(resident::NewtonArgs a, const float *__restrict__ qacc_smooth,
                                                                  int64_t ld_qacc_smooth, const float *__restrict__ aref,
                                                                  int64_t ld_aref) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int nv = a.nv, njmax = a.njmax;
  uint32_t *term = (uint32_t *)lds;
  int *radr = (int *)(term + a.nterm);
  float *mine = (float *)(radr + nv + 1) + wv * init_wave_words(nv, njmax);
  float *tile = mine, *sv = tile + 64 * 17, *Ma_l = sv + nv, *gl = Ma_l + nv, *Jaref_l = gl + nv, *f = Jaref_l + njmax;
  int *rowl = (int *)(f + njmax);
  for (int k = threadIdx.x; k < a.nterm; k += blockDim.x) term[k] = (uint32_t)a.mulm_col[k] | (uint32_t)a.mulm_madr[k] << 16;
  for (int k = threadIdx.x; k <= nv; k += blockDim.x) radr[k] = a.mulm_rowadr[k];
  __syncthreads();  // the only workgroup barrier
  const int64_t w = (int64_t)blockIdx.x * 4 + wv;
  if (w >= a.nworld) return;
  const int nefc_raw = a.nefc ? a.nefc[w] : njmax;
  const bool empty = nefc_raw == 0;
  int nefc = nefc_raw < njmax ? nefc_raw : njmax;
  nefc = __builtin_amdgcn_readfirstlane(nefc > 0 ? nefc : 0);
  if (lane == 0) {
    a.niter[w] = 0;
    a.search_dot[w] = 0.0f;
    a.done[w] = empty ? 1 : 0;
  }
  // a world without constraint rows starts done, at the smooth acceleration
  for (int k = lane; k < nv; k += 64) {
    const float q = empty ? qacc_smooth[w * ld_qacc_smooth + k] : a.qacc[w * nv + k];
    if (empty) a.qacc[w * nv + k] = q;
    sv[k] = q;
  }
  resident::wave_sync();
  // Ma = M qacc, for every world
  resident::mul_m_world(a, term, radr, a.M + w * a.ldM, sv, a.Ma + w * nv, Ma_l, lane);
  if (empty) {  // what the stages leave of a done world: zero counts and the `unchanged` byte
    if (lane == 0) {
      a.quad_count[w] = 0;
      a.state_count[w] = 0;
      a.unchanged[w] = 1;
    }
    return;
  }
  const float *Jw = a.J + w * (int64_t)njmax * nv;
  resident::jv_world_tiled<true, true>(a, Jw, nefc, tile, sv, nullptr, Jaref_l, lane);
  resident::wave_sync();
  // Jaref = J qacc - aref, then force and state of every row (newton_stages.py:385-444 at step 0),
  // the rows whose being quadratic differs from the state that lay there, the rows with a force
  const int ne = __builtin_amdgcn_readfirstlane(a.ne ? a.ne[w] : 0), nf = __builtin_amdgcn_readfirstlane(a.nf ? a.nf[w] : 0);
  int nquad = 0, nstate = 0, cnt = 0;
  for (int base = 0; base < nefc; base += 64) {
    const int r = base + lane;
    bool quad_flip = false, changed = false;
    float fv = 0.0f;
    if (r < nefc) {
      const float x = Jaref_l[r] - aref[w * ld_aref + r], d = a.D[w * njmax + r];
      a.Jaref[w * njmax + r] = x;
      fv = -d * x;
      int st = 1;
      if (r >= ne && r < ne + nf) {
        const float fr = a.frictionloss[w * njmax + r], rf = search::safe_div(fr, d);
        if (x <= -rf) fv = fr, st = 2;
        else if (x >= rf) fv = -fr, st = 3;
      } else if (r >= ne && x >= 0.0f) {
        fv = 0.0f, st = 0;
      }
      const int old = a.state[w * njmax + r];
      a.force[w * njmax + r] = fv;
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
    const unsigned long long mf = __ballot(fv != 0.0f);
    if (fv != 0.0f) {
      const int pos = cnt + __popcll(mf & below);
      f[pos] = fv;
      rowl[pos] = r;
    }
    cnt += __popcll(mf);
  }
  if (lane == 0) {
    a.quad_count[w] = nquad;
    a.state_count[w] = nstate;
  }
  resident::wave_sync();
  resident::Scalars sc{};
  resident::gradient_world<true>(a, w, Jw, true, cnt, f, rowl, Ma_l, gl, sc, lane);
}

}  // namespace
}  // namespace im

extern "C" int im_newton_init_context(const im_newton_args *p, const float *qacc_smooth, int64_t ld_qacc_smooth,
                                      const float *efc_aref, int64_t ld_aref, int nv, int nM, void *stream) {
  if (!p || !qacc_smooth || !efc_aref || p->nworld < 0 || nv <= 0 || nM <= 0) return IM_ERR_ARG;
  if (p->nworld == 0) return IM_OK;
  im::resident::NewtonArgs a{};
  const int bad = im::resident::convert_args(*p, nv, nM, a);
  if (bad != IM_OK) return bad;
  if (ld_qacc_smooth < nv || ld_aref < p->njmax) return IM_ERR_STRIDE;
  const size_t lds = 4 * ((size_t)p->nterm + nv + 1 + 4 * im::init_wave_words(nv, p->njmax));
  if (lds > 160 * 1024) return IM_ERR_UNSUPPORTED;
  if (lds > 64 * 1024)
    IM_HIP_CHECK(hipFuncSetAttribute((const void *)im::newton_init_context_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
  hipLaunchKernelGGL(im::newton_init_context_kernel, dim3((unsigned)((p->nworld + 3) / 4)), dim3(256), lds,
                     (hipStream_t)stream, a, qacc_smooth, ld_qacc_smooth, efc_aref, ld_aref);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
