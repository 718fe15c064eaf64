// The matrix of the implicit-fast integrator, qH = M - h dF/dv on M's pattern, as far as the
// reference assembles it around upstream's derivative kernels
// (src/instantmimic/utils/mjw_step_optimized.py: deriv_smooth_vel :3803-3900,
// _prepare_implicit_qh :3734-3745, implicit_factor_optimized :4936-4968):
//   joint damping on the diagonal, the rows of free bodies reset to M, and the per-actuator
//   velocity gain that weights the actuator term moment' diag(gain) moment (which the deterministic
//   pair gather of the muscle kernels adds, like the tendon-damping and muscle terms).
// Upstream's kernels (derivative._qderiv_*, forward._implicit_free_body_reset_m) are third-party
// and not part of the reference tree; the arithmetic here follows MuJoCo's published
// mjd_smooth_vel for the implicit-fast integrator.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace im {
namespace {

// out[w, e] = M[w, e] + h damping[dof(e)] where e is the diagonal element of a dof that belongs to
// no free body, M[w, e] elsewhere.  Four elements a lane.
__global__ __launch_bounds__(256) void implicit_qh_base_kernel(const float *__restrict__ M, int64_t ldM,
                                                               const int32_t *__restrict__ elem_dof,
                                                               const float *__restrict__ damping,
                                                               int64_t ld_damping, float timestep,
                                                               float *__restrict__ out, int64_t ldo, int nM) {
  const int64_t w = blockIdx.y;
  const float *Mw = M + w * ldM, *dw = damping + w * ld_damping;
  float *ow = out + w * ldo;
  const int e0 = (blockIdx.x * 256 + threadIdx.x) * 4;
  float v[4];
  int d[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int e = e0 + k < nM ? e0 + k : nM - 1;
    v[k] = Mw[e];
    d[k] = elem_dof[e];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k)
    if (e0 + k < nM) ow[e0 + k] = d[k] >= 0 ? __builtin_fmaf(timestep, dw[d[k]], v[k]) : v[k];
}

// d force / d velocity of an actuator with affine gain and bias (MuJoCo mjGAIN_AFFINE = 1,
// mjBIAS_AFFINE = 1): bias parameter 2 plus gain parameter 2 times the control (or the
// activation for a stateful actuator: `input` is what the caller's model says drives the gain);
// zero where the force sits outside its limits.  One lane per (world, actuator).
__global__ __launch_bounds__(256) void actuator_velocity_gain_kernel(
    const int32_t *__restrict__ gaintype, const int32_t *__restrict__ biastype,
    const float *__restrict__ gainprm, const float *__restrict__ biasprm, int ldprm,
    const uint8_t *__restrict__ forcelimited, const float *__restrict__ forcerange,
    const float *__restrict__ input, int64_t ld_input, const float *__restrict__ force, int64_t ld_force,
    float *__restrict__ gain, int64_t ld_gain, int nu) {
  const int a = blockIdx.x * 256 + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (a >= nu) return;
  float v = 0.0f;
  if (biastype[a] == 1) v = biasprm[a * ldprm + 2];
  if (gaintype[a] == 1) v = __builtin_fmaf(gainprm[a * ldprm + 2], input[w * ld_input + a], v);
  if (forcelimited && forcelimited[a] && force) {
    const float f = force[w * ld_force + a];
    if (f <= forcerange[2 * a] || f >= forcerange[2 * a + 1]) v = 0.0f;
  }
  gain[w * ld_gain + a] = v;
}

}  // namespace
}  // namespace im

extern "C" {

int im_implicit_qh_base(const float *M, int64_t ldM, int nM, const int32_t *elem_dof, const float *dof_damping,
                        int64_t ld_damping, float timestep, float *qH, int64_t ld_qH, int nworld, void *stream) {
  if (nworld < 0 || nM < 0 || ld_damping < 0) return IM_ERR_ARG;
  if (nworld == 0 || nM == 0) return IM_OK;
  if (!M || !elem_dof || !dof_damping || !qH) return IM_ERR_ARG;
  if (ldM < nM || ld_qH < nM) return IM_ERR_STRIDE;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(im::implicit_qh_base_kernel, dim3((unsigned)((nM + 1023) / 1024), (unsigned)nw), dim3(256), 0,
                       (hipStream_t)stream, M + (int64_t)w0 * ldM, ldM, elem_dof, dof_damping + (int64_t)w0 * ld_damping,
                       ld_damping, timestep, qH + (int64_t)w0 * ld_qH, ld_qH, nM);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

int im_actuator_velocity_gain(const int32_t *gaintype, const int32_t *biastype, const float *gainprm,
                              const float *biasprm, int ld_prm, const uint8_t *forcelimited,
                              const float *forcerange, const float *input, int64_t ld_input, const float *force,
                              int64_t ld_force, float *gain, int64_t ld_gain, int nu, int nworld, void *stream) {
  if (nworld < 0 || nu < 0) return IM_ERR_ARG;
  if (nworld == 0 || nu == 0) return IM_OK;
  if (!gaintype || !biastype || !gainprm || !biasprm || !input || !gain || ld_prm < 3) return IM_ERR_ARG;
  if (forcelimited && !forcerange) return IM_ERR_ARG;
  if (ld_input < nu || ld_gain < nu || (force && ld_force < nu)) return IM_ERR_STRIDE;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(im::actuator_velocity_gain_kernel, dim3((unsigned)((nu + 255) / 256), (unsigned)nw), dim3(256), 0,
                       (hipStream_t)stream, gaintype, biastype, gainprm, biasprm, ld_prm, forcelimited, forcerange,
                       input + (int64_t)w0 * ld_input, ld_input, force ? force + (int64_t)w0 * ld_force : nullptr, ld_force,
                       gain + (int64_t)w0 * ld_gain, ld_gain, nu);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
