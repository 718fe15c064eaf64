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

// Damping with polynomial terms, as a damping coefficient for the implicit matrix: a damper whose
// force is  -v (b + p_1 |v| + ... + p_K |v|^K)  has the slope  -(b + 2 p_1 |v| + ... + (K + 1) p_K |v|^K)
// in v, evaluated by Horner's rule with fused multiply-adds from the highest term down.
// One lane per (world, item).
__global__ __launch_bounds__(256) void polynomial_damping_kernel(const float *__restrict__ base, int64_t ld_base,
                                                                 const float *__restrict__ poly, int64_t ld_poly,
                                                                 int nterm, const float *__restrict__ velocity,
                                                                 int64_t ld_velocity, float *__restrict__ out,
                                                                 int64_t ld_out, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (i >= n) return;
  const float a = fabsf(velocity[w * ld_velocity + i]);
  const float *p = poly + w * ld_poly + (int64_t)i * nterm;
  float acc = 0.0f;
  for (int k = nterm; k >= 1; --k) acc = __builtin_fmaf(acc, a, (float)(k + 1) * p[k - 1]);
  out[w * ld_out + i] = __builtin_fmaf(acc, a, base[w * ld_base + i]);
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

// Everything above and the two pair-sum terms in one launch, a workgroup per world: the row of
// qH lives in LDS from the damped copy of M to the last term, the actuators' gains next to it.
// A term adds  scale * sum over the rows r of weight_r row_r' row_r  on M's pattern with the
// tables and the order of the muscle gather (csrc/muscle_kernels.hip: products of entry pairs
// summed in chunks of 16 from zero, an element's chunks added in order, one fused multiply-add
// into the element), so the result equals im_implicit_qh_base, im_actuator_velocity_gain and one
// im_muscle_implicit_gather per term called one after the other, bit for bit.
struct QhGain {
  const int32_t *gaintype, *biastype;
  const float *gainprm, *biasprm;
  int ldprm;
  const uint8_t *forcelimited;
  const float *forcerange, *input;
  int64_t ld_input;
  const float *force;
  int64_t ld_force;
  float *gain;  // (nworld, ld_gain) output, may be null
  int64_t ld_gain;
  int nu;
};

__global__ __launch_bounds__(256) void implicit_qh_kernel(const float *__restrict__ M, int64_t ldM, int nM,
                                                          const int32_t *__restrict__ elem_dof,
                                                          const float *__restrict__ damping, int64_t ld_damping,
                                                          float timestep, QhGain g, im_row_pair_term ta,
                                                          im_row_pair_term tt, int max_entries,
                                                          float *__restrict__ out, int64_t ldo) {
  extern __shared__ float lds[];
  float *q = lds;                           // [nM]
  float *gain = q + nM;                     // [nu]
  float *m = gain + g.nu;                   // [max_entries + 1]
  float *weighted = m + max_entries + 1;    // [max_entries + 1]
  float *partial = weighted + max_entries + 1;  // [max chunk count]
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t w = blockIdx.x;
  const float *Mw = M + w * ldM, *dw = damping + w * ld_damping;
  for (int e = tid; e < nM; e += nt) {
    const int d = elem_dof[e];
    const float v = Mw[e];
    q[e] = d >= 0 ? __builtin_fmaf(timestep, dw[d], v) : v;
  }
  for (int a = tid; a < g.nu; a += nt) {
    float v = 0.0f;
    if (g.biastype[a] == 1) v = g.biasprm[a * g.ldprm + 2];
    if (g.gaintype[a] == 1) v = __builtin_fmaf(g.gainprm[a * g.ldprm + 2], g.input[w * g.ld_input + a], v);
    if (g.forcelimited && g.forcelimited[a] && g.force) {
      const float f = g.force[w * g.ld_force + a];
      if (f <= g.forcerange[2 * a] || f >= g.forcerange[2 * a + 1]) v = 0.0f;
    }
    gain[a] = v;
    if (g.gain) g.gain[w * g.ld_gain + a] = v;
  }
  __syncthreads();
  for (int which = 0; which < 2; ++which) {
    const im_row_pair_term &t = which == 0 ? ta : tt;
    if (t.nentry <= 0 || t.nelem <= 0) continue;  // the same for the whole workgroup
    for (int e = tid; e < t.nentry; e += nt) {
      const float v = t.values[w * t.ld_values + (t.entry_source ? t.entry_source[e] : e)];
      const int row = t.entry_row[e];
      const float wt = t.weight ? t.weight[w * t.ld_weight + row] : gain[row];
      m[e] = v;
      weighted[e] = wt * v;
    }
    if (tid == 0) {
      m[t.nentry] = 0.0f;
      weighted[t.nentry] = 0.0f;
    }
    __syncthreads();
    for (int c = tid; c < t.chunk_count; c += nt) {
      float total = 0.0f;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int packed = t.chunk_pairs[(size_t)k * t.chunk_count + c];
        total = __builtin_fmaf(weighted[packed & 0xFFFF], m[packed >> 16], total);
      }
      partial[c] = total;
    }
    __syncthreads();
    for (int slot = tid; slot < t.nelem; slot += nt) {
      float acc = 0.0f;
      const int c1 = t.chunk_offsets[slot + 1];
      for (int c = t.chunk_offsets[slot]; c < c1; ++c) acc = acc + partial[c];
      const int e = t.elem_ids[slot];
      q[e] = __builtin_fmaf(t.scale, acc, q[e]);
    }
    __syncthreads();
  }
  float *ow = out + w * ldo;
  for (int e = tid; e < nM; e += nt) ow[e] = q[e];
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

int im_polynomial_damping(const float *base, int64_t ld_base, const float *poly, int64_t ld_poly, int nterm,
                          const float *velocity, int64_t ld_velocity, float *out, int64_t ld_out, int n, int nworld,
                          void *stream) {
  if (nworld < 0 || n < 0 || nterm < 0 || ld_base < 0 || ld_poly < 0) return IM_ERR_ARG;
  if (nworld == 0 || n == 0) return IM_OK;
  if (!base || (nterm > 0 && !poly) || !velocity || !out) return IM_ERR_ARG;
  if (ld_velocity < n || ld_out < n || (ld_base != 0 && ld_base < n) || (ld_poly != 0 && ld_poly < (int64_t)n * nterm))
    return IM_ERR_STRIDE;
  for (int w0 = 0; w0 < nworld; w0 += 65535) {
    const int nw = nworld - w0 < 65535 ? nworld - w0 : 65535;
    hipLaunchKernelGGL(im::polynomial_damping_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)nw), dim3(256), 0,
                       (hipStream_t)stream, base + (int64_t)w0 * ld_base, ld_base, poly + (int64_t)w0 * ld_poly, ld_poly, nterm,
                       velocity + (int64_t)w0 * ld_velocity, ld_velocity, out + (int64_t)w0 * ld_out, ld_out, n);
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

int im_implicit_qh(const float *M, int64_t ldM, int nM, const int32_t *elem_dof, const float *dof_damping,
                   int64_t ld_damping, float timestep, const int32_t *gaintype, const int32_t *biastype,
                   const float *gainprm, const float *biasprm, int ld_prm, const uint8_t *forcelimited,
                   const float *forcerange, const float *input, int64_t ld_input, const float *force, int64_t ld_force,
                   float *gain, int64_t ld_gain, int nu, const im_row_pair_term *actuators,
                   const im_row_pair_term *tendons, float *qH, int64_t ld_qH, int nworld, void *stream) {
  if (nworld < 0 || nM < 0 || ld_damping < 0 || nu < 0) return IM_ERR_ARG;
  if (nworld == 0 || nM == 0) return IM_OK;
  if (!M || !elem_dof || !dof_damping || !qH) return IM_ERR_ARG;
  if (ldM < nM || ld_qH < nM) return IM_ERR_STRIDE;
  if (nu > 0 && (!gaintype || !biastype || !gainprm || !biasprm || !input || ld_prm < 3)) return IM_ERR_ARG;
  if (nu > 0 && ((forcelimited && !forcerange) || ld_input < nu || (gain && ld_gain < nu) || (force && ld_force < nu)))
    return IM_ERR_ARG;
  im_row_pair_term none{};
  const im_row_pair_term ta = actuators ? *actuators : none, tt = tendons ? *tendons : none;
  int max_entries = 0, max_chunks = 0;
  for (const im_row_pair_term *t : {&ta, &tt}) {
    if (t->nentry < 0 || t->nelem < 0 || t->chunk_count < 0) return IM_ERR_ARG;
    if (t->nentry == 0 || t->nelem == 0) continue;
    if (!t->values || !t->entry_row || !t->elem_ids || !t->chunk_offsets || !t->chunk_pairs) return IM_ERR_ARG;
    if (t->nentry >= 0x7FFF) return IM_ERR_UNSUPPORTED;  // two entry indices share one int32
    max_entries = t->nentry > max_entries ? t->nentry : max_entries;
    max_chunks = t->chunk_count > max_chunks ? t->chunk_count : max_chunks;
  }
  if (ta.nentry > 0 && ta.nelem > 0 && !ta.weight && nu <= 0) return IM_ERR_ARG;  // the gains are its weights
  if (tt.nentry > 0 && tt.nelem > 0 && !tt.weight) return IM_ERR_ARG;
  const size_t lds_bytes = sizeof(float) * ((size_t)nM + nu + 2 * ((size_t)max_entries + 1) + max_chunks);
  if (lds_bytes > 64 * 1024) return IM_ERR_UNSUPPORTED;
  const im::QhGain g{gaintype, biastype, gainprm, biasprm, ld_prm, forcelimited, forcerange, input, ld_input,
                     force, ld_force, gain, ld_gain, nu};
  hipLaunchKernelGGL(im::implicit_qh_kernel, dim3((unsigned)nworld), dim3(256), lds_bytes, (hipStream_t)stream, M, ldM,
                     nM, elem_dof, dof_damping, ld_damping, timestep, g, ta, tt, max_entries, qH, ld_qH);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

}  // extern "C"
