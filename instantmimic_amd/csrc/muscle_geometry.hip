// Muscle path geometry and activation <-> joint-torque contractions for gfx950.
//
//   waypoints[w, i]   = xpos[w, body(i)] + rot(local(i), normalize(xquat[w, body(i)]))
//     reference: src/instantmimic/muscle/muscle_dynamics_kernels.py:73-86
//   unit/passive force magnitudes per (world, muscle) from the polyline length
//     reference: muscle_dynamics_kernels.py:644-705, curves muscle_qfrc_projector.py:103-277
//   torque[w, j]      = sum over the active (segment, muscle) entries of torque dof j of
//                       contribution(segment, dof j, unit * activation (+ passive))
//     reference: muscle_dynamics_kernels.py:1707-1793
//   grad_act[w, m]    = sum over muscle m's (segment, torque) entries of
//                       grad_out[w, j] * contribution(segment, dof j, unit)
//     reference: muscle_dynamics_kernels.py:1796-1859
//   moment[w, e]      = sum over entry e's segments of contribution(segment, dof(e), 1)
//     reference: muscle_qfrc_projector.py:2617-2662
//   contribution      = dot(a (lin + ang x (p0 - c0)) - b (lin + ang x (p1 - c1)), f dir)
//     reference: muscle_qfrc_projector.py:280-304
//
// All five are gathers over a world's row of poses (a few KB, L1/L2 resident after the
// first touch) and write one float per thread; none of them reuses data across worlds, so
// they are HBM bound on the pose rows.  Threads are laid out output-major inside a world
// so that a wavefront's writes coalesce.  Arithmetic is written out operation by operation
// (this file is compiled without floating-point contraction) and the CPU checker follows
// the same order.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>

#include "../../include/imhip.h"
#include "common.h"

namespace im {
namespace {

struct V3 {
  float x, y, z;
};
__device__ __forceinline__ V3 ld3(const float *p) { return {p[0], p[1], p[2]}; }
__device__ __forceinline__ V3 sub(V3 a, V3 b) { return {a.x - b.x, a.y - b.y, a.z - b.z}; }
__device__ __forceinline__ V3 add(V3 a, V3 b) { return {a.x + b.x, a.y + b.y, a.z + b.z}; }
__device__ __forceinline__ V3 scale(float s, V3 a) { return {s * a.x, s * a.y, s * a.z}; }
__device__ __forceinline__ float dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ __forceinline__ V3 cross(V3 a, V3 b) {
  return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ __forceinline__ float length(V3 a) { return sqrtf(dot(a, a)); }

// muscle_qfrc_projector.py:280-304
__device__ __forceinline__ float contribution(V3 lin, V3 ang, V3 p0, V3 p1, V3 c0, V3 c1, float a,
                                              float b, float force) {
  const V3 seg = sub(p1, p0);
  const float len = length(seg);
  if (len < 1.0e-8f) return 0.0f;
  const V3 dir = {seg.x / len, seg.y / len, seg.z / len};
  const V3 f = scale(force, dir);
  const V3 st = add(lin, cross(ang, sub(p0, c0)));
  const V3 en = add(lin, cross(ang, sub(p1, c1)));
  return dot(sub(scale(a, st), scale(b, en)), f);
}

struct Geo {
  const float *wp, *com, *cdof;
  int64_t ldw, ldc, ldd;
};
struct Seg {
  const int32_t *p0, *p1, *b0, *b1;
};

__device__ __forceinline__ float seg_term(const Geo &g, const Seg &s, int64_t w, int seg, V3 lin,
                                          V3 ang, float a, float b, float force) {
  const float *wp = g.wp + w * g.ldw, *com = g.com + w * g.ldc;
  return contribution(lin, ang, ld3(wp + 3 * s.p0[seg]), ld3(wp + 3 * s.p1[seg]),
                      ld3(com + 3 * s.b0[seg]), ld3(com + 3 * s.b1[seg]), a, b, force);
}

// One waypoint in the world frame: the body's position plus its local offset turned by the
// body's (renormalised) quaternion.  xpos and xquat are one world's rows.
__device__ __forceinline__ V3 world_waypoint(const float *__restrict__ xpos,
                                             const float *__restrict__ xquat,
                                             const int32_t *__restrict__ wp_body,
                                             const float *__restrict__ wp_local, int i) {
  const int b = wp_body[i];
  const float *q = xquat + 4 * b;
  const float q0 = q[0], q1 = q[1], q2 = q[2], q3 = q[3];
  // muscle_qfrc_projector.py:91-100
  const float inv = 1.0f / sqrtf(q0 * q0 + q1 * q1 + q2 * q2 + q3 * q3 + 1.0e-8f);
  const float s = q0 * inv;
  const V3 u = {q1 * inv, q2 * inv, q3 * inv};
  const V3 v = ld3(wp_local + 3 * i);
  // mujoco_warp math.rot_vec_quat: 2 (u.v) u + (s s - u.u) v + 2 s (u x v)
  V3 r = add(scale(2.0f, scale(dot(u, v), u)), scale(s * s - dot(u, u), v));
  r = add(r, scale(2.0f * s, cross(u, v)));
  return add(ld3(xpos + 3 * b), r);
}

__global__ __launch_bounds__(256) void waypoints_kernel(
    const float *__restrict__ xpos, int64_t ldp, const float *__restrict__ xquat, int64_t ldq,
    const int32_t *__restrict__ wp_body, const float *__restrict__ wp_local, int nwp,
    float *__restrict__ out, int64_t ldo, int nworld) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (i >= nwp) return;
  const V3 p = world_waypoint(xpos + w * ldp, xquat + w * ldq, wp_body, wp_local, i);
  float *o = out + w * ldo + 3 * i;
  o[0] = p.x;
  o[1] = p.y;
  o[2] = p.z;
}

// muscle_qfrc_projector.py:103-187
__device__ __forceinline__ float active_fl(float l, const float *m) {
  if (m[0] < 0.5f) return expf(-((l - 1.0f) * (l - 1.0f)) / m[1]);
  const float lmin = m[1], lmax = m[2];
  if (l < lmin || l > lmax) return 0.0f;
  const float lo = 0.5f * (lmin + 1.0f), hi = 0.5f * (1.0f + lmax);
  if (l <= lo) {
    const float x = (l - lmin) / fmaxf(lo - lmin, 1.0e-8f);
    return 0.5f * x * x;
  }
  if (l <= 1.0f) {
    const float x = (1.0f - l) / fmaxf(1.0f - lo, 1.0e-8f);
    return 1.0f - 0.5f * x * x;
  }
  if (l <= hi) {
    const float x = (l - 1.0f) / fmaxf(hi - 1.0f, 1.0e-8f);
    return 1.0f - 0.5f * x * x;
  }
  const float x = (lmax - l) / fmaxf(lmax - hi, 1.0e-8f);
  return 0.5f * x * x;
}
__device__ __forceinline__ float passive_fl(float l, const float *m) {
  if (m[0] < 0.5f) {
    if (l < 1.0f) return 0.0f;
    float x = m[1] * (l - 1.0f) / m[2];
    x = fminf(fmaxf(x, -80.0f), 80.0f);
    return (expf(x) - 1.0f) / (expf(m[1]) - 1.0f);
  }
  const float lmax = m[1], fpmax = m[2];
  if (l <= 1.0f) return 0.0f;
  const float mid = 0.5f * (1.0f + lmax), width = fmaxf(mid - 1.0f, 1.0e-8f);
  if (l <= mid) {
    const float st = (l - 1.0f) / width;
    return 0.5f * fpmax * st * st;
  }
  return fpmax * (0.5f + (l - mid) / width);
}

// Length of muscle m along one world's waypoints and its force magnitudes.
__device__ __forceinline__ void muscle_force_magnitudes(
    const float *row, const int32_t *__restrict__ seg_start,
    const int32_t *__restrict__ seg_offsets, const float *__restrict__ params, int ldpar,
    const float *__restrict__ rest, const im_muscle_force_model &model, int m, float *unit,
    float *passive) {
  float len = 0.0f;  // muscle_dynamics_kernels.py:452-473
  for (int s = seg_offsets[m]; s < seg_offsets[m + 1]; ++s) {
    const int i = seg_start[s];
    len = len + length(sub(ld3(row + 3 * (i + 1)), ld3(row + 3 * i)));
  }
  const float f0 = params[m * ldpar], lm0 = params[m * ldpar + 1], lt0 = params[m * ldpar + 2],
              pen = params[m * ldpar + 3];
  // muscle_qfrc_projector.py:190-205
  const float lm = len / fmaxf(rest[m], 1.0e-6f) - lt0;
  const float ln =
      fminf(fmaxf(lm / fmaxf(lm0, 1.0e-6f), model.length_norm_min), model.length_norm_max);
  const float c = cosf(pen);
  *unit = f0 * active_fl(ln, model.active) * c * model.force_scale;
  if (passive) {
    float pv = 0.0f;
    // muscle_qfrc_projector.py:249-277 with include_active 0, include_passive 1
    if (model.include_passive)
      pv = f0 * passive_fl(ln, model.passive) * c * model.force_scale;
    *passive = pv;
  }
}

// MuJoCo's force-velocity multiplier and its derivative in the normalised velocity
// (muscle_qfrc_projector.py:2505-2524)
__device__ __forceinline__ void force_velocity_curve(float v, float fvmax, float *mult, float *slope) {
  const float y = fvmax - 1.0f;
  if (v <= -1.0f) {
    *mult = 0.0f;
    *slope = 0.0f;
  } else if (v <= 0.0f) {
    const float shifted = v + 1.0f;
    *mult = shifted * shifted;
    *slope = 2.0f * shifted;
  } else if (v <= y) {
    const float remaining = y - v;
    *mult = fvmax - remaining * remaining / y;
    *slope = 2.0f * remaining / y;
  } else {
    *mult = fvmax;
    *slope = 0.0f;
  }
}

// eval_muscle_force_velocity_state_kernel (muscle_qfrc_projector.py:2816-2884): one muscle of
// one world -- its length over consecutive waypoints, its lengthening velocity -sum moment qvel
// over its (muscle, dof) entries, and the force-velocity response (:2528-2570).
__global__ __launch_bounds__(256) void force_velocity_state_kernel(
    const float *__restrict__ wp, int64_t ldw, const int32_t *__restrict__ waypoint_start,
    const float *__restrict__ params, int ldpar, const float *__restrict__ rest,
    const float *__restrict__ length_scale, const float *__restrict__ activation, int64_t lda,
    const float *__restrict__ qvel, int64_t ldq, const float *__restrict__ moment, int64_t ldm,
    const int32_t *__restrict__ dof_offsets, const int32_t *__restrict__ dof_torque_idx, int root,
    im_muscle_force_model model, im_muscle_force_velocity_model fv, int nmuscle, float *__restrict__ out_length,
    float *__restrict__ out_activation, float *__restrict__ out_velocity, float *__restrict__ out_multiplier,
    float *__restrict__ out_slope, int64_t ldo) {
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (m >= nmuscle) return;
  const float *row = wp + w * ldw;
  float len = 0.0f;
  for (int i = waypoint_start[m]; i < waypoint_start[m + 1] - 1; ++i)
    len = len + length(sub(ld3(row + 3 * (i + 1)), ld3(row + 3 * i)));
  float velocity = 0.0f;
  for (int e = dof_offsets[m]; e < dof_offsets[m + 1]; ++e)
    velocity = __builtin_fmaf(-moment[w * ldm + e], qvel[w * ldq + dof_torque_idx[e] + root], velocity);
  const float f0 = params[m * ldpar], lm0 = params[m * ldpar + 1], lt0 = params[m * ldpar + 2],
              pen = params[m * ldpar + 3];
  const float velocity_scale = fmaxf(length_scale[m] * fv.vmax, 1.0e-6f);
  float mult, dmult;
  force_velocity_curve(velocity / velocity_scale, fv.fvmax, &mult, &dmult);
  float active = activation[w * lda + m];
  if (fv.clamp_activation != 0.0f) active = fminf(fmaxf(active, 0.0f), 1.0f);
  const float lm = len / fmaxf(rest[m], 1.0e-6f) - lt0;
  const float ln = fminf(fmaxf(lm / fmaxf(lm0, 1.0e-6f), model.length_norm_min), model.length_norm_max);
  const float unit = f0 * active_fl(ln, model.active) * cosf(pen) * model.force_scale;
  out_length[w * ldo + m] = len;
  out_activation[w * ldo + m] = active * mult;
  out_velocity[w * ldo + m] = velocity;
  out_multiplier[w * ldo + m] = mult;
  out_slope[w * ldo + m] = fv.include_active * active * unit * dmult / velocity_scale;
}

// The same per world in one workgroup: the world's waypoints, moment entries and velocities come
// into LDS with coalesced loads (a lane of the kernel above walks a few 12-byte waypoints and a
// few scattered entries of its own, a cache line per request), then every muscle reads LDS.  Same
// operations in the same order, so the same bits.  nwords_wp / nentry: what is staged (the
// arrays' row lengths).
__global__ __launch_bounds__(256) void force_velocity_state_world_kernel(
    const float *__restrict__ wp, int64_t ldw, int nwords_wp, const int32_t *__restrict__ waypoint_start,
    const float *__restrict__ params, int ldpar, const float *__restrict__ rest,
    const float *__restrict__ length_scale, const float *__restrict__ activation, int64_t lda,
    const float *__restrict__ qvel, int64_t ldq, int nqvel, const float *__restrict__ moment, int64_t ldm, int nentry,
    const int32_t *__restrict__ dof_offsets, const int32_t *__restrict__ dof_torque_idx, int root,
    im_muscle_force_model model, im_muscle_force_velocity_model fv, int nmuscle, float *__restrict__ out_length,
    float *__restrict__ out_activation, float *__restrict__ out_velocity, float *__restrict__ out_multiplier,
    float *__restrict__ out_slope, int64_t ldo) {
  extern __shared__ float fv_lds[];
  float *row = fv_lds;            // [nwords_wp]
  float *mom = row + nwords_wp;   // [nentry]
  float *qv = mom + nentry;       // [nqvel]
  const int64_t w = blockIdx.x;
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int i = tid; i < nwords_wp; i += nt) row[i] = wp[w * ldw + i];
  for (int i = tid; i < nentry; i += nt) mom[i] = moment[w * ldm + i];
  for (int i = tid; i < nqvel; i += nt) qv[i] = qvel[w * ldq + i];
  __syncthreads();
  for (int m = tid; m < nmuscle; m += nt) {
    float len = 0.0f;
    for (int i = waypoint_start[m]; i < waypoint_start[m + 1] - 1; ++i)
      len = len + length(sub(ld3(row + 3 * (i + 1)), ld3(row + 3 * i)));
    float velocity = 0.0f;
    for (int e = dof_offsets[m]; e < dof_offsets[m + 1]; ++e)
      velocity = __builtin_fmaf(-mom[e], qv[dof_torque_idx[e] + root], velocity);
    const float f0 = params[m * ldpar], lm0 = params[m * ldpar + 1], lt0 = params[m * ldpar + 2],
                pen = params[m * ldpar + 3];
    const float velocity_scale = fmaxf(length_scale[m] * fv.vmax, 1.0e-6f);
    float mult, dmult;
    force_velocity_curve(velocity / velocity_scale, fv.fvmax, &mult, &dmult);
    float active = activation[w * lda + m];
    if (fv.clamp_activation != 0.0f) active = fminf(fmaxf(active, 0.0f), 1.0f);
    const float lm = len / fmaxf(rest[m], 1.0e-6f) - lt0;
    const float ln = fminf(fmaxf(lm / fmaxf(lm0, 1.0e-6f), model.length_norm_min), model.length_norm_max);
    const float unit = f0 * active_fl(ln, model.active) * cosf(pen) * model.force_scale;
    out_length[w * ldo + m] = len;
    out_activation[w * ldo + m] = active * mult;
    out_velocity[w * ldo + m] = velocity;
    out_multiplier[w * ldo + m] = mult;
    out_slope[w * ldo + m] = fv.include_active * active * unit * dmult / velocity_scale;
  }
}

__global__ __launch_bounds__(256) void force_kernel(
    const float *__restrict__ wp, int64_t ldw, const int32_t *__restrict__ seg_start,
    const int32_t *__restrict__ seg_offsets, const float *__restrict__ params, int ldpar,
    const float *__restrict__ rest, im_muscle_force_model model, int nmuscle,
    float *__restrict__ unit, int64_t ldu, float *__restrict__ passive, int64_t ldpa) {
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (m >= nmuscle) return;
  muscle_force_magnitudes(wp + w * ldw, seg_start, seg_offsets, params, ldpar, rest, model, m,
                          unit + w * ldu + m, passive ? passive + w * ldpa + m : nullptr);
}

// Waypoints and force magnitudes of one world in one workgroup: the waypoints go to memory and
// stay in LDS, from where the muscle lengths are taken.  Same operations as the two kernels
// above, so the results are theirs bit for bit.
__global__ __launch_bounds__(512) void waypoints_forces_kernel(
    const float *__restrict__ xpos, int64_t ldp, const float *__restrict__ xquat, int64_t ldq,
    const int32_t *__restrict__ wp_body, const float *__restrict__ wp_local, int nwp,
    float *__restrict__ out, int64_t ldo, const int32_t *__restrict__ seg_start,
    const int32_t *__restrict__ seg_offsets, const float *__restrict__ params, int ldpar,
    const float *__restrict__ rest, im_muscle_force_model model, int nmuscle,
    float *__restrict__ unit, int64_t ldu, float *__restrict__ passive, int64_t ldpa) {
  extern __shared__ float wpl[];  // [3 * nwp]
  const int64_t w = blockIdx.x;
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int i = tid; i < nwp; i += nt) {
    const V3 p = world_waypoint(xpos + w * ldp, xquat + w * ldq, wp_body, wp_local, i);
    wpl[3 * i] = p.x;
    wpl[3 * i + 1] = p.y;
    wpl[3 * i + 2] = p.z;
  }
  __syncthreads();
  float *o = out + w * ldo;
  for (int k = tid; k < 3 * nwp; k += nt) o[k] = wpl[k];
  for (int m = tid; m < nmuscle; m += nt)
    muscle_force_magnitudes(wpl, seg_start, seg_offsets, params, ldpar, rest, model, m,
                            unit + w * ldu + m, passive ? passive + w * ldpa + m : nullptr);
}

__global__ __launch_bounds__(256) void torque_forward_kernel(
    Geo g, Seg s, const int32_t *__restrict__ offsets, const int32_t *__restrict__ e_seg,
    const int32_t *__restrict__ e_muscle, const float *__restrict__ e_a,
    const float *__restrict__ e_b, const float *__restrict__ unit, int64_t ldu,
    const float *__restrict__ passive, int64_t ldpa, const float *__restrict__ act, int64_t lda,
    int root, int ntorque, float *__restrict__ out, int64_t ldo) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (j >= ntorque) return;
  const float *cd = g.cdof + w * g.ldd + 6 * (int64_t)(j + root);
  const V3 ang = ld3(cd), lin = ld3(cd + 3);
  float total = 0.0f;
  for (int e = offsets[j]; e < offsets[j + 1]; ++e) {
    const int m = e_muscle[e];
    float f = unit[w * ldu + m] * act[w * lda + m];
    if (passive) f = f + passive[w * ldpa + m];
    if (f == 0.0f) continue;
    total = total + seg_term(g, s, w, e_seg[e], lin, ang, e_a[e], e_b[e], f);
  }
  out[w * ldo + j] = total;
}

__global__ __launch_bounds__(256) void activation_grad_kernel(
    Geo g, Seg s, const int32_t *__restrict__ offsets, const int32_t *__restrict__ e_seg,
    const int32_t *__restrict__ e_torque, const float *__restrict__ e_a,
    const float *__restrict__ e_b, const float *__restrict__ unit, int64_t ldu,
    const float *__restrict__ gout, int64_t ldg, int root, int nmuscle, float *__restrict__ gact,
    int64_t lda) {
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (m >= nmuscle) return;
  const float f = unit[w * ldu + m];
  float grad = 0.0f;
  // The reference returns before the store when f == 0 and relies on a zero-filled
  // output (muscle_dynamics_kernels.py:1817-1819); the store of 0 here is the same value.
  if (f != 0.0f) {
    for (int e = offsets[m]; e < offsets[m + 1]; ++e) {
      const int j = e_torque[e];
      const float *cd = g.cdof + w * g.ldd + 6 * (int64_t)(j + root);
      grad = grad + gout[w * ldg + j] *
                        seg_term(g, s, w, e_seg[e], ld3(cd + 3), ld3(cd), e_a[e], e_b[e], f);
    }
  }
  gact[w * lda + m] = grad;
}

__global__ __launch_bounds__(256) void sparse_moment_kernel(
    Geo g, Seg s, const int32_t *__restrict__ entry_torque, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ e_seg, const float *__restrict__ e_a,
    const float *__restrict__ e_b, int root, int nentry, float *__restrict__ moment, int64_t ldm) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (e >= nentry) return;
  const float *cd = g.cdof + w * g.ldd + 6 * (int64_t)(entry_torque[e] + root);
  const V3 ang = ld3(cd), lin = ld3(cd + 3);
  float total = 0.0f;
  for (int k = offsets[e]; k < offsets[e + 1]; ++k)
    total = total + seg_term(g, s, w, e_seg[k], lin, ang, e_a[k], e_b[k], 1.0f);
  moment[w * ldm + e] = total;
}

// Feasible torque box over activations in [0, 1]: per torque dof the entries are grouped by
// muscle (consecutive entries of one muscle); a muscle's total goes to the lower bound when
// negative, else to the upper (muscle_dynamics_kernels.py:1453-1528).
__global__ __launch_bounds__(256) void torque_bounds_kernel(
    Geo g, Seg s, const int32_t *__restrict__ offsets, const int32_t *__restrict__ e_seg,
    const int32_t *__restrict__ e_muscle, const float *__restrict__ e_a,
    const float *__restrict__ e_b, const float *__restrict__ unit, int64_t ldu, int root,
    int ntorque, float *__restrict__ lower, float *__restrict__ upper, int64_t ldo) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t w = blockIdx.y;
  if (j >= ntorque) return;
  const float *cd = g.cdof + w * g.ldd + 6 * (int64_t)(j + root);
  const V3 ang = ld3(cd), lin = ld3(cd + 3);
  int current = -1;
  float total = 0.0f, lo = 0.0f, hi = 0.0f;
  for (int e = offsets[j]; e < offsets[j + 1]; ++e) {
    const int m = e_muscle[e];
    if (current >= 0 && m != current) {
      if (total < 0.0f) lo = lo + total;
      else hi = hi + total;
      total = 0.0f;
    }
    current = m;
    total = total + seg_term(g, s, w, e_seg[e], lin, ang, e_a[e], e_b[e], unit[w * ldu + m]);
  }
  if (current >= 0) {
    if (total < 0.0f) lo = lo + total;
    else hi = hi + total;
  }
  lower[w * ldo + j] = lo;
  upper[w * ldo + j] = hi;
}

// ---- one workgroup per world --------------------------------------------------------------
// One workgroup of 512 threads per world (three of them share a CU at the 553-segment rig's
// 49 KB of LDS; 384, 640, 768 and 1024 threads measured 2 - 7 % slower there).
// The four contractions above visit every applied segment once per (segment, dof) entry and
// redo its square root and three divisions each time, and they fetch a muscle's force and a
// dof's motion axis from memory once per entry.  Here a workgroup first leaves in LDS each
// segment's unit direction and its two lever vectors, every muscle's force and every torque
// dof's axis; then every thread evaluates entries (same operations, same order as
// contribution()), and a last pass adds each output's entries in list order, reading them
// several at a time so that only the additions wait on one another.  Results equal the
// one-thread-per-output kernels bit for bit.
enum { MW_FORWARD, MW_GRAD, MW_BOUNDS, MW_MOMENT };

struct MwArgs {
  Geo g;
  Seg s;
  const int32_t *offsets, *e_seg, *e_other, *row_torque;  // row_torque: MW_MOMENT only
  const float *e_a, *e_b;
  const float *unit, *passive, *act, *gout;
  int64_t ldu, ldpa, lda, ldg;
  float *out0, *out1;
  int64_t ldo;
  int root, nrow, nentry, nseg;
  int ntorque, nmuscle;  // sizes of the staged axes and forces (nmuscle 0 for MW_MOMENT)
};

constexpr int kContribPad = 4;  // floats read past the last entry by ordered_sum()
struct MwLds {
  float *segd;     // [nseg][9]: dir (0 for a degenerate segment), p0 - c0, p1 - c1
  float *contrib;  // [nentry]
  float *axis;     // [ntorque][6]: the dof's cdof
  float *force;    // [nmuscle]: force of a muscle as the contraction sees it
  float *gout;     // [ntorque], MW_GRAD only
  unsigned short *rowid;  // [nentry]
};
template <int MODE>
__host__ __device__ inline size_t mw_lds_floats(const MwArgs &a) {
  return (size_t)9 * a.nseg + (size_t)a.nentry + kContribPad + (size_t)6 * a.ntorque + (size_t)a.nmuscle +
         (MODE == MW_GRAD ? (size_t)a.ntorque : 0);
}

// What the lists hold about one entry.
struct MwEntry {
  int row, other, seg;
  float a, b;
};
template <int MODE>
__device__ __forceinline__ MwEntry load_entry(const MwArgs &a, const MwLds &l, int e) {
  MwEntry t;
  t.row = l.rowid[e];
  t.other = MODE == MW_MOMENT ? 0 : a.e_other[e];
  t.seg = a.e_seg[e];
  t.a = a.e_a[e];
  t.b = a.e_b[e];
  return t;
}

template <int MODE>
__device__ __forceinline__ float entry_contribution(const MwArgs &a, const MwLds &l, const MwEntry &t) {
  int torque, muscle;
  if (MODE == MW_GRAD) { muscle = t.row; torque = t.other; }
  else if (MODE == MW_MOMENT) { muscle = 0; torque = a.row_torque[t.row]; }
  else { torque = t.row; muscle = t.other; }
  float f = 1.0f;
  if (MODE != MW_MOMENT) f = l.force[muscle];
  const float *cd = l.axis + 6 * torque;
  const V3 ang = ld3(cd), lin = ld3(cd + 3);
  const float *sd = l.segd + 9 * t.seg;
  const V3 dir = {sd[0], sd[1], sd[2]}, r0 = {sd[3], sd[4], sd[5]}, r1 = {sd[6], sd[7], sd[8]};
  const V3 fv = scale(f, dir);
  const V3 st = add(lin, cross(ang, r0));
  const V3 en = add(lin, cross(ang, r1));
  float c = dot(sub(scale(t.a, st), scale(t.b, en)), fv);
  // evaluated for every entry, without a branch around it: a thread's entries then proceed
  // side by side instead of one after the other
  asm volatile("" : "+v"(c));
  // an entry whose force is zero is skipped by the reference: it enters the sum as 0
  c = f == 0.0f ? 0.0f : c;
  if (MODE == MW_GRAD) c = l.gout[torque] * c;
  return c;
}

// Sum of contrib[e0..e1) in list order from +0.  Whole groups of 16 (LONG) and of 4 entries are
// read with one address and added without a test; the last group reads up to three floats past
// e1 (contrib is padded for that) and enters them as +0, which leaves every bit of a sum that
// started at +0 (such a sum is never -0).
template <bool LONG>
__device__ __forceinline__ float ordered_sum(const float *contrib, int e0, int e1) {
  float total = 0.0f;
  int e = e0;
  if (LONG) {
    for (; e + 16 <= e1; e += 16) {
      float c[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) c[k] = contrib[e + k];
#pragma unroll
      for (int k = 0; k < 16; ++k) total = total + c[k];
    }
  }
  for (; e + 4 <= e1; e += 4) {
    float c[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) c[k] = contrib[e + k];
#pragma unroll
    for (int k = 0; k < 4; ++k) total = total + c[k];
  }
  if (e < e1) {
    float c[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) c[k] = contrib[e + k];
#pragma unroll
    for (int k = 0; k < 3; ++k) total = total + (e + k < e1 ? c[k] : 0.0f);
  }
  return total;
}

template <int MODE>
__global__ __launch_bounds__(1024) void muscle_world_kernel(MwArgs a) {
  extern __shared__ float lds[];
  MwLds l;
  l.segd = lds;
  l.contrib = l.segd + 9 * a.nseg;
  l.axis = l.contrib + a.nentry + kContribPad;
  l.force = l.axis + 6 * a.ntorque;
  l.gout = l.force + a.nmuscle;
  l.rowid = (unsigned short *)(lds + mw_lds_floats<MODE>(a));
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t w = blockIdx.x;
  const float *wp = a.g.wp + w * a.g.ldw, *com = a.g.com + w * a.g.ldc, *cdof = a.g.cdof + w * a.g.ldd;
  for (int sg = tid; sg < a.nseg; sg += nt) {
    const V3 p0 = ld3(wp + 3 * a.s.p0[sg]), p1 = ld3(wp + 3 * a.s.p1[sg]);
    const V3 c0 = ld3(com + 3 * a.s.b0[sg]), c1 = ld3(com + 3 * a.s.b1[sg]);
    const V3 seg = sub(p1, p0);
    const float len = length(seg);
    const bool ok = !(len < 1.0e-8f);
    const V3 r0 = sub(p0, c0), r1 = sub(p1, c1);
    // a degenerate segment contributes nothing: with a zero direction its entries come out as
    // +-0, and adding +-0 to a sum that started at +0 leaves every bit of it
    float *o = l.segd + 9 * sg;
    o[0] = ok ? seg.x / len : 0.0f;
    o[1] = ok ? seg.y / len : 0.0f;
    o[2] = ok ? seg.z / len : 0.0f;
    o[3] = r0.x; o[4] = r0.y; o[5] = r0.z;
    o[6] = r1.x; o[7] = r1.y; o[8] = r1.z;
  }
  for (int i = tid; i < 6 * a.ntorque; i += nt) l.axis[i] = cdof[6 * a.root + i];
  for (int m = tid; m < a.nmuscle; m += nt) {
    float f = a.unit[w * a.ldu + m];
    if (MODE == MW_FORWARD) {
      f = f * a.act[w * a.lda + m];
      if (a.passive) f = f + a.passive[w * a.ldpa + m];
    }
    l.force[m] = f;
  }
  if (MODE == MW_GRAD)
    for (int j = tid; j < a.ntorque; j += nt) l.gout[j] = a.gout[w * a.ldg + j];
  if (a.nentry < 32 * a.nrow) {  // short rows: a thread writes its row's
    for (int r = tid; r < a.nrow; r += nt)
      for (int e = a.offsets[r]; e < a.offsets[r + 1]; ++e) l.rowid[e] = (unsigned short)r;
  } else {  // long rows: a wave writes a row's
    for (int r = tid >> 6; r < a.nrow; r += nt >> 6)
      for (int e = a.offsets[r] + (tid & 63); e < a.offsets[r + 1]; e += 64) l.rowid[e] = (unsigned short)r;
  }
  __syncthreads();
  // four entries per thread and trip while whole trips remain (all their loads are issued
  // before the first is needed), then one entry per thread
  int base = 0;
  for (; base + 4 * nt <= a.nentry; base += 4 * nt) {
    MwEntry t[4];
    float c[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) t[k] = load_entry<MODE>(a, l, base + k * nt + tid);
#pragma unroll
    for (int k = 0; k < 4; ++k) c[k] = entry_contribution<MODE>(a, l, t[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) l.contrib[base + k * nt + tid] = c[k];
  }
  for (int e = base + tid; e < a.nentry; e += nt)
    l.contrib[e] = entry_contribution<MODE>(a, l, load_entry<MODE>(a, l, e));
  __syncthreads();
  const float *contrib = l.contrib;
  for (int r = tid; r < a.nrow; r += nt) {
    const int e0 = a.offsets[r], e1 = a.offsets[r + 1];
    if (MODE == MW_FORWARD) {
      a.out0[w * a.ldo + r] = ordered_sum<true>(contrib, e0, e1);
    } else if (MODE == MW_MOMENT) {  // a (muscle, dof) pair has a few segments
      a.out0[w * a.ldo + r] = ordered_sum<false>(contrib, e0, e1);
    } else if (MODE == MW_GRAD) {
      // The one-thread-per-muscle kernel leaves 0 for a muscle without force; its entries are
      // 0 here as well (gout * 0), but an infinite gout would turn them into NaN
      a.out0[w * a.ldo + r] = l.force[r] != 0.0f ? ordered_sum<true>(contrib, e0, e1) : 0.0f;
    } else {
      int current = -1;
      float total = 0.0f, lo = 0.0f, hi = 0.0f;
      for (int e = e0; e < e1; ++e) {
        const int m = a.e_other[e];
        if (current >= 0 && m != current) {
          if (total < 0.0f) lo = lo + total;
          else hi = hi + total;
          total = 0.0f;
        }
        current = m;
        total = total + contrib[e];
      }
      if (current >= 0) {
        if (total < 0.0f) lo = lo + total;
        else hi = hi + total;
      }
      a.out0[w * a.ldo + r] = lo;
      a.out1[w * a.ldo + r] = hi;
    }
  }
}

// Launches the workgroup-per-world kernel when a world's segments and entries fit in LDS and
// the entry list states the range of its `other` column; returns false for the caller to use
// the one-thread-per-output kernel instead.
template <int MODE>
bool launch_world(const MwArgs &a, int nworld, hipStream_t stream) {
  const size_t lds_bytes = 4 * mw_lds_floats<MODE>(a) + 2 * (((size_t)a.nentry + 1) & ~(size_t)1);
  static const bool forced_off = [] {
    const char *e = std::getenv("IMHIP_MUSCLE_KERNEL");
    return e && std::strcmp(e, "simple") == 0;
  }();
  if (forced_off || lds_bytes > 64 * 1024 || a.nentry == 0 || a.nseg == 0 || a.nrow > 65535 ||
      a.ntorque <= 0 || (MODE != MW_MOMENT && a.nmuscle <= 0))
    return false;
  hipLaunchKernelGGL(muscle_world_kernel<MODE>, dim3((unsigned)nworld), dim3(512), lds_bytes, stream, a);
  return true;
}

bool geo_ok(const im_muscle_geometry *g) {
  return g && g->waypoints && g->subtree_com && g->cdof && g->ld_waypoints >= 0 &&
         g->ld_subtree_com >= 0 && g->ld_cdof >= 0;
}
bool seg_ok(const im_muscle_segments *s) {
  return s && s->start_waypoint && s->end_waypoint && s->start_root_body && s->end_root_body;
}
Geo geo(const im_muscle_geometry *g) {
  return {g->waypoints, g->subtree_com, g->cdof, g->ld_waypoints, g->ld_subtree_com, g->ld_cdof};
}
Seg seg(const im_muscle_segments *s) {
  return {s->start_waypoint, s->end_waypoint, s->start_root_body, s->end_root_body};
}
dim3 grid2(int n, int nworld) { return dim3((unsigned)((n + 255) / 256), (unsigned)nworld); }
constexpr int kMaxGridY = 65535;
int slab_count(int nworld, int w0) { return nworld - w0 < kMaxGridY ? nworld - w0 : kMaxGridY; }

}  // namespace
}  // namespace im

using namespace im;

// The y dimension of a grid carries the world; launches are split so that it stays within
// the limit of 65535.
#define IM_FOR_WORLD_SLABS(nworld, w0, nw)                                     \
  for (int w0 = 0, nw = slab_count(nworld, 0); w0 < (nworld); \
       w0 += kMaxGridY, nw = slab_count(nworld, w0))

extern "C" int im_muscle_waypoints(const float *xpos, int64_t ld_xpos, const float *xquat,
                                   int64_t ld_xquat, const int32_t *waypoint_body,
                                   const float *waypoint_local, int nwaypoint, float *waypoints,
                                   int64_t ld_waypoints, int nworld, void *stream) {
  if (nworld < 0 || nwaypoint < 0) return IM_ERR_ARG;
  if (nworld == 0 || nwaypoint == 0) return IM_OK;
  if (!xpos || !xquat || !waypoint_body || !waypoint_local || !waypoints) return IM_ERR_ARG;
  if (ld_waypoints < 3 * (int64_t)nwaypoint) return IM_ERR_STRIDE;
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(waypoints_kernel, grid2(nwaypoint, nw), dim3(256), 0, (hipStream_t)stream,
                       xpos + w0 * ld_xpos, ld_xpos, xquat + w0 * ld_xquat, ld_xquat,
                       waypoint_body, waypoint_local, nwaypoint, waypoints + w0 * ld_waypoints,
                       ld_waypoints, nw);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_force_magnitudes(const float *waypoints, int64_t ld_waypoints,
                                          const int32_t *all_segment_start_idx,
                                          const int32_t *all_muscle_segment_offsets,
                                          const float *muscle_params, int ld_params,
                                          const float *muscle_rest_length,
                                          const im_muscle_force_model *model, int nmuscle,
                                          float *unit_force, int64_t ld_unit,
                                          float *passive_force, int64_t ld_passive, int nworld,
                                          void *stream) {
  if (nworld < 0 || nmuscle < 0 || !model) return IM_ERR_ARG;
  if (nworld == 0 || nmuscle == 0) return IM_OK;
  if (!waypoints || !all_segment_start_idx || !all_muscle_segment_offsets || !muscle_params ||
      !muscle_rest_length || !unit_force || ld_params < 4)
    return IM_ERR_ARG;
  if (ld_unit < nmuscle || (passive_force && ld_passive < nmuscle)) return IM_ERR_STRIDE;
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(force_kernel, grid2(nmuscle, nw), dim3(256), 0, (hipStream_t)stream,
                       waypoints + w0 * ld_waypoints, ld_waypoints, all_segment_start_idx,
                       all_muscle_segment_offsets, muscle_params, ld_params, muscle_rest_length,
                       *model, nmuscle, unit_force + w0 * ld_unit, ld_unit,
                       passive_force ? passive_force + w0 * ld_passive : nullptr, ld_passive);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_force_velocity_state(
    const float *waypoints, int64_t ld_waypoints, const int32_t *muscle_waypoint_start,
    const float *muscle_params, int ld_params, const float *muscle_rest_length,
    const float *force_velocity_length_scale, const float *activation, int64_t ld_activation,
    const float *qvel, int64_t ld_qvel, const float *moment, int64_t ld_moment,
    const int32_t *muscle_dof_offsets, const int32_t *muscle_dof_torque_idx, int root_dof_count,
    const im_muscle_force_model *model, const im_muscle_force_velocity_model *fv, int nmuscle,
    float *muscle_length, float *effective_activation, float *length_velocity,
    float *force_velocity_multiplier, float *force_velocity_slope, int64_t ld_out, int nworld, void *stream) {
  if (nworld < 0 || nmuscle < 0 || root_dof_count < 0) return IM_ERR_ARG;
  if (nworld == 0 || nmuscle == 0) return IM_OK;
  if (!waypoints || !muscle_waypoint_start || !muscle_params || !muscle_rest_length ||
      !force_velocity_length_scale || !activation || !qvel || !moment || !muscle_dof_offsets ||
      !muscle_dof_torque_idx || !model || !fv || !muscle_length || !effective_activation || !length_velocity ||
      !force_velocity_multiplier || !force_velocity_slope || ld_params < 4)
    return IM_ERR_ARG;
  if (ld_out < nmuscle || ld_activation < nmuscle) return IM_ERR_STRIDE;
  // a world's rows of waypoints, moments and velocities staged in LDS when they fit (the rows'
  // strides bound what the tables can address); IMHIP_MUSCLE_KERNEL=simple keeps the lane-per-muscle kernel
  static const bool forced_off = [] {
    const char *e = std::getenv("IMHIP_MUSCLE_KERNEL");
    return e && std::strcmp(e, "simple") == 0;
  }();
  const int64_t staged_words = ld_waypoints + ld_moment + ld_qvel;
  if (!forced_off && ld_waypoints > 0 && ld_moment > 0 && ld_qvel > 0 && staged_words * 4 <= 64 * 1024) {
    const int threads = 256;  // measured at 284 muscles: 45 us; 192 threads (two even passes) 49 us, 320 (one pass) 52 us
    hipLaunchKernelGGL(force_velocity_state_world_kernel, dim3((unsigned)nworld), dim3(threads), (size_t)staged_words * 4,
                       (hipStream_t)stream, waypoints, ld_waypoints, (int)ld_waypoints, muscle_waypoint_start,
                       muscle_params, ld_params, muscle_rest_length, force_velocity_length_scale, activation,
                       ld_activation, qvel, ld_qvel, (int)ld_qvel, moment, ld_moment, (int)ld_moment, muscle_dof_offsets,
                       muscle_dof_torque_idx, root_dof_count, *model, *fv, nmuscle, muscle_length, effective_activation,
                       length_velocity, force_velocity_multiplier, force_velocity_slope, ld_out);
    IM_HIP_CHECK(hipGetLastError());
    return IM_OK;
  }
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(force_velocity_state_kernel, grid2(nmuscle, nw), dim3(256), 0, (hipStream_t)stream,
                       waypoints + w0 * ld_waypoints, ld_waypoints, muscle_waypoint_start, muscle_params, ld_params,
                       muscle_rest_length, force_velocity_length_scale, activation + w0 * ld_activation,
                       ld_activation, qvel + w0 * ld_qvel, ld_qvel, moment + w0 * ld_moment, ld_moment,
                       muscle_dof_offsets, muscle_dof_torque_idx, root_dof_count, *model, *fv, nmuscle,
                       muscle_length + w0 * ld_out, effective_activation + w0 * ld_out, length_velocity + w0 * ld_out,
                       force_velocity_multiplier + w0 * ld_out, force_velocity_slope + w0 * ld_out, ld_out);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_waypoints_forces(
    const float *xpos, int64_t ld_xpos, const float *xquat, int64_t ld_xquat,
    const int32_t *waypoint_body, const float *waypoint_local, int nwaypoint, float *waypoints,
    int64_t ld_waypoints, const int32_t *all_segment_start_idx,
    const int32_t *all_muscle_segment_offsets, const float *muscle_params, int ld_params,
    const float *muscle_rest_length, const im_muscle_force_model *model, int nmuscle,
    float *unit_force, int64_t ld_unit, float *passive_force, int64_t ld_passive, int nworld,
    void *stream) {
  const size_t lds_bytes = (size_t)12 * (nwaypoint > 0 ? nwaypoint : 0);
  if (nworld <= 0 || nwaypoint <= 0 || nmuscle <= 0 || lds_bytes > 64 * 1024) {
    // nothing to share between the two, or a world's waypoints do not fit in LDS
    const int rc = im_muscle_waypoints(xpos, ld_xpos, xquat, ld_xquat, waypoint_body,
                                       waypoint_local, nwaypoint, waypoints, ld_waypoints, nworld,
                                       stream);
    if (rc != IM_OK) return rc;
    return im_muscle_force_magnitudes(waypoints, ld_waypoints, all_segment_start_idx,
                                      all_muscle_segment_offsets, muscle_params, ld_params,
                                      muscle_rest_length, model, nmuscle, unit_force, ld_unit,
                                      passive_force, ld_passive, nworld, stream);
  }
  if (!model || !xpos || !xquat || !waypoint_body || !waypoint_local || !waypoints ||
      !all_segment_start_idx || !all_muscle_segment_offsets || !muscle_params ||
      !muscle_rest_length || !unit_force || ld_params < 4)
    return IM_ERR_ARG;
  if (ld_waypoints < 3 * (int64_t)nwaypoint || ld_unit < nmuscle ||
      (passive_force && ld_passive < nmuscle))
    return IM_ERR_STRIDE;
  hipLaunchKernelGGL(waypoints_forces_kernel, dim3((unsigned)nworld), dim3(512), lds_bytes,
                     (hipStream_t)stream, xpos, ld_xpos, xquat, ld_xquat, waypoint_body,
                     waypoint_local, nwaypoint, waypoints, ld_waypoints, all_segment_start_idx,
                     all_muscle_segment_offsets, muscle_params, ld_params, muscle_rest_length,
                     *model, nmuscle, unit_force, ld_unit, passive_force, ld_passive);
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

static Geo slab(const im_muscle_geometry *g, int64_t w0) {
  Geo r = geo(g);
  r.wp += w0 * r.ldw;
  r.com += w0 * r.ldc;
  r.cdof += w0 * r.ldd;
  return r;
}

extern "C" int im_muscle_torque_forward(const im_muscle_geometry *geometry,
                                        const im_muscle_segments *segments,
                                        const im_muscle_entries *torque_entries,
                                        const float *unit_force, int64_t ld_unit,
                                        const float *passive_force, int64_t ld_passive,
                                        const float *activation, int64_t ld_activation,
                                        int root_dof_count, float *torque, int64_t ld_torque,
                                        int nworld, void *stream) {
  if (nworld < 0 || !torque_entries || torque_entries->nrow < 0 || root_dof_count < 0)
    return IM_ERR_ARG;
  const int nt = torque_entries->nrow;
  if (nworld == 0 || nt == 0) return IM_OK;
  if (!geo_ok(geometry) || !seg_ok(segments) || !torque_entries->offsets || !unit_force ||
      !activation || !torque)
    return IM_ERR_ARG;
  if (torque_entries->nentry > 0 && (!torque_entries->segment || !torque_entries->other ||
                                     !torque_entries->start_coeff || !torque_entries->end_coeff))
    return IM_ERR_ARG;
  if (ld_torque < nt) return IM_ERR_STRIDE;
  {
    MwArgs a{geo(geometry), seg(segments), torque_entries->offsets, torque_entries->segment,
             torque_entries->other, nullptr, torque_entries->start_coeff, torque_entries->end_coeff,
             unit_force, passive_force, activation, nullptr, ld_unit, ld_passive, ld_activation, 0,
             torque, nullptr, ld_torque, root_dof_count, nt, torque_entries->nentry,
             segments->nsegment, nt, torque_entries->nother};
    if (launch_world<MW_FORWARD>(a, nworld, (hipStream_t)stream)) {
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(torque_forward_kernel, grid2(nt, nw), dim3(256), 0, (hipStream_t)stream,
                       slab(geometry, w0), seg(segments), torque_entries->offsets,
                       torque_entries->segment, torque_entries->other,
                       torque_entries->start_coeff, torque_entries->end_coeff,
                       unit_force + w0 * ld_unit, ld_unit,
                       passive_force ? passive_force + w0 * ld_passive : nullptr, ld_passive,
                       activation + w0 * ld_activation, ld_activation, root_dof_count, nt,
                       torque + w0 * ld_torque, ld_torque);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_activation_grad(const im_muscle_geometry *geometry,
                                         const im_muscle_segments *segments,
                                         const im_muscle_entries *muscle_entries,
                                         const float *unit_force, int64_t ld_unit,
                                         const float *grad_output, int64_t ld_grad_output,
                                         int root_dof_count, float *grad_activation,
                                         int64_t ld_grad_activation, int nworld, void *stream) {
  if (nworld < 0 || !muscle_entries || muscle_entries->nrow < 0 || root_dof_count < 0)
    return IM_ERR_ARG;
  const int nm = muscle_entries->nrow;
  if (nworld == 0 || nm == 0) return IM_OK;
  if (!geo_ok(geometry) || !seg_ok(segments) || !muscle_entries->offsets || !unit_force ||
      !grad_output || !grad_activation)
    return IM_ERR_ARG;
  if (muscle_entries->nentry > 0 && (!muscle_entries->segment || !muscle_entries->other ||
                                     !muscle_entries->start_coeff || !muscle_entries->end_coeff))
    return IM_ERR_ARG;
  if (ld_grad_activation < nm || ld_unit < nm) return IM_ERR_STRIDE;
  {
    MwArgs a{geo(geometry), seg(segments), muscle_entries->offsets, muscle_entries->segment,
             muscle_entries->other, nullptr, muscle_entries->start_coeff, muscle_entries->end_coeff,
             unit_force, nullptr, nullptr, grad_output, ld_unit, 0, 0, ld_grad_output,
             grad_activation, nullptr, ld_grad_activation, root_dof_count, nm, muscle_entries->nentry,
             segments->nsegment, muscle_entries->nother, nm};
    if (launch_world<MW_GRAD>(a, nworld, (hipStream_t)stream)) {
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(activation_grad_kernel, grid2(nm, nw), dim3(256), 0, (hipStream_t)stream,
                       slab(geometry, w0), seg(segments), muscle_entries->offsets,
                       muscle_entries->segment, muscle_entries->other,
                       muscle_entries->start_coeff, muscle_entries->end_coeff,
                       unit_force + w0 * ld_unit, ld_unit, grad_output + w0 * ld_grad_output,
                       ld_grad_output, root_dof_count, nm,
                       grad_activation + w0 * ld_grad_activation, ld_grad_activation);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_sparse_moment(const im_muscle_geometry *geometry,
                                       const im_muscle_segments *segments,
                                       const int32_t *muscle_dof_torque_idx,
                                       const im_muscle_entries *entry_segments,
                                       int root_dof_count, float *moment, int64_t ld_moment,
                                       int nworld, void *stream) {
  if (nworld < 0 || !entry_segments || entry_segments->nrow < 0 || root_dof_count < 0)
    return IM_ERR_ARG;
  const int ne = entry_segments->nrow;
  if (nworld == 0 || ne == 0) return IM_OK;
  if (!geo_ok(geometry) || !seg_ok(segments) || !muscle_dof_torque_idx ||
      !entry_segments->offsets || !moment)
    return IM_ERR_ARG;
  if (entry_segments->nentry > 0 && (!entry_segments->segment || !entry_segments->start_coeff ||
                                     !entry_segments->end_coeff))
    return IM_ERR_ARG;
  if (ld_moment < ne) return IM_ERR_STRIDE;
  {
    MwArgs a{geo(geometry), seg(segments), entry_segments->offsets, entry_segments->segment, nullptr,
             muscle_dof_torque_idx, entry_segments->start_coeff, entry_segments->end_coeff, nullptr,
             nullptr, nullptr, nullptr, 0, 0, 0, 0, moment, nullptr, ld_moment, root_dof_count, ne,
             entry_segments->nentry, segments->nsegment, entry_segments->nother, 0};
    if (launch_world<MW_MOMENT>(a, nworld, (hipStream_t)stream)) {
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(sparse_moment_kernel, grid2(ne, nw), dim3(256), 0, (hipStream_t)stream,
                       slab(geometry, w0), seg(segments), muscle_dof_torque_idx,
                       entry_segments->offsets, entry_segments->segment,
                       entry_segments->start_coeff, entry_segments->end_coeff, root_dof_count, ne,
                       moment + w0 * ld_moment, ld_moment);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}

extern "C" int im_muscle_torque_bounds(const im_muscle_geometry *geometry,
                                       const im_muscle_segments *segments,
                                       const im_muscle_entries *torque_entries,
                                       const float *unit_force, int64_t ld_unit, int root_dof_count,
                                       float *lower, float *upper, int64_t ld_bounds, int nworld,
                                       void *stream) {
  if (nworld < 0 || !torque_entries || torque_entries->nrow < 0 || root_dof_count < 0)
    return IM_ERR_ARG;
  const int nt = torque_entries->nrow;
  if (nworld == 0 || nt == 0) return IM_OK;
  if (!geo_ok(geometry) || !seg_ok(segments) || !torque_entries->offsets || !unit_force || !lower ||
      !upper)
    return IM_ERR_ARG;
  if (torque_entries->nentry > 0 && (!torque_entries->segment || !torque_entries->other ||
                                     !torque_entries->start_coeff || !torque_entries->end_coeff))
    return IM_ERR_ARG;
  if (ld_bounds < nt) return IM_ERR_STRIDE;
  {
    MwArgs a{geo(geometry), seg(segments), torque_entries->offsets, torque_entries->segment,
             torque_entries->other, nullptr, torque_entries->start_coeff, torque_entries->end_coeff,
             unit_force, nullptr, nullptr, nullptr, ld_unit, 0, 0, 0, lower, upper, ld_bounds,
             root_dof_count, nt, torque_entries->nentry, segments->nsegment, nt,
             torque_entries->nother};
    if (launch_world<MW_BOUNDS>(a, nworld, (hipStream_t)stream)) {
      IM_HIP_CHECK(hipGetLastError());
      return IM_OK;
    }
  }
  IM_FOR_WORLD_SLABS(nworld, w0, nw) {
    hipLaunchKernelGGL(torque_bounds_kernel, grid2(nt, nw), dim3(256), 0, (hipStream_t)stream,
                       slab(geometry, w0), seg(segments), torque_entries->offsets,
                       torque_entries->segment, torque_entries->other,
                       torque_entries->start_coeff, torque_entries->end_coeff,
                       unit_force + w0 * ld_unit, ld_unit, root_dof_count, nt,
                       lower + w0 * ld_bounds, upper + w0 * ld_bounds, ld_bounds);
  }
  IM_HIP_CHECK(hipGetLastError());
  return IM_OK;
}
