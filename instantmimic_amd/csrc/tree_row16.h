// Support for the generated plan-specialised tree kernels ("row16" layout: four
// worlds per wavefront, one 16-lane DPP row per world).  See
// instantmimic_amd/codegen/tree_row16.py for the layout and the generator.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/imhip.h"
#include "newton_wave.h"

namespace im {
namespace gen {

typedef float f32x4 __attribute__((ext_vector_type(4)));

#define IM_ROW16_PARAMS                                                                   \
  const float *__restrict__ M, int64_t ldM, const float *__restrict__ J, int njmax,       \
      const float *__restrict__ D, const int *__restrict__ state,                         \
      const int *__restrict__ nefc_p, int quad, const float *__restrict__ y, int64_t ldy, \
      float *__restrict__ x, int64_t ldx, float *__restrict__ Hout, int nworld, unsigned flags, \
      int niter, int64_t state_it, int64_t y_it, int64_t x_it, const unsigned char *__restrict__ skip

// value of lane n of the caller's 16-lane row, in every lane of the row
#define IM_BC(v, n)                                                                          \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)),     \
                                                        0x150 + (n), 0xF, 0xF, true))
#define IM_FMA(a, b, c) __builtin_fmaf((a), (b), (c))

// Per-lane selects with the lane mask in scalar registers: one v_cndmask, no compare.  The mask
// of a 16-lane row is repeated for the four rows of the wavefront.
#define IM_ROW_MASK(m16) (0x0001000100010001ull * (unsigned long long)(m16))
__device__ __forceinline__ float im_lane_select2(float on, float off, unsigned long long mask) {
  float r;
  asm("v_cndmask_b32 %0, %1, %2, %3" : "=v"(r) : "v"(off), "v"(on), "s"(mask));
  return r;
}
__device__ __forceinline__ float im_lane_select(float on, unsigned long long mask) {
  float r;
  asm("v_cndmask_b32 %0, 0, %1, %2" : "=v"(r) : "v"(on), "s"(mask));
  return r;
}

// 1.0f / x, correctly rounded, for the head of the pivot chain.  The hardware estimate (1 ulp) and
// one correction with an exact residual equal the IEEE quotient bit for bit for every x with
// 2^-101 <= |x| < 2^102 (checked over all such floats on the GPU: im_check_reciprocal); a pivot
// outside that range sends the whole wavefront through the division proper.
__device__ __forceinline__ bool im_reciprocal_in_range(float x) {
  return (__builtin_bit_cast(uint32_t, x) & 0x7fffffffu) - (26u << 23) < (203u << 23);
}
__device__ __forceinline__ float im_reciprocal_fast(float x) {
  const float r = __builtin_amdgcn_rcpf(x);
  return __builtin_fmaf(__builtin_fmaf(-x, r, 1.0f), r, r);
}
// `fast` = im_reciprocal_fast(-x) computed by the caller ahead of time (the estimate and the
// correction are odd functions, so that is -im_reciprocal_fast(x) bit for bit)
__device__ __forceinline__ float im_negative_reciprocal_checked(float x, float fast) {
  if (__builtin_expect(!__all(im_reciprocal_in_range(x)), 0)) fast = -(1.0f / x);
  return fast;
}
__device__ __forceinline__ float im_reciprocal(float x) {
  float r = im_reciprocal_fast(x);
  if (__builtin_expect(!__all(im_reciprocal_in_range(x)), 0)) r = 1.0f / x;
  return r;
}
// workgroup barrier that also orders LDS traffic (usable in wave-uniform branches)
#define IM_BLOCK_SYNC()                                     \
  do {                                                      \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  \
    __builtin_amdgcn_s_barrier();                           \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  \
  } while (0)

// orders one wavefront's LDS writes before its later reads (the workgroup is one wavefront)
#define IM_WAVE_SYNC()                                      \
  do {                                                      \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  \
    __builtin_amdgcn_wave_barrier();                        \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");  \
  } while (0)

struct Row16Entry {
  uint64_t key;  // FNV-1a over the CSR structure and the plan
  int nv, nM;
  int lds_bytes;  // dynamic LDS of the fused kernel (staged constraint rows); the launch adds
                  // 32 bytes per constraint row (rounded up to 16 rows) for the active-row lists
  int short_rows;  // njmax up to which the straight-line fused kernel applies
  const char *name;
  const void *fused;       // assemble + factor + solve, njmax <= short_rows
  const void *fused_long;  // the same with a loop over the constraint rows
  const void *solve;       // factor + solve of a given H, the same four wavefronts per four worlds
  const void *newton;      // the resident Newton loop with the fused kernel as its factor stage, njmax <= short_rows
  const void *newton_long; // the same with the loop over the constraint rows
  int solve_lds_bytes;     // dynamic LDS of the solve-only kernel (the roles' hand-over area)
};

// Registers a generated kernel at load time.
struct Row16Register {
  explicit Row16Register(const Row16Entry *e);
};

const Row16Entry *find_row16(uint64_t key);

}  // namespace gen
}  // namespace im
