// Support for the generated plan-specialised tree kernels ("row16" layout: four
// worlds per wavefront, one 16-lane DPP row per world).  See
// instantmimic_amd/codegen/tree_row16.py for the layout and the generator.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/imhip.h"

namespace im {
namespace gen {

typedef float f32x4 __attribute__((ext_vector_type(4)));

#define IM_ROW16_PARAMS                                                                   \
  const float *__restrict__ M, int64_t ldM, const float *__restrict__ J, int njmax,       \
      const float *__restrict__ D, const int *__restrict__ state,                         \
      const int *__restrict__ nefc_p, int quad, const float *__restrict__ y, int64_t ldy, \
      float *__restrict__ x, int64_t ldx, float *__restrict__ Hout, int nworld, unsigned flags

// value of lane n of the caller's 16-lane row, in every lane of the row
#define IM_BC(v, n)                                                                          \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)),     \
                                                        0x150 + (n), 0xF, 0xF, true))
#define IM_FMA(a, b, c) __builtin_fmaf((a), (b), (c))
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
  const void *solve;       // factor + solve
};

// Registers a generated kernel at load time.
struct Row16Register {
  explicit Row16Register(const Row16Entry *e);
};

const Row16Entry *find_row16(uint64_t key);

}  // namespace gen
}  // namespace im
