// Shared host-side declarations of libimhip (internal).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "../../include/imhip.h"

namespace im {

constexpr int kWave = 64;

void set_hip_error(hipError_t e);

#define IM_HIP_CHECK(expr)                 \
  do {                                     \
    hipError_t e_ = (expr);                \
    if (e_ != hipSuccess) {                \
      ::im::set_hip_error(e_);             \
      return IM_ERR_HIP;                   \
    }                                      \
  } while (0)

// Per-plan device tables of the tree kernels.  All pointers address one device
// allocation owned by the plan.
struct TreeDev {
  const int32_t *slot_e;    // [spl * 64]  CSR entry held by (lane, register) or -1
  const uint32_t *slot_d;   // [spl * 64]  a | b << 8 | p << 16 | q << 24 | (trunk row: see slot_e bit 30)
  const int4 *steps;        // [nsteps]    {rowadr[k], rownnz[k] - 1, group (4 = trunk, -1 = merge), k}
  const uint64_t *anc;      // [nsteps]    bit i set when dof i is a strict ancestor of k
  const int32_t *dof_d;     // [64]        rowadr | depth << 16 | trunk << 24, -1 past nv
  const int32_t *colind;    // [nM]
  const uint64_t *related;  // [64]        bit i set when dof i is dof k itself, an ancestor or a descendant of it
  int32_t nv, nM, nsteps, maxdepth, ngroups;
};

}  // namespace im

struct im_tree_plan {
  int nv = 0, nM = 0;
  std::vector<int> rowadr, rownnz, colind, parent, depth;
  std::vector<std::vector<int>> groups;  // dofs descending
  std::vector<int> trunk;                // ascending
  std::vector<int> elim;
  int span = 0, shared_bytes = 0, maxdepth = 0;
  int64_t dense_cost = 0;  // size^3 / 3 summed over the trees: beyond 32 bits from 1861 dofs in one tree
  bool beats_dense = false;
  // device side
  bool device_ready = false;
  int device = -1;
  void *dev_blob = nullptr;
  im::TreeDev dev{};
  int spl = 0;  // H slots per lane
  const void *row16 = nullptr;  // generated kernel for this structure, if one was built
  // kernels loaded at run time from a code object (im_tree_plan_attach_kernels): row16 then points
  // at row16_own, whose kernel fields hold hipFunction_t handles of `module`
  void *module = nullptr;
  void *row16_own = nullptr;
  // whether the resident Newton kernels of row16 keep to registers (short / long variant)
  bool resident_ok = false, resident_long_ok = false;
  int *next_world = nullptr;  // device int behind dev_blob's tables: the resident Newton kernel's counter of worlds handed out
  // false for 65 to 96 dofs: the table-driven kernel keeps a dof per lane and ancestors in 64-bit
  // masks, so such a plan runs on generated kernels only (device_ready, nothing launched before
  // kernels are attached)
  bool table_driven = true;
};

namespace im {
// Builds the device tables (tree_kernels.hip).
int tree_plan_upload(im_tree_plan *plan);
}  // namespace im
