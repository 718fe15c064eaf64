// Host-side state of a static-pattern sparse L'DL plan (internal).
#pragma once

#include <cstdint>
#include <vector>

#include "../../include/imhip.h"

namespace im {

// Order of the tables inside a plan and on the device; the public IM_SH_* ids of imhip.h.
enum SparseTable {
  LP, LT, ES, EC, RP, RAB, RKL, ORIG, BL, BS, BI, BJ, PM, SA, SB, SM, NINIT,
  PAIR = NINIT, FL, FR, RS, RKP, RK, NTABLES, GAT = NTABLES, NHOST
};

}  // namespace im

struct im_dof_pattern {
  int nv = 0, nbody = 0, words = 0;
  std::vector<uint64_t> adj;  // nv rows of `words` 64-bit words, bit b of row a: dofs a and b couple
  std::vector<int32_t> body_parent, body_dofadr, body_dofnum;
};

struct im_sparse_plan {
  int nv = 0, nv_pad = 0, block = 0, path = 0, nslots = 0, nfac = 0, nterms = 0, nlevels = 0;
  double density = 0.0;
  std::vector<int32_t> table[im::NHOST];
  std::vector<int32_t> col_ptr, col_idx, col_level;  // symbolic factor: later rows of every column
  // device side (sparse_kernels.hip)
  bool device_ready = false;
  void *blob = nullptr;
  const int32_t *t[im::NHOST] = {};
  int sizes[im::NHOST] = {};
  // per lane of the lower-triangle 16 x 16 accumulator tiles: where the element comes from in a
  // row of M and which slot it is ((M index + 1) << 16 | (slot + 1)); null when nv > 64
  int32_t *tile_index = nullptr;
  int nM = 0;
  // one int on the device: the next world of a batch nobody has started (im_newton_solve_sparse)
  int *next_world = nullptr;
};

namespace im {
// Copies the tables to the current device (sparse_kernels.hip).  IM_ERR_UNSUPPORTED when the
// device kernels do not take the plan's shape; the plan stays usable on the host.
int sparse_plan_upload(im_sparse_plan *plan);
}  // namespace im
