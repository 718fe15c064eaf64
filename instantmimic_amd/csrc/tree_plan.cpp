// Host-side integer planning of the tree L'DL: which dofs form the serial trunk,
// which subtrees are packed into which group, and in what order dofs are
// eliminated.  The numbers must equal the reference planner's exactly, since the
// plan fixes the floating-point summation order of the factorisation.
//
// Reference: src/instantmimic/utils/mjw_kernels/tree_ldl.py
//   tree_ldl_structure :66-91, _shared_bytes :98-102, plan_tree_ldl :105-170,
//   best_tree_ldl_plan :173-185, tree_ldl_beats_dense :188-193.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <numeric>

#include "common.h"

namespace {

constexpr int kMaxSharedBytes = 48 * 1024;  // tree_ldl.py:32
constexpr int kMaxShortSpan = 4096;         // tree_ldl.py:43
constexpr double kMinDenseToSpan = 8.0;     // tree_ldl.py:44

thread_local int g_last_hip_error = 0;

bool nested_ancestor_csr(int nv, const int32_t *rowadr, const int32_t *rownnz,
                         const int32_t *colind, int ncol) {
  if (nv <= 0) return false;
  for (int k = 0; k < nv; ++k) {
    if (rownnz[k] < 1 || rowadr[k] < 0) return false;
    if ((int64_t)rowadr[k] + rownnz[k] > ncol) return false;
  }
  for (int k = 0; k < nv; ++k) {
    const int32_t *row = colind + rowadr[k];
    const int n = rownnz[k];
    if (row[n - 1] != k) return false;
    for (int p = 0; p + 1 < n; ++p) {
      const int i = row[p];
      if (i < 0 || i >= k) return false;
      // ancestor i sits at depth p: its row is the first p + 1 entries of this one
      if (rownnz[i] != p + 1) return false;
      if (std::memcmp(colind + rowadr[i], row, sizeof(int32_t) * (p + 1)) != 0) return false;
    }
  }
  return true;
}

struct Tree {
  int nv;
  std::vector<int> parent, cost, subtree, size, roots;
  std::vector<std::vector<int>> children;
};

Tree build_tree(const im_tree_plan &pl) {
  Tree t;
  t.nv = pl.nv;
  t.parent.resize(pl.nv);
  t.children.assign(pl.nv, {});
  for (int k = 0; k < pl.nv; ++k) {
    t.parent[k] = pl.rownnz[k] > 1 ? pl.colind[pl.rowadr[k] + pl.rownnz[k] - 2] : -1;
    if (t.parent[k] >= 0) t.children[t.parent[k]].push_back(k);
  }
  // eliminating a dof with n row entries: n (n - 1) / 2 updates + scaling and solve
  t.cost.resize(pl.nv);
  for (int k = 0; k < pl.nv; ++k) {
    const int n = pl.rownnz[k];
    t.cost[k] = n * (n - 1) / 2 + 2 * n;
  }
  t.subtree = t.cost;
  t.size.assign(pl.nv, 1);
  for (int k = pl.nv - 1; k >= 0; --k)
    if (t.parent[k] >= 0) {
      t.subtree[t.parent[k]] += t.subtree[k];
      t.size[t.parent[k]] += t.size[k];
    }
  for (int k = 0; k < pl.nv; ++k)
    if (t.parent[k] < 0) t.roots.push_back(k);
  return t;
}

struct Cut {
  int span = -1;
  std::vector<int> trunk;
  std::vector<std::vector<int>> members;  // part roots per group
};

// Longest-processing-time packing of part roots into exactly `groups` bins.
int pack_parts(const Tree &t, std::vector<int> parts, int groups,
               std::vector<std::vector<int>> *members) {
  std::stable_sort(parts.begin(), parts.end(), [&](int a, int b) {
    if (t.subtree[a] != t.subtree[b]) return t.subtree[a] > t.subtree[b];
    return a < b;
  });
  std::vector<int> load(groups, 0);
  members->assign(groups, {});
  for (int r : parts) {
    const int g = int(std::min_element(load.begin(), load.end()) - load.begin());
    load[g] += t.subtree[r];
    (*members)[g].push_back(r);
  }
  return *std::max_element(load.begin(), load.end());
}

void plan_for_groups(im_tree_plan *pl, const Tree &t, int groups) {
  std::vector<int> parts = t.roots, trunk;
  Cut best;
  for (;;) {
    std::vector<std::vector<int>> members;
    const int heaviest = pack_parts(t, parts, groups, &members);
    int span = heaviest;
    for (int k : trunk) span += t.cost[k] + 2 * pl->rownnz[k];
    if (best.span < 0 || span < best.span) {
      best.span = span;
      best.trunk = trunk;
      best.members = members;
    }
    // the heaviest part that still has children gives its root to the trunk
    int pick = -1;
    for (int r : parts) {
      if (t.children[r].empty()) continue;
      if (pick < 0 || t.subtree[r] > t.subtree[pick] ||
          (t.subtree[r] == t.subtree[pick] && r < pick))
        pick = r;
    }
    if (pick < 0) break;
    parts.erase(std::find(parts.begin(), parts.end(), pick));
    trunk.push_back(pick);
    parts.insert(parts.end(), t.children[pick].begin(), t.children[pick].end());
  }
  pl->span = best.span;
  pl->trunk = best.trunk;
  std::sort(pl->trunk.begin(), pl->trunk.end());
  pl->groups.clear();
  for (const auto &roots : best.members) {
    std::vector<int> nodes, stack = roots;
    while (!stack.empty()) {
      const int k = stack.back();
      stack.pop_back();
      nodes.push_back(k);
      for (int c : t.children[k]) stack.push_back(c);
    }
    std::sort(nodes.begin(), nodes.end(), std::greater<int>());
    pl->groups.push_back(nodes);
  }
  pl->dense_cost = 0;
  for (int r : t.roots) pl->dense_cost += ((int64_t)t.size[r] * t.size[r] * t.size[r]) / 3;
}

int exchange_bytes(const im_tree_plan &pl, int groups) {
  if (pl.trunk.empty()) return 0;
  int entries = 0;
  for (int i : pl.trunk) entries += pl.rownnz[i];
  return 4 * 32 * (groups * (entries + int(pl.trunk.size())) + int(pl.trunk.size()));
}

}  // namespace

namespace im {
void set_hip_error(hipError_t e) { g_last_hip_error = int(e); }
#ifdef IM_PLANNER_ONLY
// this file alone as a host-only planner (used while the library itself is being built)
int tree_plan_upload(im_tree_plan *) { return IM_ERR_UNSUPPORTED; }
#endif
}  // namespace im

extern "C" {

int im_version(void) { return 100; }

int im_last_hip_error(void) { return g_last_hip_error; }

const char *im_status_string(int status) {
  switch (status) {
    case IM_OK: return "ok";
    case IM_ERR_ARG: return "invalid argument";
    case IM_ERR_STRUCTURE: return "CSR rows are not nested ancestor lists";
    case IM_ERR_UNSUPPORTED: return "shape not supported by the device kernels";
    case IM_ERR_HIP: return "HIP runtime error";
    case IM_ERR_STRIDE: return "rows must be contiguous floats";
    case IM_ERR_SCRATCH: return "the batch exceeds the library's static scratch (IM_STATIC_SCRATCH_BYTES)";
    default: return "unknown status";
  }
}

int im_tree_structure_check(int nv, const int32_t *rowadr, const int32_t *rownnz,
                            const int32_t *colind, int ncol) {
  if (!rowadr || !rownnz || !colind || ncol < 0) return IM_ERR_ARG;
  return nested_ancestor_csr(nv, rowadr, rownnz, colind, ncol) ? IM_OK : IM_ERR_STRUCTURE;
}

int im_tree_plan_create(int nv, const int32_t *rowadr, const int32_t *rownnz,
                        const int32_t *colind, int ncol, int groups,
                        int host_only, im_tree_plan **out) {
  if (!out) return IM_ERR_ARG;
  *out = nullptr;
  if (!rowadr || !rownnz || !colind || groups < 0 || groups > IM_MAX_GROUPS) return IM_ERR_ARG;
  if (!nested_ancestor_csr(nv, rowadr, rownnz, colind, ncol)) return IM_ERR_STRUCTURE;
  auto *pl = new im_tree_plan;
  pl->nv = nv;
  pl->rowadr.assign(rowadr, rowadr + nv);
  pl->rownnz.assign(rownnz, rownnz + nv);
  int nM = 0;
  for (int k = 0; k < nv; ++k) nM = std::max(nM, rowadr[k] + rownnz[k]);
  pl->nM = nM;
  pl->colind.assign(colind, colind + nM);
  const Tree t = build_tree(*pl);
  pl->parent = t.parent;
  pl->depth.resize(nv);
  for (int k = 0; k < nv; ++k) pl->depth[k] = rownnz[k] - 1;
  pl->maxdepth = *std::max_element(pl->depth.begin(), pl->depth.end());
  if (groups > 0) {
    plan_for_groups(pl, t, groups);
  } else {
    // fewest groups among the shortest spans whose exchange fits 48 KB
    im_tree_plan best;
    bool have = false;
    for (int g = 1; g <= IM_MAX_GROUPS; ++g) {
      plan_for_groups(pl, t, g);
      if (exchange_bytes(*pl, g) > kMaxSharedBytes) continue;
      if (!have || pl->span < best.span) {
        best.span = pl->span;
        best.trunk = pl->trunk;
        best.groups = pl->groups;
        best.dense_cost = pl->dense_cost;
        have = true;
      }
    }
    pl->span = best.span;
    pl->trunk = best.trunk;
    pl->groups = best.groups;
    pl->dense_cost = best.dense_cost;
  }
  pl->shared_bytes = exchange_bytes(*pl, int(pl->groups.size()));
  pl->beats_dense = pl->span <= kMaxShortSpan || double(pl->dense_cost) >= kMinDenseToSpan * pl->span;
  for (const auto &g : pl->groups) pl->elim.insert(pl->elim.end(), g.begin(), g.end());
  pl->elim.insert(pl->elim.end(), pl->trunk.rbegin(), pl->trunk.rend());
  if (!host_only) {
    const int st = im::tree_plan_upload(pl);
    if (st != IM_OK && st != IM_ERR_UNSUPPORTED) {
      delete pl;
      return st;
    }
  }
  *out = pl;
  return IM_OK;
}

void im_tree_plan_destroy(im_tree_plan *plan) {
  if (!plan) return;
  if (plan->dev_blob) (void)hipFree(plan->dev_blob);
  if (plan->module) (void)hipModuleUnload((hipModule_t)plan->module);
  std::free(plan->row16_own);
  delete plan;
}

int im_tree_plan_get_info(const im_tree_plan *plan, im_tree_plan_info *info) {
  if (!plan || !info) return IM_ERR_ARG;
  info->nv = plan->nv;
  info->nM = plan->nM;
  info->ngroups = int(plan->groups.size());
  info->ntrunk = int(plan->trunk.size());
  info->span = plan->span;
  info->dense_cost = (int32_t)std::min<int64_t>(plan->dense_cost, INT32_MAX);  // saturates; beats_dense is decided on the full value
  info->shared_bytes = plan->shared_bytes;
  info->beats_dense = plan->beats_dense ? 1 : 0;
  info->max_depth = plan->maxdepth + 1;
  info->device_ready = plan->device_ready ? 1 : 0;
  return IM_OK;
}

int im_tree_plan_get_arrays(const im_tree_plan *plan, int32_t *group_ptr,
                            int32_t *group_dofs, int32_t *trunk, int32_t *elim_order) {
  if (!plan) return IM_ERR_ARG;
  int n = 0;
  if (group_ptr) group_ptr[0] = 0;
  for (size_t j = 0; j < plan->groups.size(); ++j) {
    for (int k : plan->groups[j]) {
      if (group_dofs) group_dofs[n] = k;
      ++n;
    }
    if (group_ptr) group_ptr[j + 1] = n;
  }
  if (trunk) std::copy(plan->trunk.begin(), plan->trunk.end(), trunk);
  if (elim_order) std::copy(plan->elim.begin(), plan->elim.end(), elim_order);
  return IM_OK;
}

}  // extern "C"
