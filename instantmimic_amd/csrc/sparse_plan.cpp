// Host-side integer planning of the static-pattern sparse L'DL of H = M + J'DJ: the coupling
// pattern of a model's dofs, the symbolic factor with its elimination levels, and the tables
// the numeric kernels walk.  The numbers must equal the reference planner's exactly: slots,
// runs, the order of a level's entries and the team widths fix the floating-point summation
// order of the factor.
//
// Reference: src/instantmimic/utils/mjw_kernels/sparse_hessian.py
//   hessian_pattern :62-118, _symbolic :192-212, _team :215-221, build_plan :229-401 (tables),
//   limits :249, 337, 680-684.
//
// Everything here works on bit rows.  A pattern row, a column of the factor and a row of the
// factor are bit sets over elimination indices, so
//   * the symbolic factor is the elimination-tree recurrence
//       struct(k) = pattern(k, > k)  U  union over children c of k of struct(c) \ {k},
//     the parent of k being the lowest bit of struct(k) -- the same fill as pairing up all later
//     neighbours of every column, which is how the reference states it;
//   * slots are row-major, slot(i, k) = base(i) + number of row i's bits below k, so the
//     "runs of contiguous slots" of an entry are exactly the runs of consecutive ones in
//     row(i) & row(j) and fall out of a bit scan.
#include <algorithm>
#include <cstring>

#include "sparse_plan.h"

namespace {

constexpr int kMaxSharedBytes = 46 * 1024;  // sparse_hessian.py:178
constexpr int kRowsPerTile = 4;             // sparse_hessian.py:408

// n rows of bits, `words` 64-bit words each
struct BitRows {
  int n = 0, words = 0;
  std::vector<uint64_t> w;
  BitRows() = default;
  BitRows(int rows, int bits) : n(rows), words((bits + 63) / 64), w((size_t)rows * ((bits + 63) / 64), 0) {}
  uint64_t *row(int r) { return w.data() + (size_t)r * words; }
  const uint64_t *row(int r) const { return w.data() + (size_t)r * words; }
  void set(int r, int b) { row(r)[b >> 6] |= 1ull << (b & 63); }
  bool test(int r, int b) const { return (row(r)[b >> 6] >> (b & 63)) & 1; }
};

int lowest_bit(const uint64_t *r, int words) {
  for (int i = 0; i < words; ++i)
    if (r[i]) return i * 64 + __builtin_ctzll(r[i]);
  return -1;
}

int count_bits(const uint64_t *r, int words) {
  int c = 0;
  for (int i = 0; i < words; ++i) c += __builtin_popcountll(r[i]);
  return c;
}

// number of set bits of r strictly below position b
int rank_below(const uint64_t *r, int b) {
  int c = 0;
  for (int i = 0; i < (b >> 6); ++i) c += __builtin_popcountll(r[i]);
  if (b & 63) c += __builtin_popcountll(r[b >> 6] & ((1ull << (b & 63)) - 1));
  return c;
}

template <class F>
void for_each_bit(const uint64_t *r, int words, F &&f) {
  for (int i = 0; i < words; ++i)
    for (uint64_t m = r[i]; m; m &= m - 1) f(i * 64 + __builtin_ctzll(m));
}

// maximal runs of consecutive set bits: f(first, length)
template <class F>
void for_each_run(const uint64_t *r, int words, F &&f) {
  int start = -1, len = 0;
  for_each_bit(r, words, [&](int b) {
    if (start >= 0 && b == start + len) {
      ++len;
    } else {
      if (start >= 0) f(start, len);
      start = b;
      len = 1;
    }
  });
  if (start >= 0) f(start, len);
}

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// lanes per entry of a level: the width with the fewest sweeps x (terms per lane + shuffle
// steps there and back), the narrowest on ties (sparse_hessian.py:215-221)
int team_width(int nentries, int maxterms, int lanes) {
  int best = 1;
  long best_cost = -1;
  for (int log2t = 0; log2t <= 5; ++log2t) {
    const int T = 1 << log2t;
    const int teams = lanes / T;
    if (teams == 0) break;
    const long cost = (long)ceil_div(nentries, teams) * (ceil_div(maxterms, T) + 2 * log2t);
    if (best_cost < 0 || cost < best_cost) {
      best = T;
      best_cost = cost;
    }
  }
  return best;
}

struct Entry {
  int slot, col, nterms, run0, run1;
};

void clique(im_dof_pattern *p, const std::vector<uint64_t> &mask) {
  for_each_bit(mask.data(), p->words, [&](int a) {
    uint64_t *row = p->adj.data() + (size_t)a * p->words;
    for (int i = 0; i < p->words; ++i) row[i] |= mask[i];
    row[a >> 6] &= ~(1ull << (a & 63));
  });
}

}  // namespace

extern "C" {

int im_dof_pattern_create(int nv, const int32_t *dof_parentid, int nbody, const int32_t *body_parentid,
                          const int32_t *body_dofadr, const int32_t *body_dofnum, im_dof_pattern **out) {
  if (!out) return IM_ERR_ARG;
  *out = nullptr;
  if (nv <= 0 || !dof_parentid || nbody < 0) return IM_ERR_ARG;
  if (nbody > 0 && (!body_parentid || !body_dofadr || !body_dofnum)) return IM_ERR_ARG;
  for (int d = 0; d < nv; ++d)
    if (dof_parentid[d] < -1 || dof_parentid[d] >= d) return IM_ERR_ARG;
  for (int b = 1; b < nbody; ++b) {
    if (body_parentid[b] < 0 || body_parentid[b] >= b || body_dofnum[b] < 0) return IM_ERR_ARG;
    if (body_dofnum[b] > 0 && (body_dofadr[b] < 0 || (int64_t)body_dofadr[b] + body_dofnum[b] > nv)) return IM_ERR_ARG;
  }
  auto *p = new im_dof_pattern;
  p->nv = nv;
  p->nbody = nbody;
  p->words = (nv + 63) / 64;
  p->adj.assign((size_t)nv * p->words, 0);
  if (nbody > 0) {
    p->body_parent.assign(body_parentid, body_parentid + nbody);
    p->body_dofadr.assign(body_dofadr, body_dofadr + nbody);
    p->body_dofnum.assign(body_dofnum, body_dofnum + nbody);
  }
  // M's own pattern: a dof couples with each of its ancestors
  for (int d = 0; d < nv; ++d)
    for (int a = dof_parentid[d]; a >= 0; a = dof_parentid[a]) {
      p->adj[(size_t)d * p->words + (a >> 6)] |= 1ull << (a & 63);
      p->adj[(size_t)a * p->words + (d >> 6)] |= 1ull << (d & 63);
    }
  *out = p;
  return IM_OK;
}

void im_dof_pattern_destroy(im_dof_pattern *pattern) { delete pattern; }

int im_dof_pattern_couple_bodies(im_dof_pattern *p, const int32_t *bodies, int n) {
  if (!p || n < 0 || (n > 0 && !bodies)) return IM_ERR_ARG;
  std::vector<uint64_t> mask(p->words, 0);
  for (int q = 0; q < n; ++q) {
    if (bodies[q] < 0 || bodies[q] >= p->nbody) return IM_ERR_ARG;
    for (int b = bodies[q]; b > 0; b = p->body_parent[b])  // body 0 is the world: no dofs
      for (int d = p->body_dofadr[b]; d < p->body_dofadr[b] + p->body_dofnum[b]; ++d) mask[d >> 6] |= 1ull << (d & 63);
  }
  clique(p, mask);
  return IM_OK;
}

int im_dof_pattern_couple_dofs(im_dof_pattern *p, const int32_t *dofs, int n) {
  if (!p || n < 0 || (n > 0 && !dofs)) return IM_ERR_ARG;
  std::vector<uint64_t> mask(p->words, 0);
  for (int q = 0; q < n; ++q) {
    if (dofs[q] < 0 || dofs[q] >= p->nv) return IM_ERR_ARG;
    mask[dofs[q] >> 6] |= 1ull << (dofs[q] & 63);
  }
  clique(p, mask);
  return IM_OK;
}

int im_dof_pattern_get(const im_dof_pattern *p, uint8_t *adjacency) {
  if (!p || !adjacency) return IM_ERR_ARG;
  for (int a = 0; a < p->nv; ++a)
    for (int b = 0; b < p->nv; ++b)
      adjacency[(size_t)a * p->nv + b] = (p->adj[(size_t)a * p->words + (b >> 6)] >> (b & 63)) & 1;
  return IM_OK;
}

int im_sparse_plan_build(const im_dof_pattern *pattern, int nv_pad, int block, int path, const int32_t *M_rowi,
                         const int32_t *M_colind, int nM, int host_only, int *refused, im_sparse_plan **out) {
  if (!out || !refused) return IM_ERR_ARG;
  *out = nullptr;
  *refused = IM_SPARSE_ACCEPTED;
  if (!pattern || nv_pad <= 0 || block < 32 || block % 32 || nM < 0 || (nM > 0 && (!M_rowi || !M_colind))) return IM_ERR_ARG;
  if (path != IM_SPARSE_FUSED && path != IM_SPARSE_NONFUSED) return IM_ERR_ARG;
  const int n = pattern->nv;
  for (int e = 0; e < nM; ++e)
    if (M_rowi[e] < 0 || M_rowi[e] >= n || M_colind[e] < 0 || M_colind[e] >= n) return IM_ERR_ARG;
  const int words = (n + 63) / 64;

  // ---- symbolic factor in elimination order (leaves first: index e = nv - 1 - dof)
  BitRows col(n, n);  // col.row(k): rows below the diagonal of column k
  for (int k = 0; k < n; ++k)
    for_each_bit(pattern->adj.data() + (size_t)(n - 1 - k) * pattern->words, pattern->words, [&](int dof) {
      const int i = n - 1 - dof;
      if (i > k) col.set(k, i);
    });
  std::vector<int> level(n, 0);
  for (int k = 0; k < n; ++k) {
    const int parent = lowest_bit(col.row(k), words);
    if (parent < 0) continue;
    uint64_t *up = col.row(parent);
    const uint64_t *mine = col.row(k);
    for (int i = 0; i < words; ++i) up[i] |= mine[i];
    up[parent >> 6] &= ~(1ull << (parent & 63));
    level[parent] = std::max(level[parent], level[k] + 1);
  }
  BitRows row(n, n);  // row.row(i): columns left of the diagonal of row i
  for (int k = 0; k < n; ++k) for_each_bit(col.row(k), words, [&](int i) { row.set(i, k); });
  const int nlevels = *std::max_element(level.begin(), level.end()) + 1;
  std::vector<std::vector<int>> level_cols(nlevels);
  for (int k = 0; k < n; ++k) level_cols[level[k]].push_back(k);

  // ---- slots: row i's entries left to right, its diagonal, ...; then the right-hand side row
  std::vector<int> base(n + 1, 0);
  for (int i = 0; i < n; ++i) base[i + 1] = base[i] + count_bits(row.row(i), words) + 1;
  const int nfac = base[n], nslots = nfac + n;
  auto diag = [&](int i) { return base[i + 1] - 1; };
  auto slot = [&](int i, int k) { return i == n ? nfac + k : base[i] + rank_below(row.row(i), k); };
  if (nslots >= 65536 || (int64_t)nfac + n > (int64_t)nv_pad * nv_pad) {
    *refused = IM_SPARSE_REFUSED_LAYOUT;
    return IM_OK;
  }

  auto *pl = new im_sparse_plan;
  pl->nv = n; pl->nv_pad = nv_pad; pl->block = block; pl->path = path;
  pl->nslots = nslots; pl->nfac = nfac; pl->nlevels = nlevels;
  pl->density = (double)nfac / ((double)n * (n + 1) / 2.0);
  auto &T = pl->table;
  pl->col_ptr.push_back(0);
  for (int k = 0; k < n; ++k) {
    for_each_bit(col.row(k), words, [&](int i) { pl->col_idx.push_back(i); });
    pl->col_ptr.push_back((int)pl->col_idx.size());
  }
  pl->col_level.assign(level.begin(), level.end());

  // ---- numeric factor: per level the entries (i, j) of its columns j, i over the diagonal, the
  // column's rows and the right-hand side row; an entry's terms k run over row(j) & row(i)
  T[im::LP].push_back(0);
  T[im::RP].push_back(0);
  std::vector<uint64_t> both(words);
  std::vector<int> runs;  // a, b, k, length
  std::vector<Entry> entries;
  for (const auto &cols : level_cols) {
    entries.clear();
    runs.clear();
    for (int j : cols) {
      auto add = [&](int i) {
        const uint64_t *rj = row.row(j);
        if (i == j || i == n) {
          std::copy(rj, rj + words, both.begin());
        } else {
          const uint64_t *ri = row.row(i);
          for (int q = 0; q < words; ++q) both[q] = rj[q] & ri[q];
        }
        Entry e{i == j ? diag(j) : slot(i, j), i == j ? j : -1, count_bits(both.data(), words), (int)runs.size() / 4, 0};
        for_each_run(both.data(), words, [&](int k, int len) {
          runs.insert(runs.end(), {i == j ? slot(j, k) : slot(i, k), slot(j, k), k, len});
        });
        e.run1 = (int)runs.size() / 4;
        entries.push_back(e);
      };
      add(j);
      for_each_bit(col.row(j), words, add);
      add(n);
    }
    // longest sums first, ties in the order above
    std::stable_sort(entries.begin(), entries.end(), [](const Entry &a, const Entry &b) { return a.nterms > b.nterms; });
    int maxterms = 0;
    for (const Entry &e : entries) {
      T[im::ES].push_back(e.slot);
      T[im::EC].push_back(e.col);
      for (int r = e.run0; r < e.run1; ++r) {
        T[im::RAB].push_back((int32_t)((uint32_t)runs[4 * r] | ((uint32_t)runs[4 * r + 1] << 16)));
        T[im::RKL].push_back((int32_t)((uint32_t)runs[4 * r + 2] | ((uint32_t)runs[4 * r + 3] << 16)));
      }
      T[im::RP].push_back((int)T[im::RAB].size());
      pl->nterms += e.nterms;
      maxterms = std::max(maxterms, e.nterms);
    }
    T[im::LP].push_back((int)T[im::ES].size());
    T[im::LT].push_back(team_width((int)entries.size(), maxterms, block));
  }

  // ---- solves: forward rows by level; backward pushes, root level first
  T[im::FL].push_back(0);
  for (const auto &cols : level_cols) {
    T[im::FR].insert(T[im::FR].end(), cols.begin(), cols.end());
    T[im::FL].push_back((int)T[im::FR].size());
  }
  T[im::RKP].push_back(0);
  for (int j = 0; j < n; ++j) {
    T[im::RS].push_back(base[j]);
    for_each_bit(row.row(j), words, [&](int k) { T[im::RK].push_back(k); });
    T[im::RKP].push_back((int)T[im::RK].size());
  }
  T[im::BL].push_back(0);
  for (int l = nlevels - 1; l >= 0; --l) {
    for (int i : level_cols[l]) {
      int s = base[i];
      for_each_bit(row.row(i), words, [&](int j) {
        T[im::BS].push_back(s++);
        T[im::BI].push_back(i);
        T[im::BJ].push_back(j);
      });
    }
    T[im::BL].push_back((int)T[im::BS].size());
  }
  for (int id : {im::LP, im::ES, im::RP, im::FL, im::FR, im::RS, im::RKP, im::RK, im::BL, im::BS, im::BI, im::BJ})
    for (int32_t v : T[id])
      if (v >= 65536) {
        delete pl;
        *refused = IM_SPARSE_REFUSED_INDEX16;
        return IM_OK;
      }

  // ---- dof-order views of the slots: element of M behind each slot, gather index into a dense
  // H, slot of a dof pair, pattern row of each dof
  std::vector<int32_t> m_of(n * (size_t)n, -1);  // (min dof, max dof) -> CSR element, the last one listed
  for (int e = 0; e < nM; ++e) {
    const int a = std::min(M_rowi[e], M_colind[e]), b = std::max(M_rowi[e], M_colind[e]);
    m_of[(size_t)a * n + b] = e;
  }
  T[im::PAIR].assign((size_t)n * n, -1);
  for (int i = 0; i < n; ++i) {
    const int a = n - 1 - i;  // the row's dof: the smaller of the pair, its columns are deeper dofs
    auto emit = [&](int k, int s) {
      const int b = n - 1 - k;
      T[im::SA].push_back(a);
      T[im::SB].push_back(b);
      T[im::SM].push_back(m_of[(size_t)a * n + b]);
      T[im::GAT].push_back(a * nv_pad + b);
      T[im::PAIR][(size_t)a * n + b] = s;
    };
    int s = base[i];
    for_each_bit(row.row(i), words, [&](int k) { emit(k, s++); });
    emit(i, s);
  }
  for (int e = 0; e < n; ++e) T[im::ORIG].push_back(n - 1 - e);
  const int mask_words = (n + 31) / 32;
  T[im::PM].assign((size_t)n * mask_words, 0);
  for (int a = 0; a < n; ++a)
    for (int b = 0; b < n; ++b)
      if (a == b || T[im::PAIR][(size_t)std::min(a, b) * n + std::max(a, b)] >= 0)
        T[im::PM][(size_t)a * mask_words + b / 32] |= (int32_t)(1u << (b % 32));

  if (2 * (int64_t)nfac + n >= (int64_t)nv_pad * nv_pad - 1) {
    delete pl;
    *refused = IM_SPARSE_REFUSED_HFACTOR;
    return IM_OK;
  }
  const int init_tile = path == IM_SPARSE_FUSED ? kRowsPerTile * n + kRowsPerTile : 0;
  if (4 * (nslots + n + 2 * (block / 32) + init_tile) > kMaxSharedBytes) {
    delete pl;
    *refused = IM_SPARSE_REFUSED_SHARED;
    return IM_OK;
  }
  for (auto &t : T)
    if (t.empty()) t.push_back(0);  // the reference emits {0} for an empty table
  if (!host_only) {
    const int st = im::sparse_plan_upload(pl);
    if (st != IM_OK && st != IM_ERR_UNSUPPORTED) {
      im_sparse_plan_destroy(pl);
      return st;
    }
  }
  *out = pl;
  return IM_OK;
}

int im_sparse_plan_get_info(const im_sparse_plan *plan, im_sparse_plan_info *info) {
  if (!plan || !info) return IM_ERR_ARG;
  info->nv = plan->nv;
  info->nv_pad = plan->nv_pad;
  info->block = plan->block;
  info->path = plan->path;
  info->nslots = plan->nslots;
  info->nfac = plan->nfac;
  info->nterms = plan->nterms;
  info->nlevels = plan->nlevels;
  info->device_ready = plan->device_ready ? 1 : 0;
  info->density = plan->density;
  return IM_OK;
}

int im_sparse_plan_table_size(const im_sparse_plan *plan, int table) {
  if (!plan || table < 0 || table >= im::NHOST) return -1;
  return (int)plan->table[table].size();
}

int im_sparse_plan_get_table(const im_sparse_plan *plan, int table, int32_t *out, int capacity) {
  if (!plan || !out || table < 0 || table >= im::NHOST) return IM_ERR_ARG;
  const auto &t = plan->table[table];
  if (capacity < (int)t.size()) return IM_ERR_ARG;
  std::copy(t.begin(), t.end(), out);
  return IM_OK;
}

int im_sparse_plan_get_structure(const im_sparse_plan *plan, int32_t *col_ptr, int32_t *col_idx, int32_t *col_level) {
  if (!plan) return IM_ERR_ARG;
  if (col_ptr) std::copy(plan->col_ptr.begin(), plan->col_ptr.end(), col_ptr);
  if (col_idx) std::copy(plan->col_idx.begin(), plan->col_idx.end(), col_idx);
  if (col_level) std::copy(plan->col_level.begin(), plan->col_level.end(), col_level);
  return IM_OK;
}

}  // extern "C"
