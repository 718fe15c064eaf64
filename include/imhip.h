/* libimhip -- C ABI of the MI355X (gfx950) batched Newton linear-algebra path.
 *
 * Every entry point is what a binding of the reference's Python launchers for
 * this path would call.  Citations are relative to the reference tree
 * (Scripter36/InstantMimic).  Conventions:
 *   - plain C types only; device buffers are caller-owned device pointers;
 *   - every launcher takes a hipStream_t (as void*), never synchronises, never
 *     allocates, and is safe to capture in a hipGraph;
 *   - the return value is a status code (IM_OK == 0); nothing throws;
 *   - planners report "ineligible" through the plan info / a status code, which
 *     mirrors the reference returning None so that the caller keeps its fallback.
 */
#ifndef IMHIP_H_
#define IMHIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IM_OK 0
#define IM_ERR_ARG 1         /* null pointer, negative size, bad enum */
#define IM_ERR_STRUCTURE 2   /* CSR is not in nested-ancestor form */
#define IM_ERR_UNSUPPORTED 3 /* shape outside what the kernels are built for */
#define IM_ERR_HIP 4         /* a HIP runtime call failed (see im_last_hip_error) */
#define IM_ERR_STRIDE 5      /* rows are not contiguous floats */
#define IM_ERR_SCRATCH 6     /* the batch needs more than IM_STATIC_SCRATCH_BYTES of the static scratch */

#define IM_MAX_GROUPS 4

typedef struct im_tree_plan im_tree_plan;

typedef struct im_tree_plan_info {
  int32_t nv;           /* dofs */
  int32_t nM;           /* CSR entries of M */
  int32_t ngroups;      /* groups in the plan (may include empty ones) */
  int32_t ntrunk;       /* trunk dofs */
  int32_t span;         /* critical path in update units */
  int32_t dense_cost;   /* sum over trees of size^3 / 3 */
  int32_t shared_bytes; /* trunk exchange footprint of the reference's CUDA kernel */
  int32_t beats_dense;  /* 1 when the reference would use the tree solve */
  int32_t max_depth;    /* longest ancestor chain (row length) */
  int32_t device_ready; /* 1 when the device kernels support this shape */
} im_tree_plan_info;

/* Library / runtime ------------------------------------------------------- */
int im_version(void);
const char *im_status_string(int status);
/* hipError_t of the last failing HIP call on this thread (0 if none). */
int im_last_hip_error(void);

/* Tree L'DL planning (host, integer) -------------------------------------- */

/* Replaces tree_ldl_structure (src/instantmimic/utils/mjw_kernels/tree_ldl.py:66-91):
 * IM_OK when every CSR row is "ancestors root-first, diagonal last" and each
 * ancestor's row is a prefix of it, else IM_ERR_STRUCTURE. */
int im_tree_structure_check(int nv, const int32_t *rowadr, const int32_t *rownnz,
                            const int32_t *colind, int ncol);

/* Replaces plan_tree_ldl (tree_ldl.py:105-170) for groups in 1..4 and
 * best_tree_ldl_plan (tree_ldl.py:173-185) for groups == 0.  Builds the device
 * tables on the current HIP device unless host_only != 0 (planning without a
 * GPU).  The plan is immutable afterwards. */
int im_tree_plan_create(int nv, const int32_t *rowadr, const int32_t *rownnz,
                        const int32_t *colind, int ncol, int groups,
                        int host_only, im_tree_plan **out);
void im_tree_plan_destroy(im_tree_plan *plan);

/* TreeLdlPlan fields (tree_ldl.py:47-56), tree_ldl_beats_dense (:188-193) and
 * _shared_bytes (:98-102). */
int im_tree_plan_get_info(const im_tree_plan *plan, im_tree_plan_info *info);
/* group_ptr[ngroups + 1], group_dofs[nv - ntrunk] (each group descending),
 * trunk[ntrunk] (ascending), elim_order[nv] = groups in order then the trunk
 * descending (tree_ldl.py:256-257, 290).  Any pointer may be null. */
int im_tree_plan_get_arrays(const im_tree_plan *plan, int32_t *group_ptr,
                            int32_t *group_dofs, int32_t *trunk,
                            int32_t *elim_order);

/* Launchers ---------------------------------------------------------------- */

/* Replaces tree_factor_solve (tree_ldl.py:419-433): x = (L'DL)^-1 y for every
 * world, M (nworld, ldM >= nM) in the model's CSR layout, M is not modified.
 * ld* are row strides in floats. */
int im_tree_factor_solve(const im_tree_plan *plan, const float *M, int64_t ldM,
                         const float *y, int64_t ldy, float *x, int64_t ldx,
                         int nworld, void *stream);

#define IM_FLAG_NEGATE 1u /* write -x (the Newton search direction) */

/* The fused Newton linear step on a tree pattern: H = M + sum over rows r with
 * state == quad and r < nefc[w] of D J'J on M's CSR entries (summation order of
 * sparse_hessian.py:589, 622-629), tree L'DL of H and solve with grad
 * (tree_ldl.py:215-305).  What the reference reaches through
 * newton_fusion._update_gradient_sparse / sparse_hessian.init_factor_kernel
 * (newton_fusion.py:480-519) and tree_ldl.tree_factor_solve.
 *   J (nworld, njmax, nv) contiguous, D/state (nworld, njmax), nefc (nworld) or
 *   null for njmax rows everywhere, grad (nworld, ldg), x (nworld, ldx),
 *   Hout (nworld, nM) or null.
 * Products of a row outside M's pattern (a row over two branches) are dropped:
 * im_tree_pattern_violations counts such rows. */
int im_assemble_tree_ldl_solve(const im_tree_plan *plan, const float *M,
                               int64_t ldM, const float *J, int njmax,
                               const float *D, const int32_t *state,
                               const int32_t *nefc, int quad, const float *grad,
                               int64_t ldg, float *x, int64_t ldx, float *Hout,
                               int nworld, unsigned flags, void *stream);

/* The guard of the tree pattern.  im_assemble_tree_ldl_solve holds H on M's CSR entries, that is
 * on pairs (dof, ancestor): a constraint row whose nonzero dofs do not all lie on one
 * root-to-leaf chain has products outside that pattern, which are dropped without a trace.
 * This launch counts such rows per world -- rows r < nefc[w] with state == quad and D != 0, as
 * the reference's sparse assembly counts rows outside its declared pattern
 * (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:605-621, read back through
 * violation_counter, :786-796) -- and adds the count to violations[w] (float, accumulates until
 * the caller zeroes it: a periodic check sees every violation).  Costs one pass over J; run it
 * when a row producer changes, or every so many steps. */
int im_tree_pattern_violations(const im_tree_plan *plan, const float *J, int njmax, const float *D,
                               const int32_t *state, const int32_t *nefc, int quad,
                               float *violations, int nworld, void *stream);

/* im_assemble_tree_ldl_solve for `niter` Newton iterations that share M, J and D and differ in
 * the constraint states (and optionally the gradient): what a step of the reference's Newton
 * loop does with a world kept resident in one block across its iterations
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:57-298).  Iteration i reads
 * state + i * state_iter_stride (ints) and grad + i * grad_iter_stride (floats; 0 = one gradient
 * for all) and writes x + i * x_iter_stride.  Every iteration assembles H afresh from M, so the
 * results are those of niter calls of im_assemble_tree_ldl_solve bit for bit; where a generated
 * kernel exists for the tree the whole sequence is one launch whose grid covers (worlds,
 * iteration) with the iterations of a world scheduled next to one L2, so M and J come from
 * memory once and one iteration's factor phase overlaps another's reads. */
int im_assemble_tree_ldl_solve_iters(const im_tree_plan *plan, const float *M, int64_t ldM,
                                     const float *J, int njmax, const float *D,
                                     const int32_t *state, int64_t state_iter_stride,
                                     const int32_t *nefc, int quad, const float *grad, int64_t ldg,
                                     int64_t grad_iter_stride, float *x, int64_t ldx,
                                     int64_t x_iter_stride, int nworld, int niter, unsigned flags,
                                     void *stream);

/* Kernels generated for one structure and plan, loaded at run time.  The reference emits
 * straight-line code for any model when its scratch is created
 * (src/instantmimic/utils/mjw_kernels/tree_ldl.py:196-359, 393-416); here the library carries such
 * kernels for a few known trees and takes the others as a gfx950 code object that the host side
 * builds from the generator's source (instantmimic_amd/codegen/tree_row16.py, module form).
 * im_tree_plan_kernel_key: the 64-bit key of the plan's structure and elimination plan, and whether
 * the plan already has generated kernels.  im_tree_plan_attach_kernels: loads the code object
 * (kept by the plan until it is destroyed) after checking that it was generated for this key;
 * IM_ERR_STRUCTURE otherwise; IM_ERR_UNSUPPORTED for a code object whose fused kernels keep a
 * private segment (register spills to memory): the plan then stays on the table-driven kernel.
 * The plan's launches then use it.  Once per plan, on the plan's device, not while the plan is in
 * use by another thread. */
int im_tree_plan_kernel_key(const im_tree_plan *plan, unsigned long long *key, int *has_kernel);
int im_tree_plan_attach_kernels(im_tree_plan *plan, const void *code_object);

/* Self-check of an arithmetic shortcut (no counterpart in the reference): the generated tree
 * kernels take a pivot's reciprocal as the hardware estimate plus one exact-residual correction
 * instead of the full division whenever 2^-101 <= |pivot| < 2^102.  This launch compares the two
 * for every float whose bit pattern lies in [first_bits, last_bits] and that is in that range,
 * and adds the number of differing results to *mismatches (a device counter the caller zeroes).
 * It must stay 0: the kernels' bit-for-bit agreement with the reference's 1.0f / x rests on it. */
int im_check_reciprocal(uint32_t first_bits, uint32_t last_bits, unsigned long long *mismatches,
                        void *stream);

/* The same for the blocked Cholesky's pivots: counts the floats with bit patterns in
 * [first_bits, last_bits] and value in [2^-96, inf) for which the kernels' short square root or
 * the short reciprocal of the root differ from sqrtf(x) or 1.0f / sqrtf(x).  Expected: 0. */
int im_check_pivot_sqrt(uint32_t first_bits, uint32_t last_bits, unsigned long long *mismatches, void *stream);

/* Coupling pattern of a model's dofs: which pairs (a, b) may be nonzero in H.  Replaces
 * hessian_pattern (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:62-118) as a builder:
 * creation couples every dof with its tree ancestors (:70-75; dof_parentid[d] < d), and the
 * caller adds one clique per source of constraint rows.  body_parentid / body_dofadr /
 * body_dofnum (nbody each, body 0 = world) are the model's. */
typedef struct im_dof_pattern im_dof_pattern;
int im_dof_pattern_create(int nv, const int32_t *dof_parentid, int nbody,
                          const int32_t *body_parentid, const int32_t *body_dofadr,
                          const int32_t *body_dofnum, im_dof_pattern **out);
void im_dof_pattern_destroy(im_dof_pattern *pattern);
/* All dofs on the chains from the listed bodies to the world couple pairwise: a declared body
 * group, the two bodies of a connect / weld equality or of a collision pair, a flex element
 * (`clique` of the reference, :77-86). */
int im_dof_pattern_couple_bodies(im_dof_pattern *pattern, const int32_t *bodies, int n);
/* The listed dofs couple pairwise (a joint equality, :104-107). */
int im_dof_pattern_couple_dofs(im_dof_pattern *pattern, const int32_t *dofs, int n);
/* adjacency (nv, nv) bytes, 1 where dofs a != b couple; symmetric, zero diagonal. */
int im_dof_pattern_get(const im_dof_pattern *pattern, uint8_t *adjacency);

/* Static-pattern sparse L'DL of H = M + J'DJ -------------------------------- */

typedef struct im_sparse_plan im_sparse_plan;

#define IM_SPARSE_FUSED 0    /* path "fused": the persistent Newton's layout of hfactor */
#define IM_SPARSE_NONFUSED 1 /* path "nonfused": factor gathered from the dense H */

/* Why a plan was refused (the reference raises ValueError with these meanings,
 * sparse_hessian.py:249-250, 337-338, 680-684). */
#define IM_SPARSE_ACCEPTED 0
#define IM_SPARSE_REFUSED_LAYOUT 1  /* nslots >= 65536 or nfac + nv > nv_pad^2 */
#define IM_SPARSE_REFUSED_INDEX16 2 /* a table value does not fit 16 bits */
#define IM_SPARSE_REFUSED_HFACTOR 3 /* 2 nfac + nv >= nv_pad^2 - 1 */
#define IM_SPARSE_REFUSED_SHARED 4  /* factor larger than the reference's 46 KB of shared memory */

/* Table ids for im_sparse_plan_get_table, the reference's SH_* arrays (:360-401, SH_GAT :291-297). */
enum {
  IM_SH_LP, IM_SH_LT, IM_SH_ES, IM_SH_EC, IM_SH_RP, IM_SH_RAB, IM_SH_RKL, IM_SH_ORIG, IM_SH_BL,
  IM_SH_BS, IM_SH_BI, IM_SH_BJ, IM_SH_PM, IM_SH_SA, IM_SH_SB, IM_SH_SM, IM_SH_PAIR, IM_SH_FL,
  IM_SH_FR, IM_SH_RS, IM_SH_RKP, IM_SH_RK, IM_SH_GAT, IM_SH_COUNT
};

/* SparseHessianPlan (sparse_hessian.py:38-50). */
typedef struct im_sparse_plan_info {
  int32_t nv, nv_pad, block, path;
  int32_t nslots;  /* factor slots + nv right-hand-side slots */
  int32_t nfac;    /* factor slots: entries of L incl. the diagonal */
  int32_t nterms;  /* multiply-adds of one numeric factor */
  int32_t nlevels; /* elimination-tree levels */
  int32_t device_ready;
  double density;  /* nfac over the dense triangle */
} im_sparse_plan_info;

/* Replaces build_plan (sparse_hessian.py:229-401, 680-702): symbolic factor in elimination
 * order e = nv - 1 - dof (:192-212, 235-237), row-major slots (:239-248), per level the
 * entries with their runs of contiguous slots sorted by falling term count and the team width
 * (:263-290, 215-221), the solve, pair, assembly, gather and pattern-mask tables (:291-401).
 * M_rowi / M_colind (nM): row and column dof of every CSR element of M (m.M_hinit_i,
 * m.M_colind).  block: the workgroup width the team widths are computed for.  A pattern the
 * reference refuses yields IM_OK, *out = NULL and *refused != 0 (the caller keeps its dense
 * factor, as for None).  The device tables go to the current HIP device unless host_only. */
int im_sparse_plan_build(const im_dof_pattern *pattern, int nv_pad, int block, int path,
                         const int32_t *M_rowi, const int32_t *M_colind, int nM, int host_only,
                         int *refused, im_sparse_plan **out);
void im_sparse_plan_destroy(im_sparse_plan *plan);
int im_sparse_plan_get_info(const im_sparse_plan *plan, im_sparse_plan_info *info);
/* Number of int32 values of a table, -1 for a bad id; an empty table holds one 0. */
int im_sparse_plan_table_size(const im_sparse_plan *plan, int table);
int im_sparse_plan_get_table(const im_sparse_plan *plan, int table, int32_t *out, int capacity);
/* The fill pattern and elimination levels for a bit-exact comparison: column k of the factor
 * (elimination index) has the later rows col_idx[col_ptr[k] .. col_ptr[k + 1]) ascending
 * (col_ptr nv + 1 values, col_idx nfac - nv) and sits on level col_level[k].  Any pointer may
 * be null. */
int im_sparse_plan_get_structure(const im_sparse_plan *plan, int32_t *col_ptr, int32_t *col_idx,
                                 int32_t *col_level);

/* Replaces the launch of sparse_hessian.init_factor_kernel(plan)
 * (sparse_hessian.py:804-846, launched from newton_fusion.py:502-519) with the same
 * arrays: done (nworld) bytes or null, nefc (nworld), J (nworld, njmax, nv), D/state
 * (nworld, njmax), M (nworld, ldM), grad (nworld, ldg), hfactor (nworld, nv_pad,
 * nv_pad) used as flat scratch ([0,nfac) packed H, [nfac,2nfac) factor, then 1/D, last
 * element = pattern-violation counter, which accumulates), search (nworld, nv),
 * search_dot / decrement (nworld). */
int im_sparse_init_factor(const im_sparse_plan *plan, const uint8_t *done,
                          const int32_t *nefc, const float *J, int njmax, const float *D,
                          const int32_t *state, int quad, const float *M, int ldM,
                          const float *grad, int ldg, float *hfactor, float *search,
                          float *search_dot, float *decrement, int nworld, void *stream);

/* im_jtdj_mfma followed by im_blocked_factor_solve (block size 16, the whole H as one dense tile)
 * in one launch: a Newton iteration's dense Hessian, its upper Cholesky factor and the solve
 * (the reference runs the upstream assembly and its blocked factor as separate kernels around
 * src/instantmimic/utils/mjw_kernels/newton_stages.py:614-742).  H (nworld, nv_pad, nv_pad) is
 * written when not null (the per-iteration stage updates it later), U (nworld, pad, pad) when not
 * null (tiles on and right of the block diagonal, as im_blocked_factor_solve), x = H^-1 y when x
 * and y are given.  pad = nv rounded up to 16.  Results equal those of
 * the two entry points called one after the other, bit for bit.  nv <= 128. */
int im_jtdj_factor_solve(const float *Mdense, const float *J, int njmax, const float *D, const int32_t *state,
                         const int32_t *nefc, int quad, float *H, int nv, int nv_pad, const float *y, int64_t ldy,
                         float *U, int pad, float *x, int64_t ldx, int nworld, void *stream);

/* Replaces the factor stage of the fused Newton loop on the static pattern
 * (newton_stages.factor_factory with a sparse plan, src/instantmimic/utils/mjw_kernels/
 * newton_stages.py:614-742, and the native modes 0 / 1 / 2 of sparse_hessian.py:488-547).
 * Per world, skipped when done[w] or state_changes[w] == 0:
 *   changes[w] > 0: dof_union[w, :n] = ascending dofs the changed rows ids[w, :changes[w]]
 *     touch, n in dof_union[w, nv]; packed H in hfactor gets, per pair of those dofs,
 *     delta = sum over the changed rows of +-D a b (minus when the row's new state is not
 *     quad; newton_stages.py:451-470), pairs outside the pattern count as violations; the
 *     factor is rebuilt and stored back into hfactor;
 *   changes[w] == 0: forward solve with the factor stored in hfactor.
 * Then the backward solve, search = -x, search_dot, decrement.  The reference keeps the
 * factor in a resident block's shared memory between iterations; here hfactor carries it
 * from launch to launch.  ids (nworld, ld_ids), dof_union (nworld, nv + 1).  Needs a plan
 * created with 22 tables. */
int im_sparse_update_factor(const im_sparse_plan *plan, const uint8_t *done,
                            const int32_t *state_changes, const int32_t *changes,
                            const int32_t *ids, int ld_ids, const float *J, int njmax,
                            const float *D, const int32_t *state, int quad, const float *grad,
                            int ldg, float *hfactor, int32_t *dof_union, float *search,
                            float *search_dot, float *decrement, int nworld, void *stream);

/* Replaces the factor step of the upstream (non-fused) Newton iteration on the static pattern
 * (nonfused_kernel, src/instantmimic/utils/mjw_kernels/sparse_hessian.py:849-894, native modes 4
 * and 5 of :639-679).  Needs a plan built with IM_SPARSE_NONFUSED.  Per world, skipped when
 * done[w], or when skip_noflip and state_changed[w] == 0:
 *   refactor (always, unless skip_unchanged and quad_changed[w] == 0): the slots of the factor
 *     are gathered from the dense Hessian H[w] (nv_pad x nv_pad, world stride ldH) through SH_GAT,
 *     factored level by level with grad as the augmented row, and hfactor[w] receives
 *     [0, nfac) N = L D and [nfac, nfac + nv) 1 / D;
 *   otherwise the factor stored in hfactor[w] solves the new gradient.
 * Then the backward solve, search = -x, search_dot, decrement.  done, quad_changed,
 * state_changed may be null where the flags do not ask for them. */
int im_sparse_dense_factor(const im_sparse_plan *plan, const uint8_t *done, const float *grad, int ldg,
                           const float *H, int64_t ldH, const int32_t *quad_changed,
                           const int32_t *state_changed, int skip_unchanged, int skip_noflip,
                           float *hfactor, float *search, int ld_search, float *search_dot,
                           float *decrement, int nworld, void *stream);

/* Replaces _tile_cholesky_factorize_solve_no_l_store
 * (src/instantmimic/utils/mjw_step_optimized.py:672-701, launched from
 * _factor_solve_i_dense_no_l_store, :839-846): for every world and every tile t, the diagonal
 * block of tile_size dofs at tile_adr[t] of the dense M (ld_world floats per world, ld_row per
 * row; its lower triangle is read) is Cholesky-factored and x[w, adr .. adr + size) =
 * block^-1 y[w, same]; the factor is not kept.  tile_size <= 64 (IM_ERR_UNSUPPORTED beyond);
 * dofs outside every tile are not written. */
int im_tile_cholesky_solve(const float *M, int64_t ld_world, int64_t ld_row, const int32_t *tile_adr, int ntile,
                           int tile_size, const float *y, int64_t ldy, float *x, int64_t ldx, int nworld,
                           void *stream);

/* Replaces _tile_cholesky_factorize_solve_m_no_l_store (mjw_step_optimized.py:704-750, launched
 * from :826-836): M holds nM values per world (row stride ldM) and block b's element (r, c) is
 * M[w, block_elemid[(b tile_size + r) tile_size + c]] (the reference's tile.elemid; an id at or
 * past nM reads as zero; the upper triangle is read, as fill_mode "upper" does there);
 * block_dof[b] is the block's first dof in y and x. */
int im_tile_cholesky_solve_m(const float *M, int64_t ldM, int nM, const int32_t *block_elemid,
                             const int32_t *block_dof, int nblock, int tile_size, const float *y, int64_t ldy,
                             float *x, int64_t ldx, int nworld, void *stream);

/* The dense stage below for nv <= 32 (newton_stages.py:723-733): no factor is kept between
 * iterations; after the update of H the matrix is factored as one tile and solved for the
 * gradient at every call that state_changes[w] != 0 lets through.  im_dense_update_factor hands
 * such shapes here itself. */
int im_dense_update_tile(const uint8_t *done, const int32_t *state_changes, const int32_t *changes,
                         const int32_t *ids, int ld_ids, const float *J, int njmax, const float *D,
                         const int32_t *state, int quad, const float *grad, int64_t ldg, float *H, int nv,
                         int nv_pad, int32_t *dof_union, float *search, int64_t ld_search, float *search_dot,
                         float *decrement, int nworld, void *stream);

/* The same stage on the dense Hessian (newton_stages.py:614-742 without a sparse plan):
 * H (nworld, nv_pad, nv_pad) receives the deltas on its upper triangle
 * (H[w, row, col] += delta, row <= col, :700-701); with changed rows the augmented blocked
 * Cholesky of augmented_factor_solve_factory (:473-611) runs with 16 x 16 tiles: the
 * gradient rides as column nv_pad - 1, the corner is 1e30, U (nworld, nv_pad, nv_pad)
 * receives the factor including that column (the 16 x 16 tiles on and right of the block diagonal;
 * those below it are never written or read); without changed rows the stored U is solved
 * against.  Rows and columns >= nv of H count as the identity.  nv_pad = a multiple of 16
 * above nv (src/instantmimic/utils/mjw_model.py:30).  H and U must be 16-byte aligned
 * (IM_ERR_STRIDE otherwise).  changes[w] < 0: no row is applied and H as it lies in memory is
 * factored -- the first factor of a solve, after the full assembly that upstream's
 * solver._update_gradient makes there (src/instantmimic/utils/mjw_kernels/newton_fusion.py:470).
 * nv <= 32: the single-tile form above (U is neither read nor written). */
int im_dense_update_factor(const uint8_t *done, const int32_t *state_changes,
                           const int32_t *changes, const int32_t *ids, int ld_ids,
                           const float *J, int njmax, const float *D, const int32_t *state,
                           int quad, const float *grad, int64_t ldg, float *H, float *U, int nv,
                           int nv_pad, int32_t *dof_union, float *search, int64_t ld_search,
                           float *search_dot, float *decrement, int nworld, void *stream);

/* The same stage for nv_pad = 48 or 64 (33 to 63 dofs) on one wavefront per world, a lane per
 * column of the padded matrix: same arguments, same results bit for bit; im_dense_update_factor
 * hands such shapes here.  IM_ERR_UNSUPPORTED for other paddings. */
int im_dense_update_column(const uint8_t *done, const int32_t *state_changes, const int32_t *changes,
                           const int32_t *ids, int ld_ids, const float *J, int njmax, const float *D,
                           const int32_t *state, int quad, const float *grad, int64_t ldg, float *H, float *U, int nv,
                           int nv_pad, int32_t *dof_union, float *search, int64_t ld_search, float *search_dot,
                           float *decrement, int nworld, void *stream);

/* The first Hessian of a dense Newton solve and its factor in one launch, a wavefront per world:
 * H = M + J' diag(D [state == quad]) J (upstream's solver._update_gradient as
 * src/instantmimic/utils/mjw_kernels/newton_fusion.py:470 calls it for the dense Newton) for every
 * world, written to H (nworld, nv_pad, nv_pad) in both triangles, then, for the worlds that are not
 * done, what im_dense_update_factor does with changes[w] < 0: the factor of H as it lies there
 * (into U above 32 dofs), the solve for the gradient, search, search_dot, decrement and an empty
 * dof_union.  M (nworld rows of ldM floats) is the tree-sparse inertia, elemid (nv, nv) the element
 * of a row of M at every pair of dofs, negative outside its pattern (the layout of the reference's
 * m.M_elemid).  nefc may be null (every world has njmax rows).  Same results, bit for bit, as
 * im_dense_from_csr, im_jtdj_mfma and im_dense_update_factor one after the other.  nv <= 32 (any
 * nv_pad that is a multiple of four; U may be null) or nv_pad = 48 or 64; IM_ERR_UNSUPPORTED
 * otherwise: the caller then issues the three launches.  H must be 16-byte aligned. */
int im_dense_init_factor(const uint8_t *done, const int32_t *nefc, const float *J, int njmax, const float *D,
                         const int32_t *state, int quad, const float *M, int64_t ldM, const int32_t *elemid,
                         const float *grad, int64_t ldg, float *H, float *U, int nv, int nv_pad, int32_t *dof_union,
                         float *search, int64_t ld_search, float *search_dot, float *decrement, int nworld,
                         void *stream);

/* The same for nv <= 32 alone; im_dense_init_factor hands such shapes here. */
int im_dense_init_tile(const uint8_t *done, const int32_t *nefc, const float *J, int njmax, const float *D,
                       const int32_t *state, int quad, const float *M, int64_t ldM, const int32_t *elemid,
                       const float *grad, int64_t ldg, float *H, int nv, int nv_pad, int32_t *dof_union, float *search,
                       int64_t ld_search, float *search_dot, float *decrement, int nworld, void *stream);

/* Blocked dense factor + solve, dense J'DJ ----------------------------------- */

/* Replaces _blocked_dense_factor_solve (src/instantmimic/utils/mjw_step_optimized.py:
 * 958-993) and its kernel factor_solve_indexed_cholesky_kernel
 * (src/instantmimic/utils/mjw_kernels/indexed_factor.py:176-214): upper Cholesky
 * U'U = M by block_size x block_size tiles with indexed gather, x = M^-1 y.
 * block_idx is the (nblk, nblk, B, B)-ordered table of element ids into M[w, :] built
 * by create_blocked_dense_factor_solve_scratch (mjw_step_optimized.py:932-941); ids
 * >= nM read as zero; padded diagonal entries get +1.  U (nworld, pad, pad) receives the
 * factor (the reference's workspace; 16-byte aligned) or may be null: the tiles on and right of
 * the block diagonal are written, as by the reference's kernel (indexed_factor.py:115, 141); the
 * tiles below it keep what the caller's buffer holds (zeros in the reference's scratch) and no
 * entry point reads them.  block_size 8 or 16. */
int im_blocked_factor_solve(const float *M, int64_t ldM, int nM, const int32_t *block_idx,
                            int block_size, int nv, int pad, const float *y, int64_t ldy,
                            float *U, float *x, int64_t ldx, int nworld, void *stream);

/* The index table of create_blocked_dense_factor_solve_scratch
 * (src/instantmimic/utils/mjw_step_optimized.py:932-946), on the host: elemid (nv, nv) = element
 * of M[w, :] behind every entry of the dense tile (the model's M_tiles[0].elemid); layout
 * receives pad * pad ids in (nblk, nblk, B, B) order with pad = nv rounded up to block_size and
 * nM on the padding; identity (B * B floats, may be null) is 1 on the padded diagonal entries of
 * the last block. */
int im_blocked_index_layout(const int32_t *elemid, int nv, int nM, int block_size,
                            int32_t *layout, float *identity);

/* Replaces make_indexed_cholesky_multi_solve_kernel (indexed_factor.py:394-493): x = M^-1 y for
 * rhs_count right-hand sides from a stored factor U (nworld, pad, pad) (upper triangle read), y and
 * x (nworld, nv, rhs_count) contiguous.  Worlds with active[w] == 0 are left alone (active may be
 * null: all worlds).  A column sees the operations of im_blocked_factor_solve's own forward and
 * backward substitution in the same order. */
int im_blocked_multi_solve(const float *U, int block_size, int nv, int pad, const float *y,
                           int rhs_count, const int32_t *active, float *x, int nworld, void *stream);

/* Replaces make_indexed_cholesky_factor_multi_solve_kernel (indexed_factor.py:217-391): the
 * factor of im_blocked_factor_solve into the workspace U (nworld, pad, pad; required, 16-byte
 * aligned), then im_blocked_multi_solve from it -- two launches, so the result equals a later
 * im_blocked_multi_solve on the same U bit for bit.  Inactive worlds: neither U nor x is touched. */
int im_blocked_factor_multi_solve(const float *M, int64_t ldM, int nM, const int32_t *block_idx,
                                  int block_size, int nv, int pad, const float *y, int rhs_count,
                                  const int32_t *active, float *U, float *x, int nworld,
                                  void *stream);

/* im_blocked_factor_multi_solve for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  The
 * factor workspace U is a static device array of IM_STATIC_SCRATCH_BYTES inside the library, one
 * per GPU, held until the process ends; the call allocates nothing.  nworld * pad * pad * 4 bytes
 * beyond that size are refused with IM_ERR_SCRATCH.  Results equal im_blocked_factor_multi_solve
 * bit for bit.  All calls on one GPU share the array: calls that overlap there (two streams, two
 * threads) race, and the factor of one call is gone after the next.  The first call on a device
 * looks the array's address up and must not be made under stream capture. */
#define IM_STATIC_SCRATCH_BYTES (32u << 20)
int im_blocked_factor_multi_solve_static(const float *M, int64_t ldM, int nM,
                                         const int32_t *block_idx, int block_size, int nv, int pad,
                                         const float *y, int rhs_count, const int32_t *active,
                                         float *x, int nworld, void *stream);

/* Replaces _copy_dense_factor_kernel (src/instantmimic/utils/mjw_step_optimized.py:875-886):
 * L_out[w, block_adr[0] + row * nv + col] = U[w, row, col] for row, col < nv; block_adr is the
 * device array m.qLD_block_adr, L_out (nworld, ld_out) the caller's d.qLD. */
int im_copy_dense_factor(const float *U, int pad, const int32_t *block_adr, int nv, float *L_out,
                         int64_t ld_out, int nworld, void *stream);

/* Dense Newton Hessian on fp32 MFMA: H[w] (nv_pad, nv_pad) = Mdense[w] (nv, nv) +
 * J[w]' diag(D [state == quad, row < nefc]) J[w].  Stands in for mujoco_warp's
 * solver._update_gradient JTDAJ kernel, which the reference calls at
 * src/instantmimic/utils/mjw_kernels/newton_fusion.py:470 and sizes at
 * src/instantmimic/utils/mjw_model.py:31-35.  nv <= 128.  Rows of J that do not contribute (past
 * nefc, or in another state than `quad`) are not read behind the first 32; an element's sum is the
 * chain fma(J[r][i] * D[r], J[r][j], .) over the rows in order, from Mdense[i][j], for i <= j, and
 * H[j][i] is a copy of H[i][j].  The list of contributing rows takes 8 bytes of LDS per row of
 * njmax beside 33 KB of staged rows: IM_ERR_UNSUPPORTED where that exceeds 160 KB. */
int im_jtdj_mfma(const float *Mdense, const float *J, int njmax, const float *D,
                 const int32_t *state, const int32_t *nefc, int quad, float *H, int nv,
                 int nv_pad, int nworld, void *stream);

/* Muscle moment-arm contractions ------------------------------------------- */

/* Replaces project_muscle_sparse_moment_qfrc_kernel
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:2941-2961, launched from
 * src/instantmimic/envs/controls/fast_muscle/torque_runtime.py:895-909):
 *   qfrc[w, root + j] = sum over s in [offsets[j], offsets[j + 1]) of
 *                       moment[w, e] * force[w, entry_muscle[e]],  e = entry_idx[s]
 * summed in that order.  moment (nworld, ld_moment >= nentry), force (nworld,
 * ld_force >= nmuscle), qfrc (nworld, ld_qfrc >= root + ntorque); the three index
 * tables are device arrays built once per model. */
int im_muscle_project(const float *moment, int64_t ld_moment, const float *force,
                      int64_t ld_force, const int32_t *torque_entry_offsets,
                      const int32_t *torque_entry_idx, const int32_t *entry_muscle,
                      int nentry, int nmuscle, int ntorque, int root_dof_count,
                      float *qfrc, int64_t ld_qfrc, int nworld, void *stream);

/* The tables of build_muscle_implicit_qderiv_gather
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:614-669), on the host: the pairs
 * (pair_entry_i, pair_entry_j) grouped by their M element pair_elem_id (ties in list order), every
 * element's pairs cut into chunks of 16, packed i | j << 16 chunk-interleaved (pair k of chunk c
 * at chunk_pairs[k * chunk_count + c]) and padded with nentry | nentry << 16.  Call once with
 * the three output arrays null to learn *nelem and *chunk_count, then with elem_ids (nelem),
 * chunk_offsets (nelem + 1) and chunk_pairs (16 * chunk_count). */
int im_muscle_gather_tables(const int32_t *pair_elem_id, const int32_t *pair_entry_i,
                            const int32_t *pair_entry_j, int npair, int nentry, int32_t *elem_ids,
                            int32_t *chunk_offsets, int32_t *chunk_pairs, int *nelem,
                            int *chunk_count);

/* Replaces apply_muscle_implicit_qderiv_gather (muscle_qfrc_projector.py:777-809,
 * kernel :736-774): qderiv[w, elem_ids[slot]] += timestep * sum over the slot's
 * chunks, in order, of the chunk's 16-pair sum of
 * (slope[w, entry_muscle[i]] * moment[w, i]) * moment[w, j], pairs packed i | j << 16
 * at chunk_pairs[k * chunk_count + c], padding = nentry.  Deterministic (no atomics). */
int im_muscle_implicit_gather(const float *moment, int64_t ld_moment, const float *slope,
                              int64_t ld_slope, const int32_t *entry_muscle, int nentry,
                              const int32_t *elem_ids, int nelem,
                              const int32_t *chunk_offsets, const int32_t *chunk_pairs,
                              int chunk_count, float timestep, float *qderiv,
                              int64_t ld_qderiv, int nworld, void *stream);

/* Muscle path geometry, activation -> torque and its gradient ------------------ */

/* Curves of src/instantmimic/muscle/muscle_qfrc_projector.py:103-187.  active =
 * (type, p1, p2): type < 0.5 gaussian with gamma = p1, else MuJoCo piecewise with
 * (lmin, lmax) = (p1, p2).  passive = (type, p1, p2): type < 0.5 exponential with
 * (k_pe, e_mo), else MuJoCo with (lmax, fpmax). */
typedef struct im_muscle_force_model {
  float force_scale;
  float length_norm_min, length_norm_max;
  float active[3];
  float passive[3];
  int32_t include_passive; /* 0 writes zeros to passive_force */
} im_muscle_force_model;

/* Per-world pose arrays, ld* = row stride in floats: waypoints (nworld, 3 nwaypoint),
 * subtree_com (nworld, 3 nbody), cdof (nworld, 6 nv) with angular xyz then linear xyz. */
typedef struct im_muscle_geometry {
  const float *waypoints;
  int64_t ld_waypoints;
  const float *subtree_com;
  int64_t ld_subtree_com;
  const float *cdof;
  int64_t ld_cdof;
} im_muscle_geometry;

/* Applied segments: waypoint ids of both ends and the tree-root body of each end's body
 * (apply_segment_start_idx / _end_idx, segment_*_root_body_idx_i32 of the reference's
 * MuscleDynamicsLayer, src/instantmimic/muscle/muscle_dynamics.py:1318-1341). */
typedef struct im_muscle_segments {
  const int32_t *start_waypoint, *end_waypoint, *start_root_body, *end_root_body;
  int32_t nsegment;
} im_muscle_segments;

/* A CSR list of (segment, other) entries with the start/end subtree coefficients:
 * rows = torque dofs and other = muscle (build_torque_sparse_segment_entries,
 * muscle_qfrc_projector.py:378-456), rows = muscles and other = torque dof
 * (build_muscle_sparse_torque_entries, :459-510), or rows = (muscle, dof) entries and
 * other unused (MuscleDofSparseEntries, :513-533).
 * nother bounds the column that is not the row: every `other` is in [0, nother) (the muscle
 * count, or the torque dof count); for the third kind it is the torque dof count, which
 * bounds muscle_dof_torque_idx.  0 = not stated: the contractions then take their
 * one-thread-per-output kernels, which need no bound and are several times slower. */
typedef struct im_muscle_entries {
  const int32_t *offsets; /* nrow + 1 */
  const int32_t *segment; /* nentry */
  const int32_t *other;   /* nentry or null */
  const float *start_coeff, *end_coeff;
  int32_t nrow, nentry;
  int32_t nother;
} im_muscle_entries;

/* Replaces _transform_waypoints_from_torch_kernel
 * (src/instantmimic/muscle/muscle_dynamics_kernels.py:73-86): xpos (nworld, 3 nbody),
 * xquat (nworld, 4 nbody) scalar first, normalised with the reference's 1e-8 guard. */
int im_muscle_waypoints(const float *xpos, int64_t ld_xpos, const float *xquat,
                        int64_t ld_xquat, const int32_t *waypoint_body,
                        const float *waypoint_local, int nwaypoint, float *waypoints,
                        int64_t ld_waypoints, int nworld, void *stream);

/* Replaces _compute_force_magnitudes_from_waypoints_kernel
 * (muscle_dynamics_kernels.py:644-705): polyline length over every segment of a muscle,
 * normalised fibre length, unit (activation 1) and passive force magnitudes.
 * muscle_params (nmuscle, ld_params >= 4) = f0, l_m0, l_t0, pennation.  passive_force may
 * be null. */
int im_muscle_force_magnitudes(const float *waypoints, int64_t ld_waypoints,
                               const int32_t *all_segment_start_idx,
                               const int32_t *all_muscle_segment_offsets,
                               const float *muscle_params, int ld_params,
                               const float *muscle_rest_length,
                               const im_muscle_force_model *model, int nmuscle,
                               float *unit_force, int64_t ld_unit, float *passive_force,
                               int64_t ld_passive, int nworld, void *stream);

/* MuJoCo's force-velocity curve parameters and the two switches of
 * muscle_force_velocity_response_wp (muscle_qfrc_projector.py:2528-2570). */
typedef struct im_muscle_force_velocity_model {
  float vmax, fvmax;
  float clamp_activation; /* nonzero: activation clamped to [0, 1] */
  float include_active;   /* factor of the slope (0 switches the implicit term off) */
} im_muscle_force_velocity_model;

/* Replaces eval_muscle_force_velocity_state_kernel
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:2816-2884), the producer of the slope that
 * im_muscle_implicit_gather takes: per world and muscle the length over its consecutive
 * waypoints [muscle_waypoint_start[m], muscle_waypoint_start[m + 1]), the lengthening velocity
 * -sum over its entries e in [muscle_dof_offsets[m], muscle_dof_offsets[m + 1]) of
 * moment[w, e] * qvel[w, muscle_dof_torque_idx[e] + root_dof_count] (one fused multiply-add per
 * entry, in order), and from them effective_activation = a * fv, length_velocity,
 * force_velocity_multiplier = fv and force_velocity_slope = include_active * a * unit_force *
 * fv' / velocity_scale, velocity_scale = max(length_scale[m] * vmax, 1e-6).  The five outputs are
 * (nworld, ld_out >= nmuscle).  Only the active curve of `model` is read. */
int im_muscle_force_velocity_state(
    const float *waypoints, int64_t ld_waypoints, const int32_t *muscle_waypoint_start,
    const float *muscle_params, int ld_params, const float *muscle_rest_length,
    const float *force_velocity_length_scale, const float *activation, int64_t ld_activation,
    const float *qvel, int64_t ld_qvel, const float *moment, int64_t ld_moment,
    const int32_t *muscle_dof_offsets, const int32_t *muscle_dof_torque_idx, int root_dof_count,
    const im_muscle_force_model *model, const im_muscle_force_velocity_model *fv, int nmuscle,
    float *muscle_length, float *effective_activation, float *length_velocity,
    float *force_velocity_multiplier, float *force_velocity_slope, int64_t ld_out, int nworld,
    void *stream);

/* im_muscle_waypoints followed by im_muscle_force_magnitudes in one launch, for the caller
 * that wants both: MuscleDynamicsLayer._prepare_warp_waypoint_geometry
 * (src/instantmimic/muscle/muscle_dynamics.py:4344-4500) launches the two kernels one after
 * the other on the same workspace.  A workgroup keeps its world's waypoints in LDS between
 * the two steps, so they are written once and not read back; results are those of the two
 * calls bit for bit.  More than 5461 waypoints (64 KiB) fall back to the two launches.
 * Arguments as in the two calls. */
int im_muscle_waypoints_forces(const float *xpos, int64_t ld_xpos, const float *xquat,
                               int64_t ld_xquat, const int32_t *waypoint_body,
                               const float *waypoint_local, int nwaypoint, float *waypoints,
                               int64_t ld_waypoints, const int32_t *all_segment_start_idx,
                               const int32_t *all_muscle_segment_offsets,
                               const float *muscle_params, int ld_params,
                               const float *muscle_rest_length,
                               const im_muscle_force_model *model, int nmuscle,
                               float *unit_force, int64_t ld_unit, float *passive_force,
                               int64_t ld_passive, int nworld, void *stream);

/* Replaces _compute_muscle_dynamics_from_activation_sparse_kernel
 * (muscle_dynamics_kernels.py:1707-1793), the body of the operator
 * instantmimic_muscle::torque_forward (src/instantmimic/muscle/warp_custom_ops.py:98-114).
 * passive_force null = the include_passive_force=False specialisation.
 * torque (nworld, ld_torque >= torque_entries->nrow). */
int im_muscle_torque_forward(const im_muscle_geometry *geometry,
                             const im_muscle_segments *segments,
                             const im_muscle_entries *torque_entries, const float *unit_force,
                             int64_t ld_unit, const float *passive_force, int64_t ld_passive,
                             const float *activation, int64_t ld_activation, int root_dof_count,
                             float *torque, int64_t ld_torque, int nworld, void *stream);

/* Replaces _compute_muscle_dynamics_activation_grad_sparse_kernel
 * (muscle_dynamics_kernels.py:1796-1859), the body of instantmimic_muscle::torque_backward
 * (warp_custom_ops.py:133-149).  Every element of grad_activation is written (zero where
 * the unit force is zero), so the output needs no clearing. */
int im_muscle_activation_grad(const im_muscle_geometry *geometry,
                              const im_muscle_segments *segments,
                              const im_muscle_entries *muscle_entries, const float *unit_force,
                              int64_t ld_unit, const float *grad_output, int64_t ld_grad_output,
                              int root_dof_count, float *grad_activation,
                              int64_t ld_grad_activation, int nworld, void *stream);

/* Replaces _compute_muscle_dynamics_sparse_bounds_kernel (muscle_dynamics_kernels.py:
 * 1453-1528), the body of instantmimic_muscle::torque_bounds (warp_custom_ops.py:285-303):
 * per torque dof, each muscle's unit-activation torque adds to lower when negative, else to
 * upper.  lower / upper (nworld, ld_bounds >= torque_entries->nrow). */
int im_muscle_torque_bounds(const im_muscle_geometry *geometry,
                            const im_muscle_segments *segments,
                            const im_muscle_entries *torque_entries, const float *unit_force,
                            int64_t ld_unit, int root_dof_count, float *lower, float *upper,
                            int64_t ld_bounds, int nworld, void *stream);

/* Replaces eval_muscle_sparse_moment_kernel
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:2617-2662): moment[w, e] = sum over
 * the segments of (muscle, dof) entry e of the unit-force contribution. */
int im_muscle_sparse_moment(const im_muscle_geometry *geometry,
                            const im_muscle_segments *segments,
                            const int32_t *muscle_dof_torque_idx,
                            const im_muscle_entries *entry_segments, int root_dof_count,
                            float *moment, int64_t ld_moment, int nworld, void *stream);

/* ---- steps either side of the solve that walk a world's small trees ------------------- */

/* Replaces the product M v inside the fused Newton kernel
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:171-176; tables m.M_mulm_rowadr /
 * M_mulm_col / M_mulm_madr of the upstream model, :378-380): out[w, dof] = sum over
 * k in [mulm_rowadr[dof], mulm_rowadr[dof + 1]) of M[w, mulm_madr[k]] * vec[w, mulm_col[k]],
 * accumulated from 0 in table order with one fused multiply-add per term.  nterm = the
 * length of mulm_col and mulm_madr (= mulm_rowadr[nv]; 2 nM - nv for a full symmetric table).
 * M (nworld, ld_M >= nM), vec and out (nworld, ld >= nv); nM and nv below 65536.  skip_world (nworld bytes, may be
 * null): worlds with a nonzero byte keep their out row (the reference's done /
 * search-unchanged worlds). */
int im_mul_m_sparse(const float *M, int64_t ld_M, int nM, const int32_t *mulm_rowadr,
                    const int32_t *mulm_col, const int32_t *mulm_madr, int nterm, const float *vec,
                    int64_t ld_vec, const uint8_t *skip_world, float *out, int64_t ld_out,
                    int nv, int nworld, void *stream);

/* Replaces accumulate_body_tree_deterministic_kernel
 * (src/instantmimic/utils/mjw_kernels/tree_fusion.py:82-113; accumulate(), :137-167), in
 * place: for level = levels - 1 .. 1, every body of level - 1 adds the values of its
 * children among the bodies of `level`, in the order level_bodies lists them (body 0 is
 * never a child; with skip_root_parent the children of body 0 are not added).  The
 * reference's default kernel (:54-80) adds the same children with atomics, that is, in no
 * fixed order.  values (nworld, nbody, components) with ld_world floats between worlds.
 * level_bodies / level_offsets: bodies sorted by depth and the depth offsets
 * (create_tree_reduction_scratch, :35-51). */
int im_tree_accumulate(const int32_t *body_parentid, const int32_t *level_bodies,
                       const int32_t *level_offsets, int levels, int components,
                       int skip_root_parent, float *values, int64_t ld_world, int nbody,
                       int nworld, void *stream);

/* Inputs of the body-wrench projection, all (nworld, ...) float rows with ld floats between
 * worlds: body_force / body_torque / xipos (nbody, 3), subtree_com (nbody, 3),
 * cdof (nvfull, 6); body_rootid (nbody). */
typedef struct im_body_wrenches {
  const float *body_force, *body_torque, *xipos, *subtree_com, *cdof;
  int64_t ld_body_force, ld_body_torque, ld_xipos, ld_subtree_com, ld_cdof;
  const int32_t *body_rootid;
} im_body_wrenches;

/* WrenchProjectionTopology (src/instantmimic/muscle/wrench_projection.py:145-155). */
typedef struct im_wrench_topology {
  const int32_t *dof_bodyid, *body_parentid, *level_bodies, *level_offsets;
  int32_t levels, body_count;
} im_wrench_topology;

/* Replaces project_body_wrenches_to_dofs_kernel (wrench_projection.py:59-136): per body the
 * force and the moment torque + (xipos - subtree_com[root]) x force, folded bottom-up along
 * the body tree, then mean[w, j + output_dof_offset] = cdof_lin . force + cdof_ang . moment
 * of dof j + root_dof_count's body.  The reference folds siblings with atomics (any order);
 * here a parent adds its children in the order of level_bodies, so the result is
 * reproducible.  Any body count that fits 64 KiB of LDS (the reference: 256 bodies). */
int im_project_body_wrenches(const im_body_wrenches *wrenches,
                             const im_wrench_topology *topology, int root_dof_count,
                             int torque_dim, int output_dof_offset, float *mean,
                             int64_t ld_mean, int nworld, void *stream);

/* Replaces gradient_function of the fused Newton kernel
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:745-798), one call for all worlds:
 * a done world only gets search_unchanged = 1; a world whose state_changed_count is 0 gets
 * search_unchanged = 1 and its grad_dot, newton_decrement and grad_scale rescaled by
 * ((grad_scale - alpha) / grad_scale)^2 as there; every other world gets
 * qfrc_constraint[w, dof] = sum over rows r < min(njmax, nefc[w]) ascending of
 * J[w, r, dof] * efc_force[w, r] (one fused multiply-add per row),
 * grad = efc_Ma - qfrc_smooth - qfrc_constraint, grad_dot = grad . grad summed as a block of
 * `block` lanes (32 or 64) sums it -- lane k its dofs k, k + block, .. in order, 32 lanes in
 * a shuffle-down tree, the trees in order (the reference leaves that order to Warp's
 * tile_sum) --, newton_decrement = 0, grad_scale = 1, search_unchanged = 0.
 * J (nworld, njmax, nv) contiguous; nefc and done may be null (all rows, no world done);
 * done and search_unchanged are bytes.  A null state_changed_count counts every world as changed:
 * the first gradient of a solve (upstream's _update_gradient_zero_grad_dot and
 * _update_gradient_grad as src/instantmimic/utils/mjw_kernels/newton_fusion.py:487-500 launches
 * them, with qfrc_constraint = J' efc_force formed here as well). */
int im_newton_gradient(const int32_t *nefc, const float *J, int njmax, const float *efc_force,
                       int64_t ld_force, const float *qfrc_smooth, int64_t ld_smooth,
                       const float *efc_Ma, int64_t ld_Ma, const int32_t *state_changed_count,
                       const float *alpha, const uint8_t *done, float *qfrc_constraint,
                       int64_t ld_constraint, float *grad, int64_t ld_grad, float *grad_dot,
                       float *newton_decrement, float *grad_scale, uint8_t *search_unchanged,
                       int nv, int block, int nworld, void *stream);

/* Replaces the J v step of the fused Newton kernel's line search
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:157-178): jv[w, r] = sum over the dofs
 * of J[w, r, i] * search[w, i] for the rows r < min(njmax, nefc[w]); rows beyond keep their
 * values.  Up to 50 dofs one chain of fused multiply-adds, i ascending; beyond, as the
 * reference does to match upstream, partial sums over 20 dofs each (chains from 0) added to
 * the total one after the other with a rounding of their own.  skip_world (bytes, may be
 * null): worlds that are done or whose search direction did not change keep their jv.
 * J (nworld, njmax, nv) contiguous, search (nworld, ld >= nv), jv (nworld, ld >= njmax). */
int im_newton_jv(const float *J, int njmax, const int32_t *nefc, const float *search,
                 int64_t ld_search, const uint8_t *skip_world, float *jv, int64_t ld_jv, int nv,
                 int nworld, void *stream);

/* ---- implicit-fast integrator matrix ---------------------------------------------------------
 * qH = M - h dF/dv on M's CSR pattern, the matrix that implicit_factor_optimized
 * (src/instantmimic/utils/mjw_step_optimized.py:4936-4968) hands to _factor_solve_i_dense.
 * The reference assembles it with upstream kernels that are not part of its tree
 * (derivative._qderiv_*, forward._implicit_free_body_reset_m, called from deriv_smooth_vel
 * :3803-3900 and _prepare_implicit_qh :3734-3745); the arithmetic here is MuJoCo's published
 * mjd_smooth_vel for this integrator.
 *
 * im_implicit_qh_base: qH[w, e] = M[w, e] + timestep * dof_damping[elem_dof[e]] where
 * elem_dof[e] >= 0 (the diagonal element of a damped dof outside every free body), M[w, e]
 * elsewhere (elem_dof[e] = -1: off-diagonal elements, rows of free bodies, which
 * _prepare_implicit_qh resets to M).  dof_damping (nv) shared by the worlds with
 * ld_damping = 0, or one row per world.  The actuator term -h moment' diag(gain) moment, the
 * tendon-damping term +h J' diag(b) J and the muscle term +h A' diag(s) A are pair sums over
 * sparse rows: im_muscle_implicit_gather adds each of them on top, with pairs in free-body rows
 * left out of its tables. */
int im_implicit_qh_base(const float *M, int64_t ldM, int nM, const int32_t *elem_dof, const float *dof_damping,
                        int64_t ld_damping, float timestep, float *qH, int64_t ld_qH, int nworld, void *stream);

/* One term of qH's derivative part: scale * sum over sparse rows r of weight[w, r] row_r' row_r on M's
 * pattern (actuator moments with the gains as weights and scale -h, tendon Jacobians with the tendon
 * damping and scale +h).  values (nworld, ld_values): the rows' entries as the caller holds them;
 * entry e of the sorted entry list reads values[w, entry_source[e]] (entry_source null: e itself) and
 * belongs to row entry_row[e]; elem_ids / chunk_offsets / chunk_pairs / chunk_count are the gather
 * tables of im_muscle_gather_tables for that entry list.  weight null: the actuator gains computed
 * in the same call. */
typedef struct im_row_pair_term {
  const float *values;
  int64_t ld_values;
  const int32_t *entry_source;
  const int32_t *entry_row;
  int32_t nentry;
  const int32_t *elem_ids;
  int32_t nelem;
  const int32_t *chunk_offsets;
  const int32_t *chunk_pairs;
  int32_t chunk_count;
  const float *weight;
  int64_t ld_weight;
  float scale;
} im_row_pair_term;

/* deriv_smooth_vel (src/instantmimic/utils/mjw_step_optimized.py:3803-3900) in one launch:
 * im_implicit_qh_base, im_actuator_velocity_gain (gain (nworld, ld_gain) is written when not null)
 * and one pair-sum term each for the actuators and the tendons (either may be null), in that order;
 * qH equals the separate calls bit for bit.  A world's row of qH, the gains and the larger term's
 * entries must fit 64 KB of LDS (IM_ERR_UNSUPPORTED otherwise: use the separate calls). */
int im_implicit_qh(const float *M, int64_t ldM, int nM, const int32_t *elem_dof, const float *dof_damping,
                   int64_t ld_damping, float timestep, const int32_t *gaintype, const int32_t *biastype,
                   const float *gainprm, const float *biasprm, int ld_prm, const uint8_t *forcelimited,
                   const float *forcerange, const float *input, int64_t ld_input, const float *force, int64_t ld_force,
                   float *gain, int64_t ld_gain, int nu, const im_row_pair_term *actuators,
                   const im_row_pair_term *tendons, float *qH, int64_t ld_qH, int nworld, void *stream);

/* Replaces the polynomial part of upstream's _qderiv_actuator_passive (dof_dampingpoly with qvel)
 * and _qderiv_tendon_damping (tendon_dampingpoly with ten_velocity), as the reference's
 * deriv_smooth_vel passes them (src/instantmimic/utils/mjw_step_optimized.py:3857-3900): the
 * damping coefficient that the implicit matrix sees,
 *   out[w, i] = base[w, i] + sum over k = 1..nterm of (k + 1) poly[w, i, k - 1] |velocity[w, i]|^k,
 * the slope of a damper whose force is -v (b + p_1 |v| + ... + p_K |v|^K) (Horner's rule, fused
 * multiply-adds, highest term first).  The result goes where the plain damping went:
 * dof_damping of im_implicit_qh / im_implicit_qh_base with its world stride, the tendon term's
 * weight.  ld_base / ld_poly = 0: one set of coefficients for all worlds.  The upstream kernels
 * are not part of the reference's tree; the form of the polynomial is MuJoCo's as this library
 * reads it (coefficients of |v|, |v|^2, ... beside the constant damping). */
int im_polynomial_damping(const float *base, int64_t ld_base, const float *poly, int64_t ld_poly, int nterm,
                          const float *velocity, int64_t ld_velocity, float *out, int64_t ld_out, int n,
                          int nworld, void *stream);

/* Velocity gain of actuators with affine gain / bias (what derivative._qderiv_actuator_passive_vel
 * produces for them, mjw_step_optimized.py:3818-3846): gain[w, a] = biasprm[a, 2] (biastype 1)
 * + gainprm[a, 2] * input[w, a] (gaintype 1), zero when forcelimited[a] and force[w, a] is at or
 * beyond forcerange[a].  input is ctrl, or the activation for stateful actuators.  forcelimited
 * and force may be null. */
int im_actuator_velocity_gain(const int32_t *gaintype, const int32_t *biastype, const float *gainprm,
                              const float *biasprm, int ld_prm, const uint8_t *forcelimited,
                              const float *forcerange, const float *input, int64_t ld_input, const float *force,
                              int64_t ld_force, float *gain, int64_t ld_gain, int nu, int nworld, void *stream);

/* Replaces the step along the search direction at the end of the fused Newton kernel's line
 * search (src/instantmimic/utils/mjw_kernels/newton_stages.py:373-381): for the worlds that
 * are not done, qacc += alpha[w] search and efc_Ma += alpha[w] mv (one fused multiply-add
 * each), Jaref[r] = Jaref[r] + alpha[w] * jv[r] for r < min(njmax, nefc[w]) (product and sum
 * rounded separately: the reference's rounded_step, :18-19).  All arrays (nworld, ld). */
int im_newton_advance(const float *alpha, const float *search, int64_t ld_search, const float *mv,
                      int64_t ld_mv, const float *jv, int64_t ld_jv, const int32_t *nefc,
                      const uint8_t *done, float *qacc, int64_t ld_qacc, float *efc_Ma,
                      int64_t ld_Ma, float *Jaref, int64_t ld_Jaref, int nv, int njmax, int nworld,
                      void *stream);

/* Replaces the scalar search of the fused Newton kernel's line-search stage
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:179-372) for the worlds that are not done:
 * the step length alpha[w] along search that minimises the constraint-solver cost, the cost
 * decrease improvement[w], and ls_exhausted[w] = |alpha| below the noise floor of the line's
 * slope.  The stage's flow is the reference's: Gauss term and equality rows as one quadratic,
 * Newton step from alpha 0, then up to ls_iterations rounds of three candidates (Newton steps from
 * the bracket's ends and its midpoint) with its acceptance tests; sums over 32 lanes by a
 * shuffle-down tree.  The per-row cost model is upstream's (solver._compute_efc_eval_pt_*_pyramidal,
 * not in the reference tree), restated from MuJoCo's primal line search: rows [0, ne) equality,
 * [ne, ne + nf) friction loss, the rest one-sided.  jv and mv are the products J search and
 * M search (im_newton_jv, im_mul_m_sparse).  overflow[w] |= overflow_bit when the rounds run out;
 * tolerance arrays are indexed by w modulo their length.  ne, nf, nefc, done, overflow,
 * efc_frictionloss (with nf) may be null. */
int im_newton_linesearch(const float *opt_tolerance, int ntolerance, const float *opt_ls_tolerance,
                         int nls_tolerance, const float *stat_meaninertia, int nmeaninertia, const int32_t *ne,
                         const int32_t *nf, const int32_t *nefc, int njmax, const float *qfrc_smooth,
                         int64_t ld_smooth, const float *efc_D, int64_t ld_D, const float *efc_frictionloss,
                         int64_t ld_frictionloss, const float *Jaref, int64_t ld_Jaref, const float *search,
                         int64_t ld_search, const float *search_dot, const float *mv, int64_t ld_mv,
                         const float *jv, int64_t ld_jv, const float *efc_Ma, int64_t ld_Ma, const uint8_t *done,
                         int ls_iterations, int overflow_bit, float *alpha, float *improvement,
                         uint8_t *ls_exhausted, int32_t *overflow, int nv, int nworld, void *stream);

/* Replaces the re-evaluation of the constraints that closes the line-search stage
 * (newton_stages.py:385-444, upstream's _eval_constraint for pyramidal cones): from the Jaref
 * that im_newton_advance has moved, efc_force and efc_state of every row below nefc[w] (state 0
 * satisfied, 1 quadratic, 2 / 3 linear negative / positive for friction loss), in place; the rows
 * whose being quadratic flipped, ascending, in quad_changed_ids[w, :] with their count; and
 * state_changed_count[w] = the rows whose state changed, plus one when ls_exhausted[w].  Both
 * counts are zeroed for done worlds, which are otherwise left alone. */
int im_newton_eval_constraints(const float *Jaref, int64_t ld_Jaref, const float *efc_D, int64_t ld_D,
                               const float *efc_frictionloss, int64_t ld_frictionloss, const int32_t *ne,
                               const int32_t *nf, const int32_t *nefc, int njmax, const uint8_t *done,
                               const uint8_t *ls_exhausted, float *efc_force, int64_t ld_force,
                               int32_t *efc_state, int64_t ld_state, int32_t *quad_changed_ids, int ld_ids,
                               int32_t *quad_changed_count, int32_t *state_changed_count, int nworld,
                               void *stream);

/* Replaces the listing of the changed rows that follows it (newton_stages.py:403-426): among
 * the rows r < min(njmax, nefc[w]), those with (old_state == quad) != (new_state == quad) are
 * written to quad_changed_ids[w, :] in ascending order and counted in quad_changed_count[w]
 * (the ids and count that im_sparse_update_factor / im_dense_update_factor take), and
 * state_changed_count[w] = the rows with old_state != new_state (the reference adds one more
 * when its line search is exhausted: the caller's).  The reference evaluates the new states
 * in the same loop with upstream's _eval_constraint and overwrites the old ones in place;
 * here the two state arrays (nworld, njmax) are inputs.  Done worlds are left alone.
 * Integer work: bit-exact. */
int im_newton_changed_rows(const int32_t *old_state, const int32_t *new_state, int njmax,
                           const int32_t *nefc, int quad, const uint8_t *done,
                           int32_t *quad_changed_ids, int ld_ids, int32_t *quad_changed_count,
                           int32_t *state_changed_count, int nworld, void *stream);

/* Replaces the convergence test that closes an iteration of the fused Newton kernel
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:265-296), for the worlds that are not
 * done: niter += 1; scale = stat_meaninertia[w % nmeaninertia] * nv;
 * converged = alpha == 0 || (improvement > 0 && improvement / scale < tol)
 *          || sqrt(grad_dot) / scale < tol || 0.5 * newton_decrement / scale < tol
 * with tol = opt_tolerance[w % ntolerance]; a world that converged or reached maxiter is
 * marked done and taken off *nsolving (one atomic decrement each; may be null), one that
 * reached maxiter without converging gets overflow_bit or-ed into overflow[w] (may be null;
 * upstream's OverflowType.ITERATIONS).  done is bytes. */
int im_newton_converged(const float *alpha, const float *improvement, const float *grad_dot,
                        const float *newton_decrement, const float *opt_tolerance, int ntolerance,
                        const float *stat_meaninertia, int nmeaninertia, int nv, int maxiter,
                        int overflow_bit, int32_t *niter, int32_t *overflow, uint8_t *done,
                        int32_t *nsolving, int nworld, void *stream);

/* Jaref = J qacc - aref for the rows below nefc[w]: what upstream's solver._solve_init_jaref_kernel
 * leaves in ctx.Jaref when the reference's init_context launches it
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:451-468, with its split of a row into
 * 50- or 20-dof stretches).  The sum of a row follows im_newton_jv (one chain of fused
 * multiply-adds up to 50 dofs, 20-dof partial sums added in order beyond; upstream adds the
 * partial sums with atomics, in no fixed order), then aref is subtracted. */
int im_newton_init_jaref(const float *J, int njmax, const int32_t *nefc, const float *qacc, int64_t ld_qacc,
                         const float *aref, int64_t ld_aref, float *Jaref, int64_t ld_Jaref, int nv,
                         int nworld, void *stream);

/* The dense copy of M that upstream's solver._update_gradient starts the Newton Hessian from
 * (called at src/instantmimic/utils/mjw_kernels/newton_fusion.py:470): H (nworld, pad, pad)
 * receives M[w, elemid[i * nv + j]] at (i, j) where elemid (nv x nv, the reference's m.M_elemid
 * layout, -1 outside M's pattern) names an element, zero elsewhere and in the padding. */
int im_dense_from_csr(const float *M, int64_t ldM, const int32_t *elemid, int nv, int pad, float *H,
                      int nworld, void *stream);

/* The factor stage of a Newton iteration on the kinematic tree: for every world whose skip byte
 * is clear (the reference's stage returns for done[w] or state_changes[w] == 0,
 * src/instantmimic/utils/mjw_kernels/newton_stages.py:648-649; ctx.search_unchanged is that flag)
 * H = M + J' diag(D [state == quad]) J is assembled on M's pattern and factored by the tree L'DL
 * (im_assemble_tree_ldl_solve), search = -H^-1 grad, search_dot = search . search and
 * decrement = grad . H^-1 grad summed as the stages of the reference sum them (lane l of `block`
 * lanes adds dofs l, l + block, ..; 32-lane shuffle-down trees; the trees in order:
 * src/instantmimic/utils/mjw_kernels/sparse_hessian.py:462-479).  The reference has no tree stage
 * of its own: for a model whose constraint rows stay on single root-to-leaf chains this is its
 * sparse stage's result computed from the fresh Hessian instead of an incremental update. */
int im_newton_tree_stage(const im_tree_plan *plan, const uint8_t *skip, const float *M, int64_t ldM,
                         const float *J, int njmax, const float *D, const int32_t *state,
                         const int32_t *nefc, int quad, const float *grad, int64_t ldg, float *search,
                         int64_t ld_search, float *search_dot, float *decrement, int block, int nworld,
                         void *stream);

/* The arrays of the fused Newton loop, named as the reference's run() hands them to its kernel
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:330-393).  Rows are contiguous floats or
 * int32: nv per world for qacc, efc_Ma, qfrc_smooth, qfrc_constraint, search, mv; njmax per world
 * for efc_D, efc_frictionloss, efc_force, efc_state, Jaref, jv; one element per world for the
 * scalars; done, ls_exhausted and search_unchanged are bytes.  ne, nf, nefc, efc_frictionloss (with
 * nf), overflow and nsolving may be null.  The tolerance arrays are indexed by world modulo their
 * length. */
typedef struct im_newton_args {
  const float *opt_tolerance, *opt_ls_tolerance, *stat_meaninertia;
  int32_t ntolerance, nls_tolerance, nmeaninertia;
  int32_t ls_iterations, iterations; /* m.opt.ls_iterations, m.opt.iterations */
  int32_t block;                     /* lanes whose summation order the dot products follow: 32 or 64 (newton_block_dim) */
  int32_t quad;                      /* ConstraintState.QUADRATIC */
  int32_t ls_overflow_bit, iterations_overflow_bit; /* OverflowType bits or-ed into overflow */
  const int32_t *M_mulm_rowadr, *M_mulm_col, *M_mulm_madr; /* row tables of M v: nv + 1 offsets, nterm terms */
  int32_t nterm;
  const int32_t *ne, *nf, *nefc;
  const float *M; /* (nworld, ldM) tree CSR */
  int64_t ldM;
  const float *efc_J; /* (nworld, njmax, nv) */
  int32_t njmax;
  const float *efc_D, *efc_frictionloss, *qfrc_smooth;
  float *qacc, *efc_Ma, *efc_force;
  int32_t *efc_state;
  float *Jaref, *search, *search_dot, *mv, *jv, *alpha, *improvement;
  float *grad; /* (nworld, ld_grad) */
  int64_t ld_grad;
  float *grad_dot, *grad_scale, *newton_decrement, *qfrc_constraint;
  int32_t *quad_changed_ids; /* (nworld, ld_ids) */
  int32_t ld_ids;
  int32_t *quad_changed_count, *state_changed_count, *solver_niter, *overflow, *nsolving;
  uint8_t *done, *ls_exhausted, *search_unchanged;
  int32_t nworld;
} im_newton_args;

/* Replaces the part of init_context before the first Hessian
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:431-500: _init_efc_settling_empty_worlds,
 * Jaref = J qacc - aref, Ma = M qacc, upstream's _update_constraint and the first gradient) in
 * one launch, a wavefront per world: solver_niter = 0, search_dot = 0, done = (nefc == 0), a world
 * without constraint rows gets qacc = qacc_smooth; then for every world efc_Ma, and for the others
 * Jaref, efc_force, efc_state with the list and the counts of changed rows, qfrc_constraint, grad,
 * grad_dot, newton_decrement = 0, grad_scale = 1, search_unchanged = done.  The same operations in
 * the same order as im_newton_init_empty_worlds, im_newton_init_jaref, im_mul_m_sparse,
 * im_newton_eval_constraints and im_newton_gradient called one after the other (the same bits);
 * the caller's first factor stage follows.  args as for im_newton_solve_tree; nv, nM: dofs and
 * length of a row of M. */
int im_newton_init_context(const im_newton_args *args, const float *qacc_smooth, int64_t ld_qacc_smooth,
                           const float *efc_aref, int64_t ld_aref, int nv, int nM, void *stream);

/* Replaces the launch of solve_incremental_newton_kernel
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:57-298, launched at :396-409) for a model
 * whose factor stage is the tree stage of im_newton_tree_stage: one resident kernel, a wavefront per
 * world and four worlds per workgroup, that iterates every world from the state init_context left
 * until it converges or m.opt.iterations is reached -- M search, J search, line search, step,
 * constraint states, gradient, factor stage, convergence test, with the operations of
 * im_mul_m_sparse, im_newton_jv, im_newton_linesearch, im_newton_advance,
 * im_newton_eval_constraints, im_newton_gradient, im_newton_tree_stage and im_newton_converged in
 * their order, so the arrays end as after those launches repeated, bit for bit.  No host
 * synchronisation, nothing allocated; the loop is bounded by `iterations` whatever the data.
 * Needs generated kernels on the plan (IM_ERR_UNSUPPORTED otherwise: the caller then issues the
 * stages one by one).  The launch holds as many workgroups as the chip keeps resident; a wavefront
 * whose world is done takes the next world through a counter that belongs to the plan, so two solves
 * with one plan must not overlap on the GPU. */
int im_newton_solve_tree(const im_tree_plan *plan, const im_newton_args *args, void *stream);

/* The same resident loop with the static-pattern sparse stage of im_sparse_update_factor as its
 * factor stage, which is the reference's kernel for a model with a fused sparse plan
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:150-169 with sparse_hessian.native_func):
 * hfactor (nworld, nv_pad, nv_pad) carries packed H, the factor and 1 / D as im_sparse_init_factor
 * left them and is kept up to date, dof_union (nworld, nv + 1) receives the dofs the changed rows
 * touch.  A wavefront per world, up to sixteen worlds per workgroup sharing one copy of the plan's
 * tables in LDS; a wavefront leaves as soon as its world is done.  args->block must be the plan's
 * block width.  The arrays end as after im_sparse_update_factor and the other stage launches
 * repeated, bit for bit.  nv <= 64 (IM_ERR_UNSUPPORTED beyond, and where no variant of the kernel
 * fits the LDS: the caller then issues the stages one by one).  The launch holds as many
 * wavefronts as the chip keeps resident and hands a finished wavefront the next world through a
 * counter that belongs to the plan: two solves with one plan must not overlap on the GPU. */
int im_newton_solve_sparse(const im_sparse_plan *plan, const im_newton_args *args, float *hfactor,
                           int32_t *dof_union, void *stream);

/* The same launch for a dense model of up to 32 dofs, whose factor stage is the single-tile branch
 * of the reference's stage (src/instantmimic/utils/mjw_kernels/newton_stages.py:723-733, inside
 * the loop of newton_fusion.py:57-298): one resident kernel, a wavefront per world, the stage of
 * im_dense_update_tile once per round for the worlds whose states changed.  H: ctx.h,
 * (nworld, nv_pad, nv_pad), updated in place; dof_union (nworld, nv + 1) as in
 * im_dense_update_tile.  next_world: one int32 of the caller's on the device, the batch's world
 * counter (two solves that share it must not overlap on the GPU).  Leaves the arrays as nv <= 32
 * launches of the stages would.  IM_ERR_UNSUPPORTED beyond 32 dofs and where a CU's LDS does not
 * hold four worlds. */
int im_newton_solve_dense_tile(const im_newton_args *args, float *H, int32_t *dof_union, int nv, int nv_pad, int nM,
                               int32_t *next_world, void *stream);

/* The same for a dense model of 33 to 63 dofs with nv_pad = 48 or 64, whose factor stage is the
 * augmented blocked Cholesky (newton_stages.py:473-611, 614-742) run as im_dense_update_column
 * runs it, a wavefront per world with a lane per column.  U: ctx.hfactor, (nworld, nv_pad, nv_pad).
 * IM_ERR_UNSUPPORTED for other shapes. */
int im_newton_solve_dense_column(const im_newton_args *args, float *H, float *U, int32_t *dof_union, int nv, int nv_pad,
                                 int nM, int32_t *next_world, void *stream);

/* Replaces _init_efc_settling_empty_worlds
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:412-428): solver_niter = 0,
 * search_dot = 0, done = (nefc == 0), and a world without constraint rows gets
 * qacc = qacc_smooth (MuJoCo's result for nefc == 0), so it starts done. */
int im_newton_init_empty_worlds(const int32_t *nefc, const float *qacc_smooth, int64_t ld_smooth,
                                int32_t *solver_niter, float *search_dot, uint8_t *done,
                                float *qacc, int64_t ld_qacc, int nv, int nworld, void *stream);

/* Replaces qfrc_constraint_from_grad (newton_fusion.py:537-555):
 * qfrc_constraint = efc_Ma - qfrc_smooth - grad_scale[w] * grad, zero for a world without
 * constraint rows. */
int im_qfrc_constraint_from_grad(const int32_t *nefc, const float *qfrc_smooth, int64_t ld_smooth,
                                 const float *efc_Ma, int64_t ld_Ma, const float *grad,
                                 int64_t ld_grad, const float *grad_scale, float *qfrc_constraint,
                                 int64_t ld_constraint, int nv, int nworld, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* IMHIP_H_ */
