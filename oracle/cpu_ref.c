/* CPU oracle: fp32 restatement of the reference's numeric statements for the
 * assemble + tree L'DL + solve path.  TEST INFRASTRUCTURE ONLY -- nothing in the
 * shipped library links or calls this file; it is the checker the HIP kernels
 * are compared with, and the timed "cpu_baseline" of the benchmark.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fopenmp).  Every fused
 * multiply-add is written as fmaf(); everything else rounds once per operator.
 *
 * Rounding convention of the tree L'DL.  The reference writes plain expressions
 *     t = t - a * b * c;   s = s - a * b;
 * (src/instantmimic/utils/mjw_kernels/tree_ldl.py:227-231, 269, 302) and leaves
 * contraction to the compiler.  NVRTC (fmad on by default) and clang both
 * contract the multiply that feeds the subtraction, so the statements evaluate as
 *     t = fmaf(-(a * b), c, t);   s = fmaf(-a, b, s);
 * which is what this file does.  Reciprocals are correctly rounded 1.0f / x.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void orc_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* H = M + sum over QUADRATIC rows of D * J' J on M's CSR entries.
 * Per entry (a = column = ancestor dof, b = row dof, a <= b) the rows are summed
 * in ascending order with v = fmaf(J[r][a] * Dc[r], J[r][b], v), Dc = D for a
 * QUADRATIC row and 0 otherwise (sparse_hessian.py:589, 622-629). */
static void assemble_world(int nv, int nM, const int *rowi, const int *colind,
                           const float *M, const float *J, const float *D,
                           const int *state, int nefc, int quad, float *H) {
  for (int e = 0; e < nM; ++e) H[e] = M[e];
  for (int r = 0; r < nefc; ++r) {
    const float dc = state[r] == quad ? D[r] : 0.0f;
    const float *Jr = J + (size_t)r * nv;
    for (int e = 0; e < nM; ++e) {
      const int a = colind[e], b = rowi[e];
      H[e] = fmaf(Jr[a] * dc, Jr[b], H[e]);
    }
  }
}

int orc_assemble_csr(int nworld, int nv, int nM, const int *rowi,
                     const int *colind, const float *M, const float *J,
                     int njmax, const float *D, const int *state,
                     const int *nefc, int quad, float *H) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    int n = nefc ? nefc[w] : njmax;
    if (n > njmax) n = njmax;
    assemble_world(nv, nM, rowi, colind, M + (size_t)w * nM,
                   J + (size_t)w * njmax * nv, D + (size_t)w * njmax,
                   state + (size_t)w * njmax, n, quad, H + (size_t)w * nM);
  }
  return 0;
}

/* Static description of one tree plan (tree_ldl.py:47-56 plus the CSR). */
typedef struct {
  int nv, nM, ngroups, ntrunk, nte; /* nte = trunk CSR entries */
  const int *rowadr, *rownnz, *colind;
  const int *gptr, *gdofs, *trunk;
  int *slot;     /* CSR entry -> trunk entry slot or -1 */
  int *dslot;    /* dof -> trunk dof slot or -1 */
  char *touch_m; /* [ngroups][nte]  */
  char *touch_s; /* [ngroups][ntrunk] */
} plan_t;

static void plan_init(plan_t *p) {
  p->slot = (int *)malloc(sizeof(int) * (p->nM + 1));
  p->dslot = (int *)malloc(sizeof(int) * (p->nv + 1));
  for (int e = 0; e < p->nM; ++e) p->slot[e] = -1;
  for (int i = 0; i < p->nv; ++i) p->dslot[i] = -1;
  int n = 0;
  for (int t = 0; t < p->ntrunk; ++t) {
    const int i = p->trunk[t];
    p->dslot[i] = t;
    for (int e = p->rowadr[i]; e < p->rowadr[i] + p->rownnz[i]; ++e) p->slot[e] = n++;
  }
  p->nte = n;
  p->touch_m = (char *)calloc((size_t)p->ngroups * (n + 1), 1);
  p->touch_s = (char *)calloc((size_t)p->ngroups * (p->ntrunk + 1), 1);
  /* tree_ldl.py:236-245 */
  for (int j = 0; j < p->ngroups; ++j)
    for (int g = p->gptr[j]; g < p->gptr[j + 1]; ++g) {
      const int k = p->gdofs[g];
      for (int q = 0; q < p->rownnz[k] - 1; ++q) {
        const int anc = p->colind[p->rowadr[k] + q];
        if (p->dslot[anc] < 0) continue;
        p->touch_s[j * p->ntrunk + p->dslot[anc]] = 1;
        for (int c = 0; c <= q; ++c) p->touch_m[j * n + p->slot[p->rowadr[anc] + c]] = 1;
      }
    }
}

static void plan_free(plan_t *p) {
  free(p->slot);
  free(p->dslot);
  free(p->touch_m);
  free(p->touch_s);
}

/* One world.  work holds m[nM], s[nv], d[nv], xs[nv], a[ngroups*nte],
 * b[ngroups*ntrunk].  ld (optional) receives the factor: scaled rows of L with
 * the unscaled pivot on the diagonal. */
static void tree_world(const plan_t *p, const float *H, const float *y, float *x,
                       float *work, float *ld) {
  const int nv = p->nv, nM = p->nM, nte = p->nte, nt = p->ntrunk;
  float *m = work, *s = m + nM, *d = s + nv, *xs = d + nv;
  float *a = xs + nv, *b = a + (size_t)p->ngroups * nte;
  memcpy(m, H, sizeof(float) * nM);
  memcpy(s, y, sizeof(float) * nv);
  for (int i = 0; i < p->ngroups * nte; ++i) a[i] = 0.0f;
  for (int i = 0; i < p->ngroups * nt; ++i) b[i] = 0.0f;
  /* parts, forward (tree_ldl.py:215-232, 252-259) */
  for (int j = 0; j < p->ngroups; ++j) {
    float *aj = a + (size_t)j * nte, *bj = b + (size_t)j * nt;
    for (int g = p->gptr[j]; g < p->gptr[j + 1]; ++g) {
      const int k = p->gdofs[g], start = p->rowadr[k], count = p->rownnz[k] - 1;
      const float dk = 1.0f / m[start + count];
      d[k] = dk;
      for (int pp = 0; pp < count; ++pp) {
        const int anc = p->colind[start + pp];
        for (int q = 0; q <= pp; ++q) {
          const int e = p->rowadr[anc] + q;
          float *t = p->dslot[anc] >= 0 ? &aj[p->slot[e]] : &m[e];
          *t = fmaf(-(m[start + pp] * m[start + q]), dk, *t);
        }
      }
      for (int pp = 0; pp < count; ++pp) m[start + pp] = m[start + pp] * dk;
      for (int pp = 0; pp < count; ++pp) {
        const int anc = p->colind[start + pp];
        float *t = p->dslot[anc] >= 0 ? &bj[p->dslot[anc]] : &s[anc];
        *t = fmaf(-m[start + pp], s[k], *t);
      }
    }
  }
  /* trunk (tree_ldl.py:274-305) */
  for (int t = 0; t < nt; ++t) {
    const int i = p->trunk[t];
    for (int e = p->rowadr[i]; e < p->rowadr[i] + p->rownnz[i]; ++e) {
      float v = H[e];
      for (int j = 0; j < p->ngroups; ++j)
        if (p->touch_m[j * nte + p->slot[e]]) v = v + a[(size_t)j * nte + p->slot[e]];
      m[e] = v;
    }
    float v = y[i];
    for (int j = 0; j < p->ngroups; ++j)
      if (p->touch_s[j * nt + t]) v = v + b[(size_t)j * nt + t];
    s[i] = v;
  }
  for (int t = nt - 1; t >= 0; --t) {
    const int k = p->trunk[t], start = p->rowadr[k], count = p->rownnz[k] - 1;
    const float dk = 1.0f / m[start + count];
    d[k] = dk;
    for (int pp = 0; pp < count; ++pp) {
      const int anc = p->colind[start + pp];
      for (int q = 0; q <= pp; ++q) {
        float *tt = &m[p->rowadr[anc] + q];
        *tt = fmaf(-(m[start + pp] * m[start + q]), dk, *tt);
      }
    }
    for (int pp = 0; pp < count; ++pp) m[start + pp] = m[start + pp] * dk;
    for (int pp = 0; pp < count; ++pp) {
      float *tt = &s[p->colind[start + pp]];
      *tt = fmaf(-m[start + pp], s[k], *tt);
    }
  }
  for (int t = 0; t < nt; ++t) {
    const int i = p->trunk[t], start = p->rowadr[i];
    float u = s[i] * d[i];
    for (int pp = 0; pp < p->rownnz[i] - 1; ++pp)
      u = fmaf(-m[start + pp], xs[p->colind[start + pp]], u);
    xs[i] = u;
  }
  /* parts, backward (tree_ldl.py:262-272) */
  for (int j = 0; j < p->ngroups; ++j)
    for (int g = p->gptr[j + 1] - 1; g >= p->gptr[j]; --g) {
      const int i = p->gdofs[g], start = p->rowadr[i];
      float v = s[i] * d[i];
      for (int pp = 0; pp < p->rownnz[i] - 1; ++pp)
        v = fmaf(-m[start + pp], xs[p->colind[start + pp]], v);
      xs[i] = v;
    }
  memcpy(x, xs, sizeof(float) * nv);
  if (ld) memcpy(ld, m, sizeof(float) * nM);
}

static size_t work_floats(const plan_t *p) {
  return (size_t)p->nM + 3 * (size_t)p->nv +
         (size_t)p->ngroups * (p->nte + p->ntrunk) + 8;
}

/* x = (L'DL)^-1 y for every world; H (nworld, nM) in M's CSR layout. */
int orc_tree_ldl_solve(int nworld, int nv, int nM, const int *rowadr,
                       const int *rownnz, const int *colind, int ngroups,
                       const int *gptr, const int *gdofs, int ntrunk,
                       const int *trunk, const float *H, const float *y,
                       float *x, float *ld) {
  plan_t p = {nv, nM, ngroups, ntrunk, 0, rowadr, rownnz, colind, gptr, gdofs, trunk, 0, 0, 0, 0};
  plan_init(&p);
  const size_t wf = work_floats(&p);
#pragma omp parallel
  {
    float *work = (float *)malloc(sizeof(float) * wf);
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w)
      tree_world(&p, H + (size_t)w * nM, y + (size_t)w * nv, x + (size_t)w * nv,
                 work, ld ? ld + (size_t)w * nM : 0);
    free(work);
  }
  plan_free(&p);
  return 0;
}

/* The fused path: assemble H on the CSR pattern, factor and solve with y = grad.
 * Hout (optional) receives the assembled H. */
int orc_assemble_tree_ldl_solve(int nworld, int nv, int nM, const int *rowadr,
                                const int *rownnz, const int *colind,
                                const int *rowi, int ngroups, const int *gptr,
                                const int *gdofs, int ntrunk, const int *trunk,
                                const float *M, const float *J, int njmax,
                                const float *D, const int *state,
                                const int *nefc, int quad, const float *grad,
                                float *x, float *Hout) {
  plan_t p = {nv, nM, ngroups, ntrunk, 0, rowadr, rownnz, colind, gptr, gdofs, trunk, 0, 0, 0, 0};
  plan_init(&p);
  const size_t wf = work_floats(&p);
#pragma omp parallel
  {
    float *work = (float *)malloc(sizeof(float) * (wf + nM));
    float *H = work + wf;
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      int n = nefc ? nefc[w] : njmax;
      if (n > njmax) n = njmax;
      assemble_world(nv, nM, rowi, colind, M + (size_t)w * nM,
                     J + (size_t)w * njmax * nv, D + (size_t)w * njmax,
                     state + (size_t)w * njmax, n, quad, H);
      if (Hout) memcpy(Hout + (size_t)w * nM, H, sizeof(float) * nM);
      tree_world(&p, H, grad + (size_t)w * nv, x + (size_t)w * nv, work, 0);
    }
    free(work);
  }
  plan_free(&p);
  return 0;
}

/* ------------------------------------------------------------------ muscle contractions
 * Rounding convention: the reference's kernels are Warp Python (`total += a * b`), which
 * Warp lowers to add(total, mul(a, b)) in CUDA C++ and NVRTC contracts to one fused
 * multiply-add; the restatement spells those fmaf()s. */

/* tau[w, root + j] = sum over the entries of torque dof j, in torque-sorted order, of
 * moment[w, e] * force[w, muscle(e)]
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:2941-2961). */
int orc_muscle_project(int nworld, int nentry, int nmuscle, int ntorque, const float *moment,
                       const float *force, const int *offsets, const int *entry_idx,
                       const int *entry_muscle, int root, float *qfrc, int ldq) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    const float *m = moment + (size_t)w * nentry, *f = force + (size_t)w * nmuscle;
    for (int j = 0; j < ntorque; ++j) {
      float total = 0.0f;
      for (int s = offsets[j]; s < offsets[j + 1]; ++s) {
        const int e = entry_idx[s];
        total = fmaf(m[e], f[entry_muscle[e]], total);
      }
      qfrc[(size_t)w * ldq + root + j] = total;
    }
  }
  return 0;
}

/* qderiv[w, elem] += timestep * sum over the element's chunks (in order) of the chunk's
 * 16-pair sum of (slope[w, muscle(i)] * moment[w, i]) * moment[w, j]
 * (muscle_qfrc_projector.py:677-708 serial variant, 736-774 block variant). */
int orc_muscle_implicit_gather(int nworld, int nentry, int nmuscle, int nelem, int chunk_count,
                               int chunk, const float *moment, const float *slope,
                               const int *entry_muscle, const int *elem_ids,
                               const int *chunk_offsets, const int *chunk_pairs,
                               float timestep, float *qderiv, int ldq) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    const float *m = moment + (size_t)w * nentry, *sl = slope + (size_t)w * nmuscle;
    for (int slot = 0; slot < nelem; ++slot) {
      float acc = 0.0f;
      for (int c = chunk_offsets[slot]; c < chunk_offsets[slot + 1]; ++c) {
        float total = 0.0f;
        for (int k = 0; k < chunk; ++k) {
          const int packed = chunk_pairs[(size_t)k * chunk_count + c];
          const int i = packed & 0xFFFF, j = packed >> 16;
          if (i < nentry) {
            const float weighted = sl[entry_muscle[i]] * m[i];
            total = fmaf(weighted, m[j], total);
          }
        }
        acc = acc + total;
      }
      float *q = qderiv + (size_t)w * ldq + elem_ids[slot];
      *q = fmaf(timestep, acc, *q);
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ static-pattern sparse L'DL
 * Restatement of the reference's initial assemble + factor + solve kernel
 * (src/instantmimic/utils/mjw_kernels/sparse_hessian.py: assembly 578-630, level factor
 * 410-452, backward solve and sums 453-479) executed lane by lane: the result depends on
 * which lane of a team sums which terms and on the shuffle tree, so both are emulated.
 * Plain `a - b * c` expressions of the CUDA snippet contract to fmaf(-b, c, a). */
typedef struct {
  int nv, nv_pad, block, nslots, nlevels;
  const int *LP, *LT, *ES, *EC, *RP, *RAB, *RKL, *ORIG, *BL, *BS, *BI, *BJ, *PM, *SA, *SB, *SM;
} sparse_t;

/* level-scheduled numeric factor (sparse_hessian.py:410-452), team lanes emulated */
static void sp_factor_levels(const sparse_t *p, float *N, float *iD) {
  for (int l = 0; l < p->nlevels; ++l) {
    const int T = p->LT[l];
    for (int e = p->LP[l]; e < p->LP[l + 1]; ++e) {
      float part[32];
      for (int tl = 0; tl < T; ++tl) {
        float v = 0.0f;
        for (int r = p->RP[e]; r < p->RP[e + 1]; ++r) {
          const unsigned ab = (unsigned)p->RAB[r], kl = (unsigned)p->RKL[r];
          const float *pa = N + (ab & 0xFFFFu), *pb = N + (ab >> 16), *pd = iD + (kl & 0xFFFFu);
          const int len = (int)(kl >> 16);
          for (int t = tl; t < len; t += T) v = fmaf(pa[t] * pb[t], pd[t], v);
        }
        part[tl] = v;
      }
      for (int off = T >> 1; off > 0; off >>= 1)
        for (int i = 0; i < off; ++i) part[i] = part[i] + part[i + off];
      /* entries of one level never read what the level writes, so in-place is a sweep */
      const float wv = N[p->ES[e]] - part[0];
      N[p->ES[e]] = wv;
      if (p->EC[e] >= 0) iD[p->EC[e]] = 1.0f / wv;
    }
  }
}

/* backward pushes, search = -x and the two sums (sparse_hessian.py:453-479) */
static void sp_backward_sums(const sparse_t *p, float *N, const float *iD, const float *grad,
                             float *search, float *sdot, float *decr) {
  const int n = p->nv, nfac = p->nslots - n, rhs = nfac, block = p->block;
  for (int l = 0; l < p->nlevels; ++l)
    for (int q = p->BL[l]; q < p->BL[l + 1]; ++q) {
      const int i = p->BI[q], j = p->BJ[q];
      N[rhs + j] = fmaf(-N[p->BS[q]], N[rhs + i] * iD[i], N[rhs + j]);
    }
  /* per-lane sums, 32-lane shuffle tree, warps added in order */
  float s0[128] = {0}, s1[128] = {0};
  for (int lane = 0; lane < block; ++lane)
    for (int j = lane; j < n; j += block) {
      const int d = p->ORIG[j];
      const float v = N[rhs + j] * iD[j];
      search[d] = -v;
      s0[lane] = fmaf(v, v, s0[lane]);
      s1[lane] = fmaf(grad[d], v, s1[lane]);
    }
  float ra = 0.0f, rb = 0.0f;
  for (int wv = 0; wv < (block + 31) / 32; ++wv) {
    float *a = s0 + 32 * wv, *b = s1 + 32 * wv;
    for (int off = 16; off > 0; off >>= 1)
      for (int i = 0; i < off; ++i) {
        a[i] = a[i] + a[i + off];
        b[i] = b[i] + b[i + off];
      }
    ra = ra + a[0];
    rb = rb + b[0];
  }
  *sdot = ra;
  *decr = rb;
}

static void sparse_world(const sparse_t *p, const float *J, int njmax, const float *D,
                         const int *state, int nefc, int quad, const float *M, const float *grad,
                         float *U, float *search, float *sdot, float *decr, float *N) {
  const int n = p->nv, nfac = p->nslots - n, rhs = nfac;
  float *iD = N + p->nslots;
  const int words = (n + 31) / 32;
  for (int s = 0; s < nfac; ++s) N[s] = p->SM[s] >= 0 ? M[p->SM[s]] : 0.0f;
  if (nefc > njmax) nefc = njmax;
  for (int k = 0; k < nefc; k += 4) {
    float Dc[4];
    const float *Jr[4];
    static const float zero_row[1024] = {0};
    for (int r = 0; r < 4; ++r) {
      const int row = k + r;
      Dc[r] = (row < nefc && state[row] == quad) ? D[row] : 0.0f;
      Jr[r] = row < nefc ? J + (size_t)row * n : zero_row;
    }
    /* pattern check: every active row's support must lie inside the pattern */
    for (int r = 0; r < 4; ++r) {
      if (Dc[r] == 0.0f) continue;
      unsigned rm[32] = {0};
      for (int d = 0; d < n; ++d)
        if (Jr[r][d] != 0.0f) rm[d / 32] |= 1u << (d % 32);
      int bad = 0;
      for (int d = 0; d < n; ++d)
        if ((rm[d / 32] >> (d % 32)) & 1u)
          for (int q = 0; q < words; ++q) bad |= (rm[q] & ~(unsigned)p->PM[d * words + q]) != 0u;
      if (bad) U[p->nv_pad * p->nv_pad - 1] += 1.0f;
    }
    for (int s = 0; s < nfac; ++s) {
      const int a = p->SA[s], b = p->SB[s];
      float v = N[s];
      for (int r = 0; r < 4; ++r) v = fmaf(Jr[r][a] * Dc[r], Jr[r][b], v);
      N[s] = v;
    }
  }
  for (int s = 0; s < nfac; ++s) U[s] = N[s];
  for (int j = 0; j < n; ++j) N[rhs + j] = grad[p->ORIG[j]];
  sp_factor_levels(p, N, iD);
  for (int s = 0; s < nfac; ++s) U[nfac + s] = N[s];
  for (int j = 0; j < n; ++j) U[2 * nfac + j] = iD[j];
  sp_backward_sums(p, N, iD, grad, search, sdot, decr);
}

int orc_sparse_init_factor(int nv, int nv_pad, int block, int nslots, int nlevels,
                           const int *const *tables, int nworld, const unsigned char *done,
                           const int *nefc, const float *J, int njmax, const float *D,
                           const int *state, int quad, const float *M, int ldM, const float *grad,
                           int ldg, float *hfactor, float *search, float *sdot, float *decr) {
  sparse_t p = {nv, nv_pad, block, nslots, nlevels, tables[0], tables[1], tables[2], tables[3],
                tables[4], tables[5], tables[6], tables[7], tables[8], tables[9], tables[10],
                tables[11], tables[12], tables[13], tables[14], tables[15]};
  if (nv > 1024 || block > 64) return 1;
#pragma omp parallel
  {
    float *N = (float *)malloc(sizeof(float) * (nslots + nv + 8));
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      if (done && done[w]) continue;
      sparse_world(&p, J + (size_t)w * njmax * nv, njmax, D + (size_t)w * njmax,
                   state + (size_t)w * njmax, nefc[w], quad, M + (size_t)w * ldM,
                   grad + (size_t)w * ldg, hfactor + (size_t)w * nv_pad * nv_pad,
                   search + (size_t)w * nv, sdot + w, decr + w, N);
    }
    free(N);
  }
  return 0;
}

/* Changed rows' dof union in ascending order and the incremental update of one H entry
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:451-470, 651-701;
 * sparse_hessian.py:505-523): delta = fold over the changed rows t, in list order, of
 * fmaf(+-D a, b, delta), the sign negative when the row's new state is not QUADRATIC,
 * rows that do not reach both dofs skipped. */
static int dof_union(int n, const float *J, const int *ids, int count, int *uni) {
  int m = 0;
  for (int d = 0; d < n; ++d)
    for (int t = 0; t < count; ++t)
      if (J[(size_t)ids[t] * n + d] != 0.0f) {
        uni[m++] = d;
        break;
      }
  uni[n] = m;
  return m;
}
static float pair_delta(int n, const float *J, const float *D, const int *state, int quad,
                        const int *ids, int count, int row, int col) {
  float delta = 0.0f;
  for (int t = 0; t < count; ++t) {
    const int r = ids[t];
    const float a = J[(size_t)r * n + row], b = J[(size_t)r * n + col];
    float da = D[r] * a;
    if (state[r] != quad) da = -da;
    if (a != 0.0f && b != 0.0f) delta = fmaf(da, b, delta);
  }
  return delta;
}

/* Per-iteration factor stage on the static pattern (sparse_hessian.py:488-547 with the
 * factor kept in hfactor between calls instead of in a resident block's shared memory):
 * count > 0: update packed H through SH_PAIR, refactor (mode 0); count == 0: forward solve
 * with the stored factor (modes 2 + 1).  tables[16..21] = SH_PAIR, SH_FL, SH_FR, SH_RS,
 * SH_RKP, SH_RK. */
int orc_sparse_update_factor(int nv, int nv_pad, int block, int nslots, int nlevels,
                             const int *const *tables, int nworld, const unsigned char *done,
                             const int *state_changes, const int *changes, const int *ids,
                             int ld_ids, const float *J, int njmax, const float *D,
                             const int *state, int quad, const float *grad, int ldg,
                             float *hfactor, int *uni_out, float *search, float *sdot,
                             float *decr) {
  sparse_t p = {nv, nv_pad, block, nslots, nlevels, tables[0], tables[1], tables[2], tables[3],
                tables[4], tables[5], tables[6], tables[7], tables[8], tables[9], tables[10],
                tables[11], tables[12], tables[13], tables[14], tables[15]};
  const int *PAIR = tables[16], *FL = tables[17], *FR = tables[18], *RS = tables[19],
            *RKP = tables[20], *RK = tables[21];
  const int n = nv, nfac = nslots - nv, rhs = nfac;
  if (nv > 1024 || block > 64) return 1;
#pragma omp parallel
  {
    float *N = (float *)malloc(sizeof(float) * (nslots + nv + 8));
    float *iD = N + nslots;
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      if ((done && done[w]) || state_changes[w] == 0) continue;
      float *U = hfactor + (size_t)w * nv_pad * nv_pad;
      const float *Jw = J + (size_t)w * njmax * n, *Dw = D + (size_t)w * njmax;
      const int *sw = state + (size_t)w * njmax, *idw = ids + (size_t)w * ld_ids;
      const float *g = grad + (size_t)w * ldg;
      int *uni = uni_out + (size_t)w * (n + 1);
      const int count = changes[w] < ld_ids ? changes[w] : ld_ids;
      if (count > 0) {
        const int nu = dof_union(n, Jw, idw, count, uni);
        for (int cj = 0; cj < nu; ++cj)
          for (int ri = 0; ri <= cj; ++ri) {
            const int row = uni[ri], col = uni[cj];
            const float delta = pair_delta(n, Jw, Dw, sw, quad, idw, count, row, col);
            if (delta != 0.0f) {
              const int sl = PAIR[row * n + col];
              if (sl >= 0) U[sl] = U[sl] + delta;
              else U[nv_pad * nv_pad - 1] += 1.0f;
            }
          }
        for (int s = 0; s < nfac; ++s) N[s] = U[s];
        for (int j = 0; j < n; ++j) N[rhs + j] = g[p.ORIG[j]];
        sp_factor_levels(&p, N, iD);
        for (int s = 0; s < nfac; ++s) U[nfac + s] = N[s];
        for (int j = 0; j < n; ++j) U[2 * nfac + j] = iD[j];
      } else {
        for (int s = 0; s < nfac; ++s) N[s] = U[nfac + s];
        for (int j = 0; j < n; ++j) iD[j] = U[2 * nfac + j];
        for (int l = 0; l < nlevels; ++l)
          for (int q = FL[l]; q < FL[l + 1]; ++q) {
            const int j = FR[q];
            float v = g[p.ORIG[j]];
            const float *rowp = N + RS[j];
            for (int t = 0; t < RKP[j + 1] - RKP[j]; ++t) {
              const int k = RK[RKP[j] + t];
              v = fmaf(-(rowp[t] * iD[k]), N[rhs + k], v);
            }
            N[rhs + j] = v;
          }
      }
      sp_backward_sums(&p, N, iD, g, search + (size_t)w * n, sdot + w, decr + w);
    }
    free(N);
  }
  return 0;
}

/* Factor step of the upstream (non-fused) iteration (sparse_hessian.py:639-679, modes 4 / 5,
 * dispatched as in nonfused_kernel :849-894): refactor from the dense H through SH_GAT, or solve
 * with the stored factor; hfactor = [0, nfac) N, [nfac, nfac + n) 1 / D.  tables[16..21] as in
 * orc_sparse_update_factor, tables[22] = SH_GAT. */
int orc_sparse_dense_factor(int nv, int nv_pad, int block, int nslots, int nlevels,
                            const int *const *tables, int nworld, const unsigned char *done,
                            const float *grad, int ldg, const float *H, const int *quad_changed,
                            const int *state_changed, int skip_unchanged, int skip_noflip,
                            float *hfactor, float *search, float *sdot, float *decr) {
  sparse_t p = {nv, nv_pad, block, nslots, nlevels, tables[0], tables[1], tables[2], tables[3],
                tables[4], tables[5], tables[6], tables[7], tables[8], tables[9], tables[10],
                tables[11], tables[12], tables[13], tables[14], tables[15]};
  const int *FL = tables[17], *FR = tables[18], *RS = tables[19], *RKP = tables[20],
            *RK = tables[21], *GAT = tables[22];
  const int n = nv, nfac = nslots - nv, rhs = nfac;
  if (nv > 1024 || block > 128) return 1;
#pragma omp parallel
  {
    float *N = (float *)malloc(sizeof(float) * (nslots + nv + 8));
    float *iD = N + nslots;
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      if (done && done[w]) continue;
      if (skip_noflip && state_changed[w] == 0) continue;
      float *U = hfactor + (size_t)w * nv_pad * nv_pad;
      const float *Hw = H + (size_t)w * nv_pad * nv_pad, *g = grad + (size_t)w * ldg;
      if (!(skip_unchanged && quad_changed[w] == 0)) {
        for (int s = 0; s < nfac; ++s) N[s] = Hw[GAT[s]];
        for (int j = 0; j < n; ++j) N[rhs + j] = g[p.ORIG[j]];
        sp_factor_levels(&p, N, iD);
        for (int s = 0; s < nfac; ++s) U[s] = N[s];
        for (int j = 0; j < n; ++j) U[nfac + j] = iD[j];
      } else {
        for (int s = 0; s < nfac; ++s) N[s] = U[s];
        for (int j = 0; j < n; ++j) iD[j] = U[nfac + j];
        for (int l = 0; l < nlevels; ++l)
          for (int q = FL[l]; q < FL[l + 1]; ++q) {
            const int j = FR[q];
            float v = g[p.ORIG[j]];
            const float *rowp = N + RS[j];
            for (int t = 0; t < RKP[j + 1] - RKP[j]; ++t) {
              const int k = RK[RKP[j] + t];
              v = fmaf(-(rowp[t] * iD[k]), N[rhs + k], v);
            }
            N[rhs + j] = v;
          }
      }
      sp_backward_sums(&p, N, iD, g, search + (size_t)w * n, sdot + w, decr + w);
    }
    free(N);
  }
  return 0;
}

/* ------------------------------------------------------------------ Newton line search
 * Lane-by-lane restatement of the reference's line-search stage
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:79-444): 32 lanes stride the dofs and the
 * rows, sums go through a shuffle-down tree whose lane 0 is broadcast.  The per-row cost model
 * (solver._compute_efc_eval_pt_*_pyramidal, _eval_pt, _in_bracket, _eval_constraint, safe_div,
 * _ALPHA_NOISE_EPS) is upstream mujoco_warp code absent from the reference tree: it is restated
 * from MuJoCo's published primal line search, so bit-level parity with upstream is UNPINNED; the
 * tests pin it to the exact minimiser of the line's cost in fp64. */
typedef struct {
  float c, g, h;
} pt3;
static pt3 pt_add(pt3 a, pt3 b) { pt3 r = {a.c + b.c, a.g + b.g, a.h + b.h}; return r; }
static float ls_safe_div(float x, float y) { return x / (y != 0.0f ? y : 1.0e-15f); }
static pt3 ls_eval_pt(pt3 q, float a) {
  pt3 r = {a * a * q.h + a * q.g + q.c, 2.0f * a * q.h + q.g, 2.0f * q.h};
  return r;
}
static int ls_in_bracket(pt3 x, pt3 y) { return (x.g < y.g && y.g < 0.0f) || (x.g > y.g && y.g > 0.0f); }
static pt3 ls_row_quad(int friction, float D, float f, float jaref, float jv, float x) {
  pt3 quad = {0.5f * jaref * jaref * D, jv * jaref * D, 0.5f * jv * jv * D};
  pt3 zero = {0.0f, 0.0f, 0.0f};
  if (friction) {
    const float rf = ls_safe_div(f, D);
    if (x <= -rf) { pt3 r = {f * (-0.5f * rf - jaref), -f * jv, 0.0f}; return r; }
    if (x >= rf) { pt3 r = {f * (-0.5f * rf + jaref), f * jv, 0.0f}; return r; }
    return quad;
  }
  return x < 0.0f ? quad : zero;
}
static pt3 ls_row_point(int friction, float D, float f, float jaref, float jv, float alpha) {
  pt3 p = ls_eval_pt(ls_row_quad(friction, D, f, jaref, jv, jaref + alpha * jv), alpha);
  p.c = p.c - ls_row_quad(friction, D, f, jaref, jv, jaref).c;
  return p;
}
static float ls_tree(float *a) {
  for (int off = 16; off > 0; off >>= 1)
    for (int i = 0; i < off; ++i) a[i] = a[i] + a[i + off];
  return a[0] + 0.0f;
}
typedef struct {
  int ne, nf, nefc;
  const float *D, *fl, *Jaref, *jv;
} ls_rows;
/* sum over the rows [ne, nefc) of the row points at alpha (zero != 0: the absolute point at alpha 0) */
static pt3 ls_rows_at(const ls_rows *R, float alpha, int zero) {
  float c[32] = {0}, g[32] = {0}, h[32] = {0};
  for (int lane = 0; lane < 32; ++lane)
    for (int r = R->ne + lane; r < R->nefc; r += 32) {
      const int fr = r < R->ne + R->nf;
      const float f = R->fl ? R->fl[r] : 0.0f;
      pt3 p;
      if (zero) {
        const pt3 q = ls_row_quad(fr, R->D[r], f, R->Jaref[r], R->jv[r], R->Jaref[r]);
        p.c = q.c, p.g = q.g, p.h = 2.0f * q.h;
      } else {
        p = ls_row_point(fr, R->D[r], f, R->Jaref[r], R->jv[r], alpha);
      }
      c[lane] = c[lane] + p.c, g[lane] = g[lane] + p.g, h[lane] = h[lane] + p.h;
    }
  pt3 out = {ls_tree(c), ls_tree(g), ls_tree(h)};
  return out;
}

int orc_newton_linesearch(int nworld, int nv, int njmax, const float *tolerance, int ntol,
                          const float *ls_tolerance, int nls, const float *meaninertia, int nmi,
                          const int *ne_, const int *nf_, const int *nefc_, const float *smooth,
                          const float *D, const float *frictionloss, const float *Jaref,
                          const float *search, const float *search_dot, const float *mv,
                          const float *jv, const float *Ma, const unsigned char *done,
                          int ls_iterations, int overflow_bit, float *alpha_out, float *improvement_out,
                          unsigned char *exhausted, int *overflow) {
  const float noise = 0x1p-20f;
  for (int w = 0; w < nworld; ++w) {
    if (done && done[w]) continue;
    ls_rows R = {ne_ ? ne_[w] : 0, nf_ ? nf_[w] : 0, 0, D + (size_t)w * njmax,
                 frictionloss ? frictionloss + (size_t)w * njmax : NULL, Jaref + (size_t)w * njmax,
                 jv + (size_t)w * njmax};
    R.nefc = nefc_ ? nefc_[w] : njmax;
    if (R.nefc > njmax) R.nefc = njmax;
    const float snorm = sqrtf(search_dot[w]);
    const float scale = meaninertia[w % nmi] * (float)nv;
    const float gtol = fmaxf(tolerance[w % ntol] * ls_tolerance[w % nls] * snorm * scale, 1.0e-6f);
    float a1[32] = {0}, a2[32] = {0};
    for (int lane = 0; lane < 32; ++lane) {
      for (int dof = lane; dof < nv; dof += 32) {
        const float sv = search[(size_t)w * nv + dof];
        a1[lane] = a1[lane] + sv * (Ma[(size_t)w * nv + dof] - smooth[(size_t)w * nv + dof]);
        a2[lane] = a2[lane] + 0.5f * sv * mv[(size_t)w * nv + dof];
      }
      for (int r = lane; r < R.ne; r += 32) {
        const float jvD = R.jv[r] * R.D[r];
        a1[lane] = a1[lane] + jvD * R.Jaref[r];
        a2[lane] = a2[lane] + 0.5f * R.jv[r] * jvD;
      }
    }
    pt3 gauss = {0.0f, 0.0f, 0.0f};
    gauss.g = ls_tree(a1);
    gauss.h = ls_tree(a2);
    const pt3 rows0 = ls_rows_at(&R, 0.0f, 1);
    const pt3 p0 = {gauss.c + rows0.c, gauss.g + rows0.g, 2.0f * gauss.h + rows0.h};
    const pt3 p0_delta = {0.0f, p0.g, p0.h};
    const float q1_abs = sqrtf(2.0f * fmaxf(rows0.c, 0.0f) * fmaxf(rows0.h, 0.0f)) + fabsf(gauss.g);
    const float gtol_accept = fmaxf(gtol, noise * q1_abs);
    const float noise_floor = noise * fmaxf(1.0f, ls_safe_div(q1_abs, p0.h));
    float alpha = 0.0f, improvement = 0.0f;
    int converged = fabsf(p0.g) < noise * q1_abs;
    const float lo_alpha_in = -ls_safe_div(p0.g, p0.h);
    pt3 lo_in = {0.0f, 0.0f, 0.0f};
    if (!converged) {
      lo_in = pt_add(ls_eval_pt(gauss, lo_alpha_in), ls_rows_at(&R, lo_alpha_in, 0));
      if (fabsf(lo_in.g) < gtol_accept && lo_in.c < 0.0f) {
        converged = 1;
        alpha = lo_alpha_in;
        improvement = -lo_in.c;
      }
    }
    if (!converged) {
      const int lo_less = lo_in.g < p0.g;
      pt3 lo = lo_less ? lo_in : p0_delta, hi = lo_less ? p0_delta : lo_in;
      float lo_alpha = lo_less ? lo_alpha_in : 0.0f, hi_alpha = lo_less ? 0.0f : lo_alpha_in;
      for (int it = 0; it < ls_iterations; ++it) {
        const float lo_next_alpha = lo_alpha - ls_safe_div(lo.g, lo.h);
        const float hi_next_alpha = hi_alpha - ls_safe_div(hi.g, hi.h);
        const float mid_alpha = 0.5f * (lo_alpha + hi_alpha);
        const pt3 lo_next = pt_add(ls_eval_pt(gauss, lo_next_alpha), ls_rows_at(&R, lo_next_alpha, 0));
        const pt3 hi_next = pt_add(ls_eval_pt(gauss, hi_next_alpha), ls_rows_at(&R, hi_next_alpha, 0));
        const pt3 mid = pt_add(ls_eval_pt(gauss, mid_alpha), ls_rows_at(&R, mid_alpha, 0));
        const int conv_lo = fabsf(lo_next.g) < gtol_accept && lo_next.c < 0.0f;
        const int conv_hi = fabsf(hi_next.g) < gtol_accept && hi_next.c < 0.0f;
        const int conv_mid = fabsf(mid.g) < gtol_accept && mid.c < 0.0f;
        const int conv = conv_lo || conv_hi || conv_mid;
        int swap_lo = 0, swap_hi = 0;
        if (conv) {
          pt3 best = {1.0e10f, 0.0f, 0.0f};
          float best_alpha = 0.0f;
          if (conv_lo && lo_next.c < best.c) best = lo_next, best_alpha = lo_next_alpha;
          if (conv_hi && hi_next.c < best.c) best = hi_next, best_alpha = hi_next_alpha;
          if (conv_mid && mid.c < best.c) best = mid, best_alpha = mid_alpha;
          lo = hi = best;
          lo_alpha = hi_alpha = best_alpha;
        } else {
          const int s1 = ls_in_bracket(lo, lo_next);
          if (s1) lo = lo_next, lo_alpha = lo_next_alpha;
          const int s2 = ls_in_bracket(lo, mid);
          if (s2) lo = mid, lo_alpha = mid_alpha;
          const int s3 = ls_in_bracket(lo, hi_next);
          if (s3) lo = hi_next, lo_alpha = hi_next_alpha;
          swap_lo = s1 || s2 || s3;
          const int t1 = ls_in_bracket(hi, hi_next) || (hi.g < 0.0f && hi_next.g > 0.0f);
          if (t1) hi = hi_next, hi_alpha = hi_next_alpha;
          const int t2 = ls_in_bracket(hi, mid);
          if (t2) hi = mid, hi_alpha = mid_alpha;
          const int t3 = ls_in_bracket(hi, lo_next);
          if (t3) hi = lo_next, hi_alpha = lo_next_alpha;
          swap_hi = t1 || t2 || t3;
        }
        const int ls_done = conv || (!swap_lo && !swap_hi) || (lo.c < 0.0f && lo.g < 0.0f && lo.g > -gtol) ||
                            (hi.c < 0.0f && hi.g > 0.0f && hi.g < gtol);
        if (lo.c < 0.0f || hi.c < 0.0f) {
          const int lo_better = lo.c < hi.c;
          alpha = lo_better ? lo_alpha : hi_alpha;
          improvement = -(lo_better ? lo.c : hi.c);
        }
        if (ls_done) {
          converged = 1;
          break;
        }
      }
    }
    alpha_out[w] = alpha;
    improvement_out[w] = improvement;
    exhausted[w] = fabsf(alpha) < noise_floor;
    if (!converged && overflow) overflow[w] |= overflow_bit;
  }
  return 0;
}

/* force and state of every row from the new Jaref, ascending list of the rows whose being
 * QUADRATIC flipped, counts (newton_stages.py:385-444; upstream's _eval_constraint restated) */
int orc_newton_eval_constraints(int nworld, int njmax, const float *Jaref, const float *D,
                                const float *frictionloss, const int *ne_, const int *nf_,
                                const int *nefc_, const unsigned char *done,
                                const unsigned char *exhausted, float *force, int *state, int *ids,
                                int ld_ids, int *quad_count, int *state_count) {
  for (int w = 0; w < nworld; ++w) {
    quad_count[w] = 0;
    state_count[w] = 0;
    if (done && done[w]) continue;
    const int ne = ne_ ? ne_[w] : 0, nf = nf_ ? nf_[w] : 0;
    int nefc = nefc_ ? nefc_[w] : njmax;
    if (nefc > njmax) nefc = njmax;
    int nq = 0, ns = 0;
    for (int r = 0; r < nefc; ++r) {
      const size_t k = (size_t)w * njmax + r;
      const float x = Jaref[k], d = D[k];
      float f = -d * x;
      int s = 1;
      if (r >= ne && r < ne + nf) {
        const float fr = frictionloss[k], rf = ls_safe_div(fr, d);
        if (x <= -rf) f = fr, s = 2;
        else if (x >= rf) f = -fr, s = 3;
      } else if (r >= ne && x >= 0.0f) {
        f = 0.0f, s = 0;
      }
      const int old = state[k];
      force[k] = f;
      state[k] = s;
      if ((old == 1) != (s == 1)) {
        if (nq < ld_ids) ids[(size_t)w * ld_ids + nq] = r;
        ++nq;
      }
      ns += old != s;
    }
    quad_count[w] = nq;
    state_count[w] = ns + (exhausted && exhausted[w] ? 1 : 0);
  }
  return 0;
}

/* The damping coefficient the implicit matrix sees from a damper with polynomial terms: the
 * slope of  -v (b + p_1 |v| + ... + p_K |v|^K), i.e.  b + sum_k (k + 1) p_k |v|^k, by Horner's rule
 * from the highest term (upstream's derivative._qderiv_actuator_passive / _qderiv_tendon_damping
 * take dof_dampingpoly / tendon_dampingpoly beside the plain coefficients:
 * src/instantmimic/utils/mjw_step_optimized.py:3857-3900; the kernels themselves are third party
 * and absent).  ld_base / ld_poly = 0: shared by all worlds. */
int orc_polynomial_damping(int nworld, int n, int nterm, const float *base, long ld_base,
                           const float *poly, long ld_poly, const float *velocity, long ld_velocity,
                           float *out, long ld_out) {
  for (int w = 0; w < nworld; ++w)
    for (int i = 0; i < n; ++i) {
      const float a = fabsf(velocity[(size_t)w * ld_velocity + i]);
      const float *p = poly + (size_t)w * ld_poly + (size_t)i * nterm;
      float acc = 0.0f;
      for (int k = nterm; k >= 1; --k) acc = fmaf(acc, a, (float)(k + 1) * p[k - 1]);
      out[(size_t)w * ld_out + i] = fmaf(acc, a, base[(size_t)w * ld_base + i]);
    }
  return 0;
}

/* ------------------------------------------------------------------ implicit-fast integrator matrix
 * qH = M + h damping on the diagonal elements of damped dofs outside free bodies (elem_dof >= 0),
 * M elsewhere; and the velocity gain of affine actuators.  MuJoCo's published mjd_smooth_vel
 * (the reference calls upstream kernels that are not in its tree:
 * src/instantmimic/utils/mjw_step_optimized.py:3803-3900, 3734-3745). */
int orc_implicit_qh_base(int nworld, int nM, const float *M, int ldM, const int *elem_dof,
                         const float *damping, int ld_damping, float timestep, float *out, int ldo) {
  for (int w = 0; w < nworld; ++w)
    for (int e = 0; e < nM; ++e) {
      const float v = M[(size_t)w * ldM + e];
      out[(size_t)w * ldo + e] =
          elem_dof[e] >= 0 ? fmaf(timestep, damping[(size_t)w * ld_damping + elem_dof[e]], v) : v;
    }
  return 0;
}

int orc_actuator_velocity_gain(int nworld, int nu, const int *gaintype, const int *biastype,
                               const float *gainprm, const float *biasprm, int ldprm,
                               const unsigned char *forcelimited, const float *forcerange,
                               const float *input, const float *force, float *gain) {
  for (int w = 0; w < nworld; ++w)
    for (int a = 0; a < nu; ++a) {
      float v = 0.0f;
      if (biastype[a] == 1) v = biasprm[a * ldprm + 2];
      if (gaintype[a] == 1) v = fmaf(gainprm[a * ldprm + 2], input[(size_t)w * nu + a], v);
      if (forcelimited && forcelimited[a] && force) {
        const float f = force[(size_t)w * nu + a];
        if (f <= forcerange[2 * a] || f >= forcerange[2 * a + 1]) v = 0.0f;
      }
      gain[(size_t)w * nu + a] = v;
    }
  return 0;
}

/* ------------------------------------------------------------------ blocked dense Cholesky
 * Restatement of the indexed blocked upper Cholesky factor + solve
 * (src/instantmimic/utils/mjw_kernels/indexed_factor.py:15-173; block index layout and
 * identity padding of src/instantmimic/utils/mjw_step_optimized.py:893-955).  The block
 * schedule is the reference's; the arithmetic inside a tile is Warp's tile library
 * (third party, absent), so the order INSIDE a tile operation is this file's own
 * convention ("parity unpinned" at bit level, pinned to fp64 algebra by the tests):
 *   matmul(A', B, C, alpha=-1):  sum = fold_t fmaf(A[t][r], B[t][c], sum) from 0; C = C - sum
 *   cholesky (lower L, U = L'):  s = A[j][j]; s = fmaf(-L[j][k], L[j][k], s) k ascending;
 *                                L[j][j] = sqrtf(s); inv = 1 / L[j][j];
 *                                L[i][j] = (A[i][j] - fold_k L[i][k] L[j][k]) * inv
 *   lower solve L z = b:         column oriented, j ascending: z[j] = s[j] * (1 / L[j][j]);
 *                                s[i] = fmaf(-L[i][j], z[j], s[i]) for i > j
 *   upper solve U x = b:         column oriented, r descending: x[r] = s[r] * (1 / U[r][r]);
 *                                s[t] = fmaf(-U[t][r], x[r], s[t]) for t < r */
/* One tile element.  bidx != NULL: indexed gather from the CSR values with +1 on padded
 * diagonal entries; bidx == NULL: M is a dense (pad, pad) matrix whose rows and columns
 * >= nv count as the identity. */
static float tile_elem(int nv, int pad, int B, int nM, const float *M, const int *bidx, int kb,
                       int ib, int e) {
  const int nblk = pad / B, r = e / B, c = e % B;
  if (!bidx) {
    const int row = kb * B + r, col = ib * B + c;
    /* only the upper triangle is kept up to date: mirror it inside a diagonal tile */
    if (row < nv && col < nv) return row <= col ? M[(size_t)row * pad + col] : M[(size_t)col * pad + row];
    return row == col ? 1.0f : 0.0f;
  }
  const int idx = bidx[(size_t)(kb * nblk + ib) * B * B + e];
  float v = idx < nM ? M[idx] : 0.0f;
  if (ib == kb && (kb + 1) * B > nv && r == c && (nblk - 1) * B + r >= nv) v = v + 1.0f;
  return v;
}

/* factor U'U = A with rhs <- U'^-1 rhs fused into the block loop */
static void blocked_factor_forward(int nv, int pad, int B, int nM, const float *M, const int *bidx,
                                   float *U, float *rhs, float *A, float *L) {
  const int nblk = pad / B, BB = B * B;
  for (int i = 0; i < pad * pad; ++i) U[i] = 0.0f;
  for (int kb = 0; kb < nblk; ++kb) {
    const int k = kb * B;
    for (int e = 0; e < BB; ++e) A[e] = tile_elem(nv, pad, B, nM, M, bidx, kb, kb, e);
    for (int jb = 0; jb < kb; ++jb) {
      const int j = jb * B;
      for (int r = 0; r < B; ++r)
        for (int c = 0; c < B; ++c) {
          float sum = 0.0f;
          for (int t = 0; t < B; ++t) sum = fmaf(U[(j + t) * pad + k + r], U[(j + t) * pad + k + c], sum);
          A[r * B + c] = A[r * B + c] - sum;
        }
      for (int r = 0; r < B; ++r) {
        float sum = 0.0f;
        for (int t = 0; t < B; ++t) sum = fmaf(U[(j + t) * pad + k + r], rhs[j + t], sum);
        rhs[k + r] = rhs[k + r] - sum;
      }
    }
    for (int j = 0; j < B; ++j) {
      float s = A[j * B + j];
      for (int q = 0; q < j; ++q) s = fmaf(-L[j * B + q], L[j * B + q], s);
      const float d = sqrtf(s), inv = 1.0f / d;
      L[j * B + j] = d;
      for (int i = j + 1; i < B; ++i) {
        float v = A[i * B + j];
        for (int q = 0; q < j; ++q) v = fmaf(-L[i * B + q], L[j * B + q], v);
        L[i * B + j] = v * inv;
      }
    }
    for (int r = 0; r < B; ++r)
      for (int c = r; c < B; ++c) U[(k + r) * pad + k + c] = L[c * B + r];
    for (int j = 0; j < B; ++j) {
      const float z = rhs[k + j] * (1.0f / L[j * B + j]);
      rhs[k + j] = z;
      for (int i = j + 1; i < B; ++i) rhs[k + i] = fmaf(-L[i * B + j], z, rhs[k + i]);
    }
    for (int ib = kb + 1; ib < nblk; ++ib) {
      const int i0 = ib * B;
      for (int e = 0; e < BB; ++e) A[e] = tile_elem(nv, pad, B, nM, M, bidx, kb, ib, e);
      for (int jb = 0; jb < kb; ++jb) {
        const int j = jb * B;
        for (int r = 0; r < B; ++r)
          for (int c = 0; c < B; ++c) {
            float sum = 0.0f;
            for (int t = 0; t < B; ++t) sum = fmaf(U[(j + t) * pad + k + r], U[(j + t) * pad + i0 + c], sum);
            A[r * B + c] = A[r * B + c] - sum;
          }
      }
      for (int c = 0; c < B; ++c)
        for (int j = 0; j < B; ++j) {
          const float z = A[j * B + c] * (1.0f / L[j * B + j]);
          A[j * B + c] = z;
          for (int i = j + 1; i < B; ++i) A[i * B + c] = fmaf(-L[i * B + j], z, A[i * B + c]);
        }
      for (int r = 0; r < B; ++r)
        for (int c = 0; c < B; ++c) U[(k + r) * pad + i0 + c] = A[r * B + c];
    }
  }
}

/* rhs <- U^-1 rhs */
static void blocked_backward(int pad, int B, const float *U, float *rhs) {
  for (int i0 = pad - B; i0 >= 0; i0 -= B) {
    for (int j = i0 + B; j < pad; j += B)
      for (int r = 0; r < B; ++r) {
        float sum = 0.0f;
        for (int t = 0; t < B; ++t) sum = fmaf(U[(i0 + r) * pad + j + t], rhs[j + t], sum);
        rhs[i0 + r] = rhs[i0 + r] - sum;
      }
    for (int r = B - 1; r >= 0; --r) {
      const float xv = rhs[i0 + r] * (1.0f / U[(i0 + r) * pad + i0 + r]);
      rhs[i0 + r] = xv;
      for (int t = 0; t < r; ++t) rhs[i0 + t] = fmaf(-U[(i0 + t) * pad + i0 + r], xv, rhs[i0 + t]);
    }
  }
}

/* rhs <- U'^-1 rhs with a finished factor: the operations factor_forward applies to rhs */
static void blocked_forward(int pad, int B, const float *U, float *rhs) {
  for (int k = 0; k < pad; k += B) {
    for (int j = 0; j < k; j += B)
      for (int r = 0; r < B; ++r) {
        float sum = 0.0f;
        for (int t = 0; t < B; ++t) sum = fmaf(U[(j + t) * pad + k + r], rhs[j + t], sum);
        rhs[k + r] = rhs[k + r] - sum;
      }
    for (int j = 0; j < B; ++j) {
      const float z = rhs[k + j] * (1.0f / U[(k + j) * pad + k + j]);
      rhs[k + j] = z;
      for (int i = j + 1; i < B; ++i) rhs[k + i] = fmaf(-U[(k + j) * pad + k + i], z, rhs[k + i]);
    }
  }
}

static void blocked_world(int nv, int pad, int B, int nM, const float *M, const int *bidx,
                          const float *y, float *U, float *x, float *rhs, float *A, float *L) {
  for (int i = 0; i < pad; ++i) rhs[i] = i < nv ? y[i] : 0.0f;
  blocked_factor_forward(nv, pad, B, nM, M, bidx, U, rhs, A, L);
  blocked_backward(pad, B, U, rhs);
  for (int i = 0; i < nv; ++i) x[i] = rhs[i];
}


int orc_blocked_factor_solve(int nworld, int nv, int pad, int B, int nM, const float *M, int ldM,
                             const int *block_idx, const float *y, float *U, float *x) {
#pragma omp parallel
  {
    float *work = (float *)malloc(sizeof(float) * (pad + 2 * B * B + 8));
    float *Ul = U ? 0 : (float *)malloc(sizeof(float) * pad * pad);
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w)
      blocked_world(nv, pad, B, nM, M + (size_t)w * ldM, block_idx, y + (size_t)w * nv,
                    U ? U + (size_t)w * pad * pad : Ul, x + (size_t)w * nv, work, work + pad,
                    work + pad + B * B);
    free(work);
    free(Ul);
  }
  return 0;
}

/* x = (U'U)^-1 y for nrhs columns from a stored factor: per column the forward and backward
 * substitution blocked_world applies to its single right-hand side
 * (src/instantmimic/utils/mjw_kernels/indexed_factor.py:394-493); y and x (nworld, nv, nrhs),
 * worlds with active[w] == 0 are left alone. */
int orc_blocked_multi_solve(int nworld, int nv, int pad, int B, const float *U, const float *y,
                            int nrhs, const int *active, float *x) {
#pragma omp parallel
  {
    float *rhs = (float *)malloc(sizeof(float) * pad);
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      if (active && active[w] == 0) continue;
      const float *Uw = U + (size_t)w * pad * pad;
      for (int c = 0; c < nrhs; ++c) {
        for (int i = 0; i < pad; ++i) rhs[i] = i < nv ? y[((size_t)w * nv + i) * nrhs + c] : 0.0f;
        blocked_forward(pad, B, Uw, rhs);
        blocked_backward(pad, B, Uw, rhs);
        for (int i = 0; i < nv; ++i) x[((size_t)w * nv + i) * nrhs + c] = rhs[i];
      }
    }
    free(rhs);
  }
  return 0;
}

/* Cholesky of one tile that fits a block (up to 64 x 64) and the solve of one right-hand side
 * with it, nothing kept: src/instantmimic/utils/mjw_step_optimized.py:672-750 (the two
 * "no L store" tile kernels) and the nv <= 32 branch of the Newton factor stage
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:723-733).  The reference takes the
 * arithmetic from Warp's tile library (third party, absent); here the tile is factored as a
 * diagonal tile of the blocked factor is: row i of L from A's row i, column by column,
 *   v = A[i][j]; for q < j ascending: v = fmaf(-L[i][q], L[j][q], v); L[i][j] = v * (1 / L[j][j]),
 * pivots sqrtf of the same chain; then the two substitutions, column oriented.
 * A: the lower triangle, row major with row length n; s: right-hand side in, solution out. */
static void tile_factor_solve(int n, const float *A, float *L, float *s) {
  for (int j = 0; j < n; ++j) {
    float p = A[j * n + j];
    for (int q = 0; q < j; ++q) p = fmaf(-L[j * n + q], L[j * n + q], p);
    const float d = sqrtf(p), inv = 1.0f / d;
    L[j * n + j] = d;
    for (int i = j + 1; i < n; ++i) {
      float v = A[i * n + j];
      for (int q = 0; q < j; ++q) v = fmaf(-L[i * n + q], L[j * n + q], v);
      L[i * n + j] = v * inv;
    }
  }
  for (int j = 0; j < n; ++j) {
    const float z = s[j] * (1.0f / L[j * n + j]);
    s[j] = z;
    for (int i = j + 1; i < n; ++i) s[i] = fmaf(-L[i * n + j], z, s[i]);
  }
  for (int r = n - 1; r >= 0; --r) {
    const float xv = s[r] * (1.0f / L[r * n + r]);
    s[r] = xv;
    for (int t = 0; t < r; ++t) s[t] = fmaf(-L[r * n + t], xv, s[t]);
  }
}

/* x[adr[t] .. + size) = tile_t^-1 y[same] for every world and tile.  elemid == NULL: M is dense,
 * (ld_world per world, ld_row per row), tile t the diagonal block at adr[t], its lower triangle
 * read (:672-701).  elemid != NULL: M holds nM values per world and tile t's element (r, c) is
 * M[elemid[t size size + r size + c]], the upper triangle read (:704-750); an id at or past nM
 * reads as zero. */
int orc_tile_cholesky_solve(int nworld, int size, int ntile, const int *adr, const float *M,
                            long ld_world, long ld_row, const int *elemid, int nM, const float *y,
                            long ldy, float *x, long ldx) {
  if (size < 1 || size > 64) return 1;
#pragma omp parallel
  {
    float *A = (float *)malloc(sizeof(float) * (2 * (size_t)size * size + size));
    float *L = A + (size_t)size * size, *s = L + (size_t)size * size;
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w)
      for (int t = 0; t < ntile; ++t) {
        const float *Mw = M + (size_t)w * ld_world;
        const int a0 = adr[t];
        for (int i = 0; i < size; ++i)
          for (int c = 0; c <= i; ++c) {
            if (elemid) {
              const int id = elemid[((size_t)t * size + c) * size + i];
              A[i * size + c] = id < nM ? Mw[id] : 0.0f;
            } else {
              A[i * size + c] = Mw[(size_t)(a0 + i) * ld_row + a0 + c];
            }
          }
        for (int i = 0; i < size; ++i) s[i] = y[(size_t)w * ldy + a0 + i];
        tile_factor_solve(size, A, L, s);
        for (int i = 0; i < size; ++i) x[(size_t)w * ldx + a0 + i] = s[i];
      }
    free(A);
  }
  return 0;
}

/* Per-iteration factor stage on the dense Hessian (src/instantmimic/utils/mjw_kernels/
 * newton_stages.py:614-742): incremental update of H's upper triangle over the changed
 * rows' dof union (:451-470, 651-701), then the augmented blocked Cholesky (:473-611; the
 * gradient as column pad - 1, corner 1e30) or, without changed rows, a solve with the stored
 * factor.  The tile arithmetic and the order of the two final sums are this file's
 * conventions (the reference's come from Warp's tile library and mujoco_warp's
 * block_cholesky, both third party): 64 lanes stride the dofs, shuffle-down tree.  Up to 32
 * dofs the stage keeps no factor (:723-733): after the update H is factored as one tile
 * (tile_factor_solve) at every call, U is not touched. */
int orc_dense_update_factor(int nworld, int nv, int pad, const unsigned char *done,
                            const int *state_changes, const int *changes, const int *ids,
                            int ld_ids, const float *J, int njmax, const float *D,
                            const int *state, int quad, const float *grad, int ldg, float *H,
                            float *Uout, int *uni_out, float *search, float *sdot, float *decr) {
  const int B = 16;
#pragma omp parallel
  {
    float *work = (float *)malloc(sizeof(float) * ((size_t)pad * pad + pad + 2 * 32 * 32 + 8));
    float *U = work, *rhs = U + (size_t)pad * pad, *A = rhs + pad, *L = A + 32 * 32;
    const int single = nv <= 32;
#pragma omp for schedule(static)
    for (int w = 0; w < nworld; ++w) {
      if ((done && done[w]) || state_changes[w] == 0) continue;
      float *Hw = H + (size_t)w * pad * pad, *Uw = Uout + (size_t)w * pad * pad;
      const float *Jw = J + (size_t)w * njmax * nv, *Dw = D + (size_t)w * njmax;
      const int *sw = state + (size_t)w * njmax, *idw = ids + (size_t)w * ld_ids;
      const float *g = grad + (size_t)w * ldg;
      int *uni = uni_out + (size_t)w * (nv + 1);
      /* a negative count: no row is applied, H is factored as it is (the first factor of a solve) */
      const int refactor = changes[w] != 0;
      const int count = changes[w] < 0 ? 0 : (changes[w] < ld_ids ? changes[w] : ld_ids);
      for (int i = 0; i < pad; ++i) rhs[i] = i < nv ? g[i] : 0.0f;
      if (refactor || single) {
        const int nu = dof_union(nv, Jw, idw, count, uni);
        for (int cj = 0; cj < nu; ++cj)
          for (int ri = 0; ri <= cj; ++ri) {
            const int row = uni[ri], col = uni[cj];
            const float delta = pair_delta(nv, Jw, Dw, sw, quad, idw, count, row, col);
            if (delta != 0.0f) Hw[(size_t)row * pad + col] = Hw[(size_t)row * pad + col] + delta;
          }
      }
      if (single) {
        for (int i = 0; i < nv; ++i)
          for (int c = 0; c <= i; ++c) A[i * nv + c] = Hw[(size_t)c * pad + i];
        tile_factor_solve(nv, A, L, rhs);
      } else if (refactor) {
        blocked_factor_forward(nv, pad, B, 0, Hw, 0, U, rhs, A, L);
        float corner = 1.0e30f;
        for (int i = 0; i < nv; ++i) corner = fmaf(-rhs[i], rhs[i], corner);
        for (int i = 0; i < pad * pad; ++i) Uw[i] = U[i];
        for (int i = 0; i < nv; ++i) Uw[(size_t)i * pad + pad - 1] = rhs[i];
        Uw[(size_t)(pad - 1) * pad + pad - 1] = sqrtf(corner);
      } else {
        for (int i = 0; i < pad * pad; ++i) U[i] = Uw[i];
        for (int i = 0; i < pad; ++i) U[(size_t)i * pad + pad - 1] = i == pad - 1 ? 1.0f : 0.0f;
        blocked_forward(pad, B, U, rhs);
      }
      if (!single) blocked_backward(pad, B, U, rhs);
      float s0[128] = {0}, s1[128] = {0};
      for (int lane = 0; lane < 64; ++lane)
        for (int i = lane; i < nv; i += 64) {
          const float v = rhs[i];
          search[(size_t)w * nv + i] = -v;
          s0[lane] = fmaf(v, v, s0[lane]);
          s1[lane] = fmaf(g[i], v, s1[lane]);
        }
      for (int off = 32; off > 0; off >>= 1)
        for (int i = 0; i < off; ++i) {
          s0[i] = s0[i] + s0[i + off];
          s1[i] = s1[i] + s1[i + off];
        }
      sdot[w] = s0[0];
      decr[w] = s1[0];
    }
    free(work);
  }
  return 0;
}

/* Dense H = M + J' diag(D [state == quad]) J into (nv_pad, nv_pad) per world, rows summed
 * in ascending order with fmaf(J[r][i] * Dc, J[r][j], h) starting from M (upper and lower
 * triangle filled).  The reference takes this from mujoco_warp's solver (third party,
 * absent); call sites src/instantmimic/utils/mjw_kernels/newton_fusion.py:470. */
int orc_jtdj_dense(int nworld, int nv, int nv_pad, const float *Mdense, const float *J, int njmax,
                   const float *D, const int *state, const int *nefc, int quad, float *H) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    float *h = H + (size_t)w * nv_pad * nv_pad;
    const float *m = Mdense + (size_t)w * nv * nv;
    int n = nefc ? nefc[w] : njmax;
    if (n > njmax) n = njmax;
    for (int i = 0; i < nv_pad * nv_pad; ++i) h[i] = 0.0f;
    for (int i = 0; i < nv; ++i)
      for (int j = 0; j < nv; ++j) {
        float v = m[i * nv + j];
        for (int r = 0; r < n; ++r) {
          const float dc = state[(size_t)w * njmax + r] == quad ? D[(size_t)w * njmax + r] : 0.0f;
          const float *Jr = J + ((size_t)w * njmax + r) * nv;
          v = fmaf(Jr[i] * dc, Jr[j], v);
        }
        h[i * nv_pad + j] = v;
      }
  }
  return 0;
}

/* ---- Muscle path geometry and activation <-> torque contractions ---------------------
 * Scalar restatement, one operation per statement in the order the formulas are written in
 * the reference; built with -ffp-contract=off so nothing is fused.  expf/cosf come from
 * libm, so the force magnitudes agree with a GPU evaluation only to a few ulp. */
typedef struct {
  float x, y, z;
} v3;
static v3 v_ld(const float *p) { v3 r = {p[0], p[1], p[2]}; return r; }
static v3 v_sub(v3 a, v3 b) { v3 r = {a.x - b.x, a.y - b.y, a.z - b.z}; return r; }
static v3 v_add(v3 a, v3 b) { v3 r = {a.x + b.x, a.y + b.y, a.z + b.z}; return r; }
static v3 v_scale(float s, v3 a) { v3 r = {s * a.x, s * a.y, s * a.z}; return r; }
static float v_dot(v3 a, v3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
static v3 v_cross(v3 a, v3 b) {
  v3 r = {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
  return r;
}
static float v_len(v3 a) { return sqrtf(v_dot(a, a)); }

/* segment_generalized_force_contribution_wp
 * (src/instantmimic/muscle/muscle_qfrc_projector.py:280-304). */
static float seg_contribution(v3 lin, v3 ang, v3 p0, v3 p1, v3 c0, v3 c1, float a, float b,
                              float force) {
  v3 seg = v_sub(p1, p0);
  float len = v_len(seg);
  if (len < 1.0e-8f) return 0.0f;
  v3 dir = {seg.x / len, seg.y / len, seg.z / len};
  v3 f = v_scale(force, dir);
  v3 st = v_add(lin, v_cross(ang, v_sub(p0, c0)));
  v3 en = v_add(lin, v_cross(ang, v_sub(p1, c1)));
  return v_dot(v_sub(v_scale(a, st), v_scale(b, en)), f);
}

/* _transform_waypoints_from_torch_kernel (src/instantmimic/muscle/muscle_dynamics_kernels.py:
 * 73-86), normalize_quat_wp (muscle_qfrc_projector.py:91-100) and mujoco_warp's
 * math.rot_vec_quat (third party, absent from the tree; published form
 * 2 (u.v) u + (s^2 - u.u) v + 2 s (u x v) for q = (s, u)). */
int orc_muscle_waypoints(int nworld, int nbody, int nwp, const float *xpos, const float *xquat,
                         const int *wp_body, const float *wp_local, float *out) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w)
    for (int i = 0; i < nwp; ++i) {
      const int b = wp_body[i];
      const float *q = xquat + ((size_t)w * nbody + b) * 4;
      float inv = 1.0f / sqrtf(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3] + 1.0e-8f);
      float s = q[0] * inv;
      v3 u = {q[1] * inv, q[2] * inv, q[3] * inv};
      v3 v = v_ld(wp_local + 3 * i);
      v3 r = v_add(v_scale(2.0f, v_scale(v_dot(u, v), u)), v_scale(s * s - v_dot(u, u), v));
      r = v_add(r, v_scale(2.0f * s, v_cross(u, v)));
      v3 p = v_add(v_ld(xpos + ((size_t)w * nbody + b) * 3), r);
      float *o = out + ((size_t)w * nwp + i) * 3;
      o[0] = p.x;
      o[1] = p.y;
      o[2] = p.z;
    }
  return 0;
}

/* muscle_qfrc_projector.py:103-145 */
static float active_fl(float l, const float *m) {
  if (m[0] < 0.5f) return expf(-((l - 1.0f) * (l - 1.0f)) / m[1]);
  float lmin = m[1], lmax = m[2];
  if (l < lmin || l > lmax) return 0.0f;
  float lo = 0.5f * (lmin + 1.0f), hi = 0.5f * (1.0f + lmax), x;
  if (l <= lo) {
    x = (l - lmin) / fmaxf(lo - lmin, 1.0e-8f);
    return 0.5f * x * x;
  }
  if (l <= 1.0f) {
    x = (1.0f - l) / fmaxf(1.0f - lo, 1.0e-8f);
    return 1.0f - 0.5f * x * x;
  }
  if (l <= hi) {
    x = (l - 1.0f) / fmaxf(hi - 1.0f, 1.0e-8f);
    return 1.0f - 0.5f * x * x;
  }
  x = (lmax - l) / fmaxf(lmax - hi, 1.0e-8f);
  return 0.5f * x * x;
}
/* muscle_qfrc_projector.py:148-187 */
static float passive_fl(float l, const float *m) {
  if (m[0] < 0.5f) {
    if (l < 1.0f) return 0.0f;
    float x = m[1] * (l - 1.0f) / m[2];
    x = fminf(fmaxf(x, -80.0f), 80.0f);
    return (expf(x) - 1.0f) / (expf(m[1]) - 1.0f);
  }
  float lmax = m[1], fpmax = m[2];
  if (l <= 1.0f) return 0.0f;
  float mid = 0.5f * (1.0f + lmax), width = fmaxf(mid - 1.0f, 1.0e-8f);
  if (l <= mid) {
    float st = (l - 1.0f) / width;
    return 0.5f * fpmax * st * st;
  }
  return fpmax * (0.5f + (l - mid) / width);
}

/* _compute_force_magnitudes_from_waypoints_kernel (muscle_dynamics_kernels.py:644-705);
 * model = force_scale, lnorm_min, lnorm_max, active[3], passive[3]. */
int orc_muscle_force_magnitudes(int nworld, int nwp, int nmuscle, const float *wp,
                                const int *seg_start, const int *seg_offsets,
                                const float *params, int ldpar, const float *rest,
                                const float *model, int include_passive, float *unit,
                                float *passive) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    const float *row = wp + (size_t)w * nwp * 3;
    for (int m = 0; m < nmuscle; ++m) {
      float len = 0.0f;
      for (int s = seg_offsets[m]; s < seg_offsets[m + 1]; ++s) {
        int i = seg_start[s];
        len = len + v_len(v_sub(v_ld(row + 3 * (i + 1)), v_ld(row + 3 * i)));
      }
      const float *p = params + (size_t)m * ldpar;
      float lm = len / fmaxf(rest[m], 1.0e-6f) - p[2];
      float ln = fminf(fmaxf(lm / fmaxf(p[1], 1.0e-6f), model[1]), model[2]);
      float c = cosf(p[3]);
      unit[(size_t)w * nmuscle + m] = p[0] * active_fl(ln, model + 3) * c * model[0];
      if (passive)
        passive[(size_t)w * nmuscle + m] =
            include_passive ? p[0] * passive_fl(ln, model + 6) * c * model[0] : 0.0f;
    }
  }
  return 0;
}

/* eval_muscle_force_velocity_state_kernel (src/instantmimic/muscle/muscle_qfrc_projector.py:
 * 2816-2884) with muscle_force_velocity_curve_wp (:2505-2524) and
 * muscle_force_velocity_response_wp (:2528-2570); model as in orc_muscle_force_magnitudes,
 * fv = vmax, fvmax, clamp_activation, include_active; out = five (nworld, nmuscle) arrays one
 * after the other: length, effective activation, velocity, multiplier, slope. */
int orc_muscle_force_velocity_state(int nworld, int nwp, int nmuscle, int nentry, int nvfull,
                                    const float *wp, const int *wp_start, const float *params,
                                    int ldpar, const float *rest, const float *length_scale,
                                    const float *act, const float *qvel, const float *moment,
                                    const int *dof_offsets, const int *dof_torque, int root,
                                    const float *model, const float *fv, float *out) {
  const size_t plane = (size_t)nworld * nmuscle;
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    const float *row = wp + (size_t)w * nwp * 3;
    for (int m = 0; m < nmuscle; ++m) {
      float len = 0.0f;
      for (int i = wp_start[m]; i < wp_start[m + 1] - 1; ++i)
        len = len + v_len(v_sub(v_ld(row + 3 * (i + 1)), v_ld(row + 3 * i)));
      float vel = 0.0f;
      for (int e = dof_offsets[m]; e < dof_offsets[m + 1]; ++e)
        vel = fmaf(-moment[(size_t)w * nentry + e], qvel[(size_t)w * nvfull + dof_torque[e] + root], vel);
      const float *p = params + (size_t)m * ldpar;
      const float vscale = fmaxf(length_scale[m] * fv[0], 1.0e-6f);
      const float v = vel / vscale, fvmax = fv[1], y = fvmax - 1.0f;
      float mult, slope;
      if (v <= -1.0f) { mult = 0.0f; slope = 0.0f; }
      else if (v <= 0.0f) { const float sh = v + 1.0f; mult = sh * sh; slope = 2.0f * sh; }
      else if (v <= y) { const float rem = y - v; mult = fvmax - rem * rem / y; slope = 2.0f * rem / y; }
      else { mult = fvmax; slope = 0.0f; }
      float a = act[(size_t)w * nmuscle + m];
      if (fv[2] != 0.0f) a = fminf(fmaxf(a, 0.0f), 1.0f);
      const float lm = len / fmaxf(rest[m], 1.0e-6f) - p[2];
      const float ln = fminf(fmaxf(lm / fmaxf(p[1], 1.0e-6f), model[1]), model[2]);
      const float unit = p[0] * active_fl(ln, model + 3) * cosf(p[3]) * model[0];
      const size_t o = (size_t)w * nmuscle + m;
      out[o] = len;
      out[plane + o] = a * mult;
      out[2 * plane + o] = vel;
      out[3 * plane + o] = mult;
      out[4 * plane + o] = fv[3] * a * unit * slope / vscale;
    }
  }
  return 0;
}

/* rows of an entry list: offsets[nrow + 1], segment, other, start/end coefficient */
#define ORC_GEO(w)                                                                        \
  const float *wpw = wp + (size_t)(w) * nwp * 3, *comw = com + (size_t)(w) * nbody * 3, \
              *cdw = cdof + (size_t)(w) * nv * 6
#define ORC_TERM(segi, lin, ang, a, b, f)                                                  \
  seg_contribution(lin, ang, v_ld(wpw + 3 * seg_p0[segi]), v_ld(wpw + 3 * seg_p1[segi]),  \
                   v_ld(comw + 3 * seg_b0[segi]), v_ld(comw + 3 * seg_b1[segi]), a, b, f)

/* _compute_muscle_dynamics_from_activation_sparse_kernel (muscle_dynamics_kernels.py:1707-1793) */
int orc_muscle_torque_forward(int nworld, int nwp, int nbody, int nv, int nmuscle, int ntorque,
                              const float *wp, const float *com, const float *cdof,
                              const int *seg_p0, const int *seg_p1, const int *seg_b0,
                              const int *seg_b1, const int *offsets, const int *e_seg,
                              const int *e_muscle, const float *e_a, const float *e_b,
                              const float *unit, const float *passive, const float *act, int root,
                              float *out) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    ORC_GEO(w);
    for (int j = 0; j < ntorque; ++j) {
      v3 ang = v_ld(cdw + 6 * (j + root)), lin = v_ld(cdw + 6 * (j + root) + 3);
      float total = 0.0f;
      for (int e = offsets[j]; e < offsets[j + 1]; ++e) {
        int m = e_muscle[e];
        float f = unit[(size_t)w * nmuscle + m] * act[(size_t)w * nmuscle + m];
        if (passive) f = f + passive[(size_t)w * nmuscle + m];
        if (f == 0.0f) continue;
        total = total + ORC_TERM(e_seg[e], lin, ang, e_a[e], e_b[e], f);
      }
      out[(size_t)w * ntorque + j] = total;
    }
  }
  return 0;
}

/* _compute_muscle_dynamics_activation_grad_sparse_kernel (muscle_dynamics_kernels.py:1796-1859) */
int orc_muscle_activation_grad(int nworld, int nwp, int nbody, int nv, int nmuscle, int ntorque,
                               const float *wp, const float *com, const float *cdof,
                               const int *seg_p0, const int *seg_p1, const int *seg_b0,
                               const int *seg_b1, const int *offsets, const int *e_seg,
                               const int *e_torque, const float *e_a, const float *e_b,
                               const float *unit, const float *gout, int root, float *gact) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    ORC_GEO(w);
    for (int m = 0; m < nmuscle; ++m) {
      float f = unit[(size_t)w * nmuscle + m], grad = 0.0f;
      if (f != 0.0f)
        for (int e = offsets[m]; e < offsets[m + 1]; ++e) {
          int j = e_torque[e];
          v3 ang = v_ld(cdw + 6 * (j + root)), lin = v_ld(cdw + 6 * (j + root) + 3);
          grad = grad + gout[(size_t)w * ntorque + j] * ORC_TERM(e_seg[e], lin, ang, e_a[e], e_b[e], f);
        }
      gact[(size_t)w * nmuscle + m] = grad;
    }
  }
  return 0;
}

/* eval_muscle_sparse_moment_kernel (muscle_qfrc_projector.py:2617-2662) */
int orc_muscle_sparse_moment(int nworld, int nwp, int nbody, int nv, int nentry, const float *wp,
                             const float *com, const float *cdof, const int *seg_p0,
                             const int *seg_p1, const int *seg_b0, const int *seg_b1,
                             const int *entry_torque, const int *offsets, const int *e_seg,
                             const float *e_a, const float *e_b, int root, float *moment) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    ORC_GEO(w);
    for (int e = 0; e < nentry; ++e) {
      int j = entry_torque[e] + root;
      v3 ang = v_ld(cdw + 6 * j), lin = v_ld(cdw + 6 * j + 3);
      float total = 0.0f;
      for (int k = offsets[e]; k < offsets[e + 1]; ++k)
        total = total + ORC_TERM(e_seg[k], lin, ang, e_a[k], e_b[k], 1.0f);
      moment[(size_t)w * nentry + e] = total;
    }
  }
  return 0;
}

/* _compute_muscle_dynamics_sparse_bounds_kernel (muscle_dynamics_kernels.py:1453-1528) */
int orc_muscle_torque_bounds(int nworld, int nwp, int nbody, int nv, int nmuscle, int ntorque,
                             const float *wp, const float *com, const float *cdof,
                             const int *seg_p0, const int *seg_p1, const int *seg_b0,
                             const int *seg_b1, const int *offsets, const int *e_seg,
                             const int *e_muscle, const float *e_a, const float *e_b,
                             const float *unit, int root, float *lower, float *upper) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    ORC_GEO(w);
    for (int j = 0; j < ntorque; ++j) {
      v3 ang = v_ld(cdw + 6 * (j + root)), lin = v_ld(cdw + 6 * (j + root) + 3);
      int current = -1;
      float total = 0.0f, lo = 0.0f, hi = 0.0f;
      for (int e = offsets[j]; e < offsets[j + 1]; ++e) {
        int m = e_muscle[e];
        if (current >= 0 && m != current) {
          if (total < 0.0f) lo = lo + total;
          else hi = hi + total;
          total = 0.0f;
        }
        current = m;
        total = total + ORC_TERM(e_seg[e], lin, ang, e_a[e], e_b[e], unit[(size_t)w * nmuscle + m]);
      }
      if (current >= 0) {
        if (total < 0.0f) lo = lo + total;
        else hi = hi + total;
      }
      lower[(size_t)w * ntorque + j] = lo;
      upper[(size_t)w * ntorque + j] = hi;
    }
  }
  return 0;
}

/* ---- steps either side of the solve that walk a world's small trees ---------------------- */

/* The product M v of the fused Newton kernel
 * (src/instantmimic/utils/mjw_kernels/newton_fusion.py:171-176):
 *     value = 0;  for k in row: value += M[adr[k]] * v[col[k]]
 * with the multiply contracted into the add (one fmaf per term, as NVRTC compiles the
 * statement).  The row tables are the upstream model's M_mulm_* arrays (mujoco_warp, absent
 * from the tree): the order of a row's terms is theirs and is a parameter here.  Pinned by
 * the dense fp64 product; bit-level agreement with the reference build is unpinned. */
int orc_mul_m_sparse(int nworld, int nv, int nM, const int *rowadr, const int *col,
                     const int *madr, const float *M, const float *vec,
                     const unsigned char *skip, float *out) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    if (skip && skip[w]) continue;
    const float *m = M + (size_t)w * nM, *v = vec + (size_t)w * nv;
    for (int dof = 0; dof < nv; ++dof) {
      float value = 0.0f;
      for (int k = rowadr[dof]; k < rowadr[dof + 1]; ++k) value = fmaf(m[madr[k]], v[col[k]], value);
      out[(size_t)w * nv + dof] = value;
    }
  }
  return 0;
}

/* accumulate_body_tree_deterministic_kernel
 * (src/instantmimic/utils/mjw_kernels/tree_fusion.py:82-113), in place on
 * values (nworld, nbody, components). */
static void orc_fold_levels(float *values, int components, const int *parent, const int *bodies,
                            const int *offsets, int levels, int skip_root_parent) {
  for (int level = levels - 1; level > 0; --level)
    for (int p = offsets[level - 1]; p < offsets[level]; ++p) {
      const int parent_id = bodies[p];
      if (skip_root_parent && parent_id == 0) continue;
      for (int c = 0; c < components; ++c) {
        float value = values[parent_id * components + c];
        for (int e = offsets[level]; e < offsets[level + 1]; ++e) {
          const int body = bodies[e];
          if (body != 0 && parent[body] == parent_id) value = value + values[body * components + c];
        }
        values[parent_id * components + c] = value;
      }
    }
}

int orc_tree_accumulate(int nworld, int nbody, int components, const int *parent,
                        const int *bodies, const int *offsets, int levels,
                        int skip_root_parent, float *values) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w)
    orc_fold_levels(values + (size_t)w * nbody * components, components, parent, bodies, offsets,
                    levels, skip_root_parent);
  return 0;
}

/* project_body_wrenches_to_dofs_kernel (src/instantmimic/muscle/wrench_projection.py:59-136)
 * with the siblings of a parent added in the order of level_bodies (the reference adds them
 * with atomics, in no fixed order: its result is this one up to that order).  Pinned by the
 * masked sum of the legacy kernel (muscle_dynamics_kernels.py:2906-2955) in fp64. */
int orc_project_body_wrenches(int nworld, int nbody, int nvfull, const float *body_force,
                              const float *body_torque, const float *xipos,
                              const float *subtree_com, const float *cdof, const int *rootid,
                              const int *dof_body, const int *parent, const int *bodies,
                              const int *offsets, int levels, int root, int ntorque,
                              int out_offset, int ld_mean, float *mean) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    float *values = (float *)malloc(sizeof(float) * 6 * (size_t)nbody);
    for (int b = 0; b < nbody; ++b) {
      const float *f = body_force + ((size_t)w * nbody + b) * 3;
      const float *t = body_torque + ((size_t)w * nbody + b) * 3;
      const float *x = xipos + ((size_t)w * nbody + b) * 3;
      const float *c = subtree_com + ((size_t)w * nbody + rootid[b]) * 3;
      const float rx = x[0] - c[0], ry = x[1] - c[1], rz = x[2] - c[2];
      float *o = values + 6 * b;
      o[0] = f[0];
      o[1] = f[1];
      o[2] = f[2];
      o[3] = t[0] + (ry * f[2] - rz * f[1]);
      o[4] = t[1] + (rz * f[0] - rx * f[2]);
      o[5] = t[2] + (rx * f[1] - ry * f[0]);
    }
    orc_fold_levels(values, 6, parent, bodies, offsets, levels, 0);
    for (int j = 0; j < ntorque; ++j) {
      const int dof = j + root;
      const float *v = values + 6 * dof_body[dof];
      const float *cd = cdof + ((size_t)w * nvfull + dof) * 6;
      const float lin = cd[3] * v[0] + cd[4] * v[1] + cd[5] * v[2];
      const float ang = cd[0] * v[3] + cd[1] * v[4] + cd[2] * v[5];
      mean[(size_t)w * ld_mean + j + out_offset] = lin + ang;
    }
    free(values);
  }
  return 0;
}

/* gradient_function of the fused Newton kernel
 * (src/instantmimic/utils/mjw_kernels/newton_stages.py:745-798).  The sums over rows and the
 * squares contract into fused multiply-adds; grad . grad is summed as a block of `block` lanes
 * with a 32-lane shuffle-down tree, the convention of sp_backward_sums above (the reference
 * leaves the order to Warp's tile_sum: bit-level agreement with it is unpinned). */
int orc_newton_gradient(int nworld, int nv, int njmax, int block, const int *nefc, const float *J,
                        const float *force, const float *smooth, const float *Ma,
                        const int *changed, const float *alpha, const unsigned char *done,
                        float *qc, float *grad, float *grad_dot, float *decrement, float *scale,
                        unsigned char *unchanged) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    const int dn = done && done[w], ch = changed[w] != 0;
    unchanged[w] = (dn || !ch) ? 1 : 0;
    if (dn) continue;
    if (!ch) {
      const float sigma = scale[w], new_sigma = sigma - alpha[w];
      float ratio = 0.0f;
      if (sigma != 0.0f) ratio = new_sigma / sigma;
      const float ratio_sq = ratio * ratio;
      grad_dot[w] = grad_dot[w] * ratio_sq;
      decrement[w] = decrement[w] * ratio_sq;
      scale[w] = new_sigma;
      continue;
    }
    int ne = nefc ? nefc[w] : njmax;
    if (ne > njmax) ne = njmax;
    const float *Jw = J + (size_t)w * njmax * nv, *f = force + (size_t)w * njmax;
    for (int dof = 0; dof < nv; ++dof) {
      float sum = 0.0f;
      for (int r = 0; r < ne; ++r) sum = fmaf(Jw[(size_t)r * nv + dof], f[r], sum);
      qc[(size_t)w * nv + dof] = sum;
      grad[(size_t)w * nv + dof] = Ma[(size_t)w * nv + dof] - smooth[(size_t)w * nv + dof] - sum;
    }
    float part[64] = {0};
    for (int lane = 0; lane < block; ++lane)
      for (int dof = lane; dof < nv; dof += block) {
        const float g = grad[(size_t)w * nv + dof];
        part[lane] = fmaf(g, g, part[lane]);
      }
    float total = 0.0f;
    for (int wv = 0; wv < block / 32; ++wv) {
      float *a = part + 32 * wv;
      for (int off = 16; off > 0; off >>= 1)
        for (int i = 0; i < off; ++i) a[i] = a[i] + a[i + off];
      total = total + a[0];
    }
    grad_dot[w] = total;
    decrement[w] = 0.0f;
    scale[w] = 1.0f;
  }
  return 0;
}

/* The J v step of the line search (src/instantmimic/utils/mjw_kernels/newton_stages.py:157-178):
 * one chain of fused multiply-adds up to 50 dofs; beyond, 20-dof partial sums added with their
 * own rounding (rounded_step(jv, 1.0, partial) = jv + 1.0 * partial without contraction). */
int orc_newton_jv(int nworld, int nv, int njmax, const int *nefc, const float *J,
                  const float *search, const unsigned char *skip, float *jv) {
#pragma omp parallel for schedule(static)
  for (int w = 0; w < nworld; ++w) {
    if (skip && skip[w]) continue;
    int ne = nefc ? nefc[w] : njmax;
    if (ne > njmax) ne = njmax;
    const float *s = search + (size_t)w * nv;
    for (int r = 0; r < ne; ++r) {
      const float *row = J + ((size_t)w * njmax + r) * nv;
      float acc = 0.0f;
      if (nv > 50) {
        for (int start = 0; start < nv; start += 20) {
          const int end = start + 20 < nv ? start + 20 : nv;
          float partial = 0.0f;
          for (int i = start; i < end; ++i) partial = fmaf(row[i], s[i], partial);
          acc = acc + partial;
        }
      } else {
        for (int i = 0; i < nv; ++i) acc = fmaf(row[i], s[i], acc);
      }
      jv[(size_t)w * njmax + r] = acc;
    }
  }
  return 0;
}

/* search . search and grad . x (x = -search) of the tree factor stage, summed as the reference's
 * stages sum their two dot products (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:462-479):
 * lane l of `block` lanes adds its dofs l, l + block, .. with fused multiply-adds, 32 lanes fold in
 * a shuffle-down tree, the folds are added in order from zero.  Dofs in dof order. */
int orc_newton_search_sums(int nworld, int nv, int block, const unsigned char *skip, const float *grad,
                           int ldg, const float *search, int lds, float *sdot, float *decr) {
  for (int w = 0; w < nworld; ++w) {
    if (skip && skip[w]) continue;
    float s0[64] = {0}, s1[64] = {0};
    for (int lane = 0; lane < block; ++lane)
      for (int d = lane; d < nv; d += block) {
        const float v = -search[(size_t)w * lds + d];
        s0[lane] = fmaf(v, v, s0[lane]);
        s1[lane] = fmaf(grad[(size_t)w * ldg + d], v, s1[lane]);
      }
    float ra = 0.0f, rb = 0.0f;
    for (int wv = 0; wv < block / 32; ++wv) {
      float *a = s0 + 32 * wv, *b = s1 + 32 * wv;
      for (int off = 16; off > 0; off >>= 1)
        for (int i = 0; i < off; ++i) {  /* lane i takes lane i + off; lanes past the fold are not read again */
          a[i] = a[i] + a[i + off];
          b[i] = b[i] + b[i + off];
        }
      ra = ra + a[0];
      rb = rb + b[0];
    }
    sdot[w] = ra;
    decr[w] = rb;
  }
  return 0;
}
