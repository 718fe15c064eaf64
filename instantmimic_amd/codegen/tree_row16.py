"""Generator of plan-specialised gfx950 kernels for the fused Hessian assembly +
tree L'DL + solve.

Fused kernel: one workgroup of four wavefronts per four worlds.

* Assembly.  Wavefront v assembles world v on the matrix cores: H is cut into 16 x 16
  tiles of its lower triangle and every step of four constraint rows is three (or more)
  ``v_mfma_f32_16x16x4_f32`` with A = J and B = J * D.  The instruction accumulates its
  four products one after the other with fused multiply-adds, which is the order and
  rounding of ``v = fmaf(J[r][a] * D[r], J[r][b], v)`` over the rows r
  (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:622-629); the accumulators start
  from M.  J goes from HBM straight into the operand registers (lane = (row of the step,
  column)), never through LDS.  With at most 64 constraint rows the first 16 rows are
  requested at once and of the others only those with ``state == quad`` below ``nefc``
  (their ids packed in row order by a ballot and a prefix count): a row left out would
  have added ``(J * 0) * J`` to every entry.  All loads are unconditional and counted, so
  each step waits for exactly its own operands.
* Hand-over.  The tiles go to a copy of H's lower triangle in LDS (a row as long as its
  tile row reaches); from there each wavefront reads
  the rows it factors in the "row16" layout: a world owns one 16-lane DPP row, row b of H
  (the CSR row of dof b: its ancestors root-first, then b) lives in one VGPR per 16
  positions, lane p of register ``h{b}_{s}`` holds H[b][anc_{16 s + p}(b)].  All dofs on one
  root-to-leaf chain agree on what sits at position p.
* Factor and solve (src/instantmimic/utils/mjw_kernels/tree_ldl.py:215-305).  Wavefront j
  eliminates group j of the plan into zero-initialised trunk accumulators and publishes
  them through LDS; wavefront 0 adds them to the trunk rows in group order, eliminates and
  solves the trunk and publishes its solution; the groups then back-substitute.
  Eliminating dof k updates ancestor row anc_p with
  ``h[anc_p] = fma(bcast(h[k], p) * h[k], -1/h[k][k], h[anc_p])`` (``v_mul_f32_dpp`` then a
  plain fma); right-hand side, inverse pivots and solution are uniform per world and their
  updates are single ``v_fmac_f32_dpp`` with the scaled pivot row
  ``T[k] = h[k] * -1/h[k][k]`` as the broadcast operand.

The solve-only kernel has the same four wavefronts per four worlds and the same roles; it
reads H in the row16 layout from memory (a role fetches the rows it works on) and hands the
groups' sums to the trunk through LDS as the fused kernel does.

DPP reads of a register written by one of the two preceding VALU instructions are a
hardware hazard that the compiler does not see inside inline assembly: every block that
reads registers produced outside it starts with ``s_nop 1``.  Lanes past a row's length
hold unused values that no valid lane ever reads.
"""

from __future__ import annotations

import os

# development aid: IMHIP_EXP=timing makes the fused kernel write clock64() stamps of its phases
# over the H output buffer instead of H
EXP = os.environ.get("IMHIP_EXP", "")
# every environment variable that changes the generated source (the run-time cache keys on them)
SOURCE_KNOBS = ("IMHIP_EXP", "IMHIP_SP", "IMHIP_OCC")


class Declined(ValueError):
    """The generator does not take this (structure, plan): the caller keeps the table-driven kernel."""


def _require(ok, why: str) -> None:
    if not ok:
        raise Declined(why)


def structure_key(rowadr, rownnz, colind, groups, trunk) -> int:
    """64-bit key of a (structure, plan) pair; must match tree_key() in tree_kernels.hip."""
    h = 0xCBF29CE484222325
    def mix(v):
        nonlocal h
        h ^= (v & 0xFFFFFFFF)
        h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    mix(len(rowadr))
    for v in rowadr: mix(v)
    for v in rownnz: mix(v)
    nM = max(a + n for a, n in zip(rowadr, rownnz))
    mix(nM)
    for v in list(colind)[:nM]: mix(v)
    mix(len(groups))
    for g in groups:
        mix(len(g))
        for v in g: mix(v)
    mix(len(trunk))
    for v in trunk: mix(v)
    return h


class _Tree:
    def __init__(self, rowadr, rownnz, colind):
        self.nv = len(rowadr)
        self.rowadr, self.rownnz, self.colind = list(rowadr), list(rownnz), list(colind)
        self.nM = max(a + n for a, n in zip(rowadr, rownnz))
        self.depth = [n - 1 for n in rownnz]
        self.anc = [list(colind[rowadr[k] : rowadr[k] + rownnz[k] - 1]) for k in range(self.nv)]
        self.chain = [self.anc[k] + [k] for k in range(self.nv)]
        children = [[] for _ in range(self.nv)]
        for k in range(self.nv):
            if self.anc[k]:
                children[self.anc[k][-1]].append(k)
        self.children = children
        self.leaves = [k for k in range(self.nv) if not children[k]]
        # every dof reads J through the chain of the first leaf below it
        self.leaf_of = [None] * self.nv
        for li, leaf in enumerate(self.leaves):
            for k in self.chain[leaf]:
                if self.leaf_of[k] is None:
                    self.leaf_of[k] = li

    def sets(self, k):
        return self.depth[k] // 16 + 1


def generate(name, rowadr, rownnz, colind, groups, trunk, *, module: bool = False) -> str:
    """HIP source of the kernels for one (structure, plan).  ``module``: a stand-alone code object
    (kernels ``im_row16_fused``, ``im_row16_fused_long``, ``im_row16_solve`` with C names and the
    constants ``im_row16_key`` / ``im_row16_info`` that describe them) for loading at run time;
    otherwise a source file of the library that registers its kernels when the library loads."""
    t = _Tree(rowadr, rownnz, colind)
    nv, nM = t.nv, t.nM
    trunk_set = set(trunk)
    ngroups = len(groups)
    key = structure_key(rowadr, rownnz, colind, groups, trunk)
    out = []
    emit = out.append
    DPP = "row_mask:0xf bank_mask:0xf bound_ctrl:1"

    leaf_sets = [(li, s) for li, leaf in enumerate(t.leaves) for s in range(t.sets(leaf))]
    # chain column table: CH[li][s][p] = dof at position 16 s + p of leaf li's chain (0 past the end)
    tab = []
    for li, s in leaf_sets:
        ch = t.chain[t.leaves[li]]
        tab.append([ch[16 * s + p] if 16 * s + p < len(ch) else 0 for p in range(16)])

    emit(f"// generated by instantmimic_amd/codegen/tree_row16.py for '{name}' -- do not edit")
    emit(f"// nv={nv} nM={nM} groups={groups} trunk={list(trunk)}")
    emit('#include "../tree_row16.h"')
    emit("namespace im { namespace gen {")
    emit(f"static __device__ const unsigned char CH_{name}[{len(leaf_sets)}][16] = {{")
    for row in tab:
        emit("  {" + ",".join(str(v) for v in row) + "},")
    emit("};")
    # CSR index of every accumulator element of the lower-triangle 16 x 16 tiles, -1 off the pattern
    NT_ = -(-nv // 16)
    pos_of = {}
    for b in range(nv):
        for d_, a_ in enumerate(t.chain[b]):
            pos_of[b, a_] = t.rowadr[b] + d_
    idx_rows = []
    for ti in range(NT_):
        for tj in range(ti + 1):
            for v in range(4):
                idx_rows.append([4 * pos_of.get((16 * ti + 4 * (l // 16) + v, 16 * tj + l % 16), nM) for l in range(64)])
    emit(f"static __device__ const short IDX_{name}[{len(idx_rows)}][64] = {{")
    for row in idx_rows:
        emit("  {" + ",".join(str(v) for v in row) + "},")
    emit("};")
    # Right-hand side as lane vectors: lane p of register set s holds the entry of the dof at
    # position 16 s + p of the chain being eliminated, so that one fused multiply-add per set
    # applies a step's update to every ancestor (same operation per entry as one per ancestor).
    # A group's lanes at trunk positions are its zero-initialised accumulators.  A group with
    # several branches reuses the lanes past the fork: `segs[j]` lists, per run of dofs on one
    # chain, the lanes that take new dofs (a copy of the vector keeps the finished branch).
    tpos = {a: t.depth[a] for a in trunk}
    # the trunk's right-hand side is one lane vector with the dof of depth p in lane p: a forest's
    # trunk (several roots) or a trunk that forks has two dofs for one lane
    _require(sorted(tpos.values()) == list(range(len(trunk))), "the plan's trunk is not a single chain from one root")
    _require(all(len(g) > 0 for g in groups), "a plan with an empty group")
    _require(nv <= 96, "more than 96 dofs")
    # Per group: which owner (trunk accumulator ('t', a) or group dof ('g', b)) sits in which lane
    # while each dof is eliminated.  A new segment starts when the chain of the next dof needs a
    # lane for another owner: the lane then takes a fresh value (the dof's right-hand side, or
    # zero for an accumulator) or the owner's value from the segment it was last resident in.
    segs = []      # per group: list of dict(fresh={pos: dof or -1}, restore={pos: segment})
    seg_of = {}    # group dof -> (group, segment it is eliminated in)
    home = []      # per group: owner -> segment whose vector holds its final value
    for j, g in enumerate(groups):
        lane_owner, hm_, lst = {}, {}, []
        for k in g:
            want = {t.depth[a]: (("t", a) if a in trunk_set else ("g", a)) for a in t.chain[k]}
            if any(lane_owner.get(pos) != own for pos, own in want.items()):
                seg = {"fresh": {}, "restore": {}}
                for pos, own in want.items():
                    if lane_owner.get(pos) == own:
                        continue
                    if own in hm_:
                        seg["restore"][pos] = hm_[own]
                    else:
                        seg["fresh"][pos] = own[1] if own[0] == "g" else -1
                    lane_owner[pos] = own
                lst.append(seg)
            for own in lane_owner.values():
                hm_[own] = len(lst) - 1
            seg_of[k] = (j, len(lst) - 1)
        segs.append(lst)
        home.append(hm_)
    vsets = [max(t.sets(k) for k in g) for g in groups]
    tsets = max(t.sets(k) for k in trunk) if len(trunk) else 1
    svi_rows, svi_of = [], {}
    for j in range(ngroups):
        for i, take in enumerate(segs[j]):
            for s_ in range(vsets[j]):
                svi_of[j, i, s_] = len(svi_rows)
                svi_rows.append([take["fresh"].get(16 * s_ + p, -1) for p in range(16)])
    for s_ in range(tsets):
        svi_of["T", 0, s_] = len(svi_rows)
        svi_rows.append([trunk[16 * s_ + p] if 16 * s_ + p < len(trunk) else -1 for p in range(16)])
    emit(f"static __device__ const signed char SVI_{name}[{len(svi_rows)}][16] = {{")
    for row in svi_rows:
        emit("  {" + ",".join(str(v) for v in row) + "},")
    emit("};")
    # LONG: more constraint rows than the straight-line assembly keeps in flight (a loop instead)
    # the body as a function: the kernels at the end of the file call it, the resident Newton
    # kernel once per iteration
    # SPLIT: the workgroup's four wavefronts share the work on its four worlds by role (group j
    # on wavefront j, the trunk on wavefront 0) and hand their results on through LDS; without it
    # one wavefront takes every role in turn.  The fused kernels always split; the solve-only
    # kernel does too (taking every role, a wavefront would have to hold every row of H at once).
    emit("template <bool ASM, bool LONG, bool SPLIT = ASM>")
    # world_of: null, or four world numbers in LDS, one per wavefront / 16-lane row, in place of the
    # workgroup's own four (the resident Newton loop hands finished wavefronts new worlds; a number
    # at or past nworld stands for no world)
    emit(f"__device__ __forceinline__ void tree_row16_body_{name}(IM_ROW16_PARAMS, const int *world_of) {{")
    # the lane number as a value the compiler cannot see through: called from a loop (the resident
    # Newton kernel), nothing derived from it counts as loop-invariant, so no table entry or address
    # of this body is kept in a register from one call to the next
    emit("  int lane_ = threadIdx.x & 63;")
    emit('  asm volatile("" : "+v"(lane_));')
    emit("  const int lane = lane_, p = lane & 15, wv = threadIdx.x >> 6;")
    # Several iterations in one launch (fused kernels only): the grid covers (four worlds, iteration)
    # pairs.  Workgroups go to the chip's eight XCDs in turn, each with an L2 of its own, so the
    # iterations of one group of worlds take consecutive workgroups of one XCD: they run at about
    # the same time next to the same L2 and M and J come from memory once.
    emit("  int bid = blockIdx.x;")
    emit("  if (ASM && niter > 1) {")
    emit("    const int slot = bid >> 3, it = slot % niter;")
    emit("    bid = (slot / niter) * 8 + (bid & 7);")
    emit("    if (bid * 4 >= nworld) return;  // the grid is rounded up to whole rounds of the XCDs")
    emit("    state += it * state_it; y += it * y_it; x += it * x_it;")
    emit("  }")
    emit("  const int w = world_of ? world_of[lane >> 4] : bid * 4 + (lane >> 4);")
    emit("  const int64_t ws = w < nworld ? w : nworld - 1;")
    # a world whose `skip` byte is set is read and worked on like its neighbours (a wavefront's
    # four worlds share every instruction) and nothing of it is stored
    emit("  const bool live = w < nworld && !(skip && skip[ws]);")
    # ---- right-hand side, uniform per world (wavefront 0 factors and solves)
    emit("  const float *yw = y + ws * ldy;")
    # wavefront j factors group j of the plan, wavefront 0 also the trunk
    emit("  float " + ", ".join(f"S{b} = 0.0f" for b in range(nv)) + ";")

    def sv(j, i, s_):
        return f"SVT_{s_}" if j == "T" else f"SV{j}_{i}_{s_}"

    def load_sv(j, i, s_, var):
        emit(f"    {{ const int ix = SVI_{name}[{svi_of[j, i, s_]}][p]; const float yv = yw[ix < 0 ? 0 : ix];"
             f" {var} = ix >= 0 ? yv : 0.0f; }}")

    # The fused kernels read the right-hand side through the chain tables they hold anyway (lane p
    # of a chain's vector = the dof at position p), every wavefront all vectors, right behind
    # the requests for J and without a branch: a load under a role's branch is waited for inside
    # the branch, ahead of everything that follows.  rhs_src[j, i, s_] = (index of the chain
    # table row, lanes that take a right-hand side entry).
    rhs_src = {}
    for j, g in enumerate(groups):
        for i, take in enumerate(segs[j]):
            k_first = next(q for q in g if seg_of[q] == (j, i))
            for s_ in range(vsets[j]):
                mask = sum(1 << p for p in range(16) if take["fresh"].get(16 * s_ + p, -1) >= 0)
                ci = leaf_sets.index((t.leaf_of[k_first], s_)) if (t.leaf_of[k_first], s_) in leaf_sets else None
                if mask:
                    _require(ci is not None and all(tab[ci][p] == take["fresh"][16 * s_ + p] for p in range(16) if (mask >> p) & 1),
                             "a group's right-hand side does not lie on one chain table")
                rhs_src[j, i, s_] = (ci, mask)
    if len(trunk):
        below = next(li for li, leaf in enumerate(t.leaves) if trunk[-1] in t.chain[leaf])
        for s_ in range(tsets):
            mask = sum(1 << p for p in range(16) if 16 * s_ + p < len(trunk))
            ci = leaf_sets.index((below, s_))
            _require(all(tab[ci][p] == trunk[16 * s_ + p] for p in range(16) if (mask >> p) & 1), "the trunk does not lie on one chain table")
            rhs_src["T", 0, s_] = (ci, mask)
    else:
        for s_ in range(tsets):
            rhs_src["T", 0, s_] = (None, 0)
    rhs_tables = sorted({ci for ci, mask in rhs_src.values() if mask})
    emit("  float " + ", ".join(f"yv{ci} = 0.0f" for ci in rhs_tables) + ";")

    def take_rhs(j, i, s_, var):
        ci, mask = rhs_src[j, i, s_]
        emit(f"      {var} = " + (f"im_lane_select(yv{ci}, IM_ROW_MASK(0x{mask:x}));" if mask else "0.0f;"))

    for j in range(ngroups):
        names = [sv(j, i, s_) for i in range(len(segs[j])) for s_ in range(vsets[j])]
        names += [f"SY{j}_{i}_{s_}" for i in range(1, len(segs[j])) for s_ in range(vsets[j])]
        names += [f"SP{j}_{s_}" for s_ in range(vsets[j])]
        emit("  float " + ", ".join(f"{n_} = 0.0f" for n_ in names) + ";")
    emit("  float " + ", ".join(f"SVT_{s_} = 0.0f" for s_ in range(tsets)) + ";")
    emit("  float " + ", ".join(f"h{b}_{s}" for b in range(nv) for s in range(t.sets(b))) + ";")
    # ---- assembly on the matrix cores: wavefront v of the workgroup assembles world v of the four
    NT = -(-nv // 16)  # 16-wide blocks of dofs
    tiles = [(ti, tj) for ti in range(NT) for tj in range(ti + 1)]  # lower triangle
    # Staging copy of H's lower triangle in LDS, per world: the rows of tile row ti are 16 (ti + 1)
    # words long and follow one another, the last tile row stops at the last dof (rounded up to
    # the four rows a lane group stores), and worlds lie 16 words off a multiple of the banks so
    # that two worlds' lanes of one request fall on different banks.
    last_rows = 4 * -(-(nv - 16 * (NT - 1)) // 4)
    tile_rows = [16] * (NT - 1) + [last_rows]
    row_len = [16 * (ti + 1) for ti in range(NT)]
    band_off = [sum(tile_rows[i] * row_len[i] for i in range(ti)) for ti in range(NT + 1)]
    TW = band_off[NT] + 16  # words per world

    def h_off(b):
        return band_off[b // 16] + (b % 16) * row_len[b // 16]

    PD = max(2, min(16, 48 // NT))  # steps of 4 constraint rows in flight
    touched = [set() for _ in range(ngroups)]
    for j, g in enumerate(groups):
        for k in g:
            for a in t.anc[k]:
                if a in trunk_set:
                    touched[j].add(a)
    # exchange through LDS: every group's trunk accumulators (one 64-lane vector per register)
    # and the trunk's solution per world
    xslots = []
    xoff = 4 * TW
    for j in range(ngroups):
        sl = {}
        for a in sorted(touched[j]):
            for s_ in range(t.sets(a)):
                sl[a, s_] = xoff
                xoff += 64

        for s_ in range(vsets[j]):
            sl["S", s_] = xoff
            xoff += 64
        xslots.append(sl)
    xs_off = xoff
    lds_floats = xs_off + 4 * nv

    def xo(off):
        """LDS word of an exchange slot: behind the four staging copies in the fused kernels, from
        word 0 in the solve-only kernel (which has no staging copy)"""
        return f"(ASM ? {off} : {off - 4 * TW})"
    if EXP == "timing":
        emit("  unsigned long long *tdbg = (unsigned long long *)Hout + (size_t)bid * 16; int tn = 0;")
        emit("  #define STAMP() do { if (Hout && threadIdx.x == 0) tdbg[tn] = clock64(); ++tn; } while (0)")
        emit("  STAMP();")
    else:
        emit("  #define STAMP() do {} while (0)")
    emit("  extern __shared__ float xlds[];")
    emit("  const float " + ", ".join(f"*lh{i} = nullptr" for i in range(len(leaf_sets))) + ";")
    emit("  if (ASM) {")
    emit("    float *lds = xlds;")
    emit("    const int kq = lane >> 4;")
    emit("    const int njp = (njmax + 15) & ~15;")
    emit(f"    float *dcl = lds + {lds_floats} + wv * (LONG ? 2 * njp : 128);  // D per listed row, and the list of rows behind it")
    emit("    const int wq_ = world_of ? __builtin_amdgcn_readfirstlane(world_of[wv]) : bid * 4 + wv;")
    emit("    const int64_t wq = wq_ < nworld ? wq_ : nworld - 1;")
    emit("    int ne = nefc_p ? nefc_p[wq] : njmax; ne = ne < njmax ? ne : njmax;")
    emit("    ne = __builtin_amdgcn_readfirstlane(ne);")
    # every load below is unconditional (clamped address, value selected afterwards): a load
    # under a lane mask turns into a branch and a wait in the instruction stream
    # J through a buffer descriptor over the world's njmax x nv block: the address of a load is a
    # scalar base, one 32-bit lane offset and an immediate (no 64-bit arithmetic per load), and a
    # row at or past njmax reads as zero without a clamp
    emit("    const int wqs = __builtin_amdgcn_readfirstlane((int)wq);")
    emit(f"    const __amdgpu_buffer_rsrc_t jrs = __builtin_amdgcn_make_buffer_rsrc((void *)(J + (int64_t)wqs * njmax * {nv}), (short)0, njmax * {4 * nv}, 0x00020000);")
    for c in range(NT):
        col = f"p + {16 * c}" if 16 * c + 16 <= nv else f"min(p + {16 * c}, {nv - 1})"
        emit(f"    const int vc{c} = ({col}) * 4;            // byte offset of the lane's column")
        emit(f"    const int vo{c} = kq * {4 * nv} + vc{c};  // ... within the step's four rows")
    emit("    const float *pd = dcl + kq;")
    for u in range(PD):
        emit("    float " + ", ".join(f"g{u}_{c}" for c in range(NT)) + ";")

    def load(u, step, listed=False):
        # always issued, from a clamped row, so that the number of loads in flight is known at
        # compile time (a load under a condition makes every later wait a wait for all loads).
        # listed: the step's rows are entries 4 step .. 4 step + 3 of the list of contributing rows
        # (long variant; a step past the list reads its last entry and is never used)
        if listed:
            emit(f"        {{ const int li = 4 * ({step}) + kq; const int rowb = rowl[li < njp ? li : njp - 1] * {4 * nv};")
            for c in range(NT):
                emit(f"          g{u}_{c} = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(jrs, rowb + vc{c}, 0, 0));")
            emit("        }")
            return
        for c in range(NT):
            emit(f"        g{u}_{c} = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(jrs, vo{c}, ({step}) * {16 * nv}, 0));")

    def consume(u, step, listed=False, mixed=False):
        # rows at or past the world's nefc may hold anything: they count as zero rows; columns
        # past nv repeat the last column, which only reaches accumulator elements outside H.
        # listed: the step's rows come from the list of contributing rows, whose spare entries
        # name row 0 with weight 0 -- a row below nefc whenever a listed step runs at all
        # mixed (long variant): steps below SP are rows 4 st .. 4 st + 3 as they are, later ones are listed
        emit(f"        {{ const int st = {step}; const float d = pd[st * 4];" + ("" if listed else
             (f" const bool rv = st >= {SP} || st * 4 + kq < ne;" if mixed else " const bool rv = st * 4 + kq < ne;")))
        for c in range(NT):
            emit(f"          const float z{c} = " + (f"g{u}_{c};" if listed else f"rv ? g{u}_{c} : 0.0f;"))
        for c in range(NT):
            emit(f"          const float e{c} = d * z{c};")
        for n, (ti, tj) in enumerate(tiles):
            emit(f"          acc{n} = __builtin_amdgcn_mfma_f32_16x16x4f32(z{ti}, e{tj}, acc{n}, 0, 0, 0);")
        emit("        }")

    # Loads complete in issue order, so what the first step needs is requested first: the
    # accumulator index table, M (as a flat copy that is then gathered from LDS, so that the
    # table and M travel together instead of one after the other), the row weights; then J.
    MC = -(-nM // 64)
    _require(MC * 64 <= TW and nM < TW and 4 * nM < 32768, "M does not fit the staging copy")
    for n, (ti, tj) in enumerate(tiles):
        for v in range(4):
            emit(f"    const int ix{n}_{v} = IDX_{name}[{n * 4 + v}][lane];  // byte offset into the copy of M")
    # chain columns, needed right after the hand-over barrier: requested here, and pinned so that
    # the load is not moved down to its use
    for i in range(len(leaf_sets)):
        emit(f"    int chc{i} = CH_{name}[{i}][p];")
    for i in range(MC):
        emit(f"    const float mv{i} = M[wq * ldM + min({i * 64} + lane, {nM - 1})];")
    SP = min(PD, int(os.environ.get("IMHIP_SP", "2")))  # steps (4 rows each) requested before the row weights are known
    pin_ch = " ".join(f'asm volatile("" : "+v"(chc{i}));' for i in range(len(leaf_sets)))
    # Of the rows beyond the first 4 SP only the contributing ones are read: their numbers and
    # weights are packed behind entry 4 SP of a list, in row order (ballot and prefix count), so a
    # skipped row is one that would have added (J * 0) * J everywhere.  The first 4 SP rows are
    # requested before the weights are known and enter as they are, with weight 0 where they do
    # not contribute.  Short variant (njmax <= 64): one row per lane, every listed step in flight
    # at once.  Long variant: rows 64 lanes at a time, PD steps in flight in a loop.
    emit("    int steps = 0, cnt = 0;  // steps of four rows to run; length of the list behind the first rows")
    emit("    const int rc0 = lane < njmax ? lane : njmax - 1, rc1 = lane + 64 < njmax ? lane + 64 : njmax - 1;")
    emit("    const int sv0 = state[wq * njmax + rc0], sv1 = LONG ? state[wq * njmax + rc1] : 0;")
    emit("    const float dv0 = D[wq * njmax + rc0], dv1 = LONG ? D[wq * njmax + rc1] : 0.0f;")
    for u in range(SP):
        load(u, str(u))
    for ci in rhs_tables:
        emit(f"    yv{ci} = yw[chc{ci}];")
    emit(f"    float *mcopy = lds + wv * {TW};  // reused for this world's copy of H afterwards")
    for i in range(MC):
        emit(f"    mcopy[{i * 64} + lane] = mv{i};")
    emit(f"    mcopy[{nM}] = 0.0f;  // where the table sends accumulator elements outside the pattern")
    emit("    int *rowl = (int *)(dcl + (LONG ? njp : 64));")
    emit("    {")
    emit("      const unsigned long long below = (1ull << lane) - 1ull;")
    emit("      const bool act0 = lane < ne && sv0 == quad;")
    emit(f"      const bool tail = act0 && lane >= {4 * SP};")
    emit("      const unsigned long long tm = __ballot(tail);")
    emit("      cnt = __popcll(tm);")
    emit("      if (!LONG) { dcl[lane] = 0.0f; rowl[lane] = 0; }")
    emit(f"      if (lane < {4 * SP}) {{ dcl[lane] = act0 ? dv0 : 0.0f; rowl[lane] = lane; }}")
    emit(f"      if (tail) {{ const int pos = {4 * SP} + __popcll(tm & below); dcl[pos] = dv0; rowl[pos] = lane; }}")
    emit("      if (LONG) {")
    emit("        const bool act1 = lane + 64 < ne && sv1 == quad;")
    emit("        const unsigned long long tm1 = __ballot(act1);")
    emit(f"        if (act1) {{ const int pos = {4 * SP} + cnt + __popcll(tm1 & below); dcl[pos] = dv1; rowl[pos] = lane + 64; }}")
    emit("        cnt += __popcll(tm1);")
    emit("        for (int r0 = 128; r0 < njp; r0 += 64) {  // more than 128 rows")
    emit("          const int r = r0 + lane, rc = r < njmax ? r : njmax - 1;")
    emit("          const int sv = state[wq * njmax + rc]; const float dv = D[wq * njmax + rc];")
    emit("          const bool act = r < ne && sv == quad;")
    emit("          const unsigned long long tmr = __ballot(act);")
    emit(f"          if (act) {{ const int pos = {4 * SP} + cnt + __popcll(tmr & below); dcl[pos] = dv; rowl[pos] = r; }}")
    emit("          cnt += __popcll(tmr);")
    emit("        }")
    emit("        // the spare entries of the last step: row 0 with weight 0")
    emit(f"        if (lane < 3 && {4 * SP} + cnt + lane < njp) {{ dcl[{4 * SP} + cnt + lane] = 0.0f; rowl[{4 * SP} + cnt + lane] = 0; }}")
    emit("      }")
    emit(f"      steps = ne > {4 * SP} ? {SP} + ((cnt + 3) >> 2) : ((ne + 3) >> 2);")
    emit("    }")
    emit("    IM_WAVE_SYNC();")
    for u in range(SP, PD):
        load(u, str(u), listed=True)
    emit("    IM_WAVE_SYNC();")
    for n in range(len(tiles)):
        emit(f"    f32x4 acc{n};")
        for v in range(4):
            emit(f"    acc{n}[{v}] = *(const float *)((const char *)mcopy + ix{n}_{v});")
    emit("    IM_WAVE_SYNC();")
    emit("    " + pin_ch)
    emit("    STAMP();  // 1: row weights staged, M gathered")
    emit("    if (!LONG) {  // every row that is needed is already in flight")
    for u in range(PD):
        emit(f"      if ({u} < steps) {{")
        if u < SP:
            consume(u, str(u))
        else:
            consume(u, str(u), listed=True)
        emit("      }")
    emit("    } else {")
    emit(f"    for (int s0 = 0; s0 < steps; s0 += {PD}) {{")
    for u in range(PD):
        # guards instead of early exits: an exit from the middle of the unrolled body makes
        # the compiler keep two copies of every accumulator
        emit(f"      if (s0 + {u} < steps) {{")
        consume(u, f"s0 + {u}", mixed=True)
        emit("      }")
        # the next use of the register set is requested on every path: with the same number
        # of loads in flight whatever steps ran, each wait counts only the loads before it
        load(u, f"s0 + {u + PD}", listed=True)
    emit("    }")
    emit("    }")
    emit("    STAMP();  // 2: assembled")
    # accumulators -> lower triangle of H in LDS -> (wavefront 0) one register per row, lane = position on the chain
    for n, (ti, tj) in enumerate(tiles):
        guard = f"if (kq < {tile_rows[ti] // 4}) " if tile_rows[ti] < 16 else ""
        for v in range(4):
            emit(f"    {guard}lds[wv * {TW} + {band_off[ti]} + ({v} + 4 * kq) * {row_len[ti]} + {16 * tj} + p] = acc{n}[{v}];")
    emit("    STAMP();  // tiles written")
    emit("    __syncthreads();")
    emit("    STAMP();  // hand-over barrier passed")
    for i, (li, s) in enumerate(leaf_sets):
        emit(f"    lh{i} = lds + kq * {TW} + chc{i};")
    emit("  }")

    def bc(expr, pos):
        return f"IM_BC({expr}, {pos})"

    def fetch_rows(dofs):
        """rows of H into registers (fused kernel: from the copy in LDS), optional H output"""
        emit("    if (ASM) {")
        for b in dofs:
            for s in range(t.sets(b)):
                i = leaf_sets.index((t.leaf_of[b], s))
                emit(f"      h{b}_{s} = lh{i}[{h_off(b)}];")
        emit("      if (Hout && live && %d) {" % (0 if EXP == "timing" else 1))
        for b in dofs:
            for s in range(t.sets(b)):
                hi = t.depth[b] - 16 * s
                emit(f"        if (p <= {hi}) Hout[(int64_t)w * {nM} + {t.rowadr[b] + 16 * s} + p] = h{b}_{s};")
        emit("      }")
        emit("    } else {")
        emit("      const float *Mw = M + ws * ldM;")
        for b in dofs:
            for s in range(t.sets(b)):
                hi = t.depth[b] - 16 * s
                emit(f"      h{b}_{s} = Mw[{t.rowadr[b] + 16 * s} + (p < {hi} ? p : {hi})];")
        emit("    }")

    # group accumulators start from zero (tree_ldl.py:252-255)
    for j in range(ngroups):
        for a in sorted(touched[j]):
            for s in range(t.sets(a)):
                emit(f"  float ga{j}_{a}_{s} = 0.0f;")
    for k in range(nv):
        emit(f"  float nd{k} = 0.0f;  // -1 / pivot")
        if t.depth[k]:
            emit("  float " + ", ".join(f"T{k}_{s} = 0.0f" for s in range(t.sets(k))) + ";")

    def eliminate(k, j):
        """j: group index, or None for a trunk dof"""
        c = t.depth[k]
        nset = t.sets(k)
        emit(f"    // eliminate dof {k}")
        if j is not None and seg_of[k][1] > 0 and k == next(q for q in groups[j] if seg_of[q] == seg_of[k]):
            # a new branch of the group: its dofs take over the lanes past the fork
            i = seg_of[k][1]
            for s_ in range(vsets[j]):
                expr = sv(j, i - 1, s_)
                for src in sorted(set(segs[j][i]["restore"].values())):
                    mask = sum(1 << p for p in range(16) if segs[j][i]["restore"].get(16 * s_ + p) == src)
                    if mask:
                        expr = f"im_lane_select2({sv(j, src, s_)}, {expr}, IM_ROW_MASK(0x{mask:x}))"
                mask = sum(1 << p for p in range(16) if 16 * s_ + p in segs[j][i]["fresh"])
                if mask:
                    expr = f"im_lane_select2(SY{j}_{i}_{s_}, {expr}, IM_ROW_MASK(0x{mask:x}))"
                emit(f"    {sv(j, i, s_)} = {expr};")
        # the pivot's reciprocal is the head of the dependent chain from one pivot to the next: its
        # operand is fetched first, the products below (which need the row only) fill its latency
        emit(f"    const float piv{k} = {bc(f'h{k}_{c // 16}', c % 16)};")
        if c == 0:
            emit(f"    nd{k} = im_negative_reciprocal_checked(piv{k}, im_reciprocal_fast(-piv{k}));")
            return
        vec = (lambda s_: sv(*seg_of[k], s_)) if j is not None else (lambda s_: sv("T", 0, s_))
        # products m_kp * m_kq for every target register, the row eliminated next (the parent) first
        prods = []  # (pp, s, target)
        for pp in reversed(range(c)):
            a = t.anc[k][pp]
            to_acc = j is not None and a in trunk_set
            for s in range(t.sets(a)):
                prods.append((pp, s, f"ga{j}_{a}_{s}" if to_acc else f"h{a}_{s}"))
        # lanes at and past the dof's own position must not take part in the right-hand side
        # update (they hold other dofs' entries), and there the row register holds no data
        nsv = (c - 1) // 16 + 1
        for s_ in range(nsv):
            hi = c - 16 * s_
            emit(f"    const float hm{k}_{s_} = " + (f"im_lane_select(h{k}_{s_}, IM_ROW_MASK(0x{(1 << hi) - 1:x}));" if hi < 16 else f"h{k}_{s_};"))
        if prods:
            emit("    float " + ", ".join(f"t{k}_{pp}_{s}" for pp, s, _ in prods) + ";")

        def pack(work, weave_reciprocal=False):
            """inline-assembly statements of at most 28 operands each for the listed items; with
            weave_reciprocal the first statement also starts the pivot's reciprocal (hardware
            estimate, residual, correction: im_reciprocal_fast) with the products in its latency"""
            pos = 0
            first = True
            while pos < len(work):
                # No wait states in front of these statements: a register they read through DPP was
                # written at least two instructions earlier -- the pivot row by the update before the
                # compiler's own DPP read of its diagonal, the right-hand side vector before the
                # statement with the products
                o, n_in, lines = [], [], []
                num = {}
                weave = weave_reciprocal and first
                first = False
                if weave:
                    o += [f'"=&v"(df{k})', f'"=&v"(de{k})']
                    num["df"], num["de"] = ("o", 0), ("o", 1)
                    num["piv"] = ("i", 0)
                    n_in.append(f'"v"(piv{k})')

                def use_in(tag, text):
                    if tag not in num:
                        num[tag] = ("i", len(n_in))
                        n_in.append(text)
                    return tag

                items = []
                while pos < len(work):
                    it = work[pos]
                    if it[0] == "T":
                        need_i = (("hm", it[1]) not in num) + ("nd" not in num)
                    elif it[0] == "P":
                        need_i = (("h", it[1] // 16) not in num) + (("h", it[2]) not in num)
                    else:
                        need_i = (("Tin", it[1]) not in num and ("T", it[1]) not in num) + (("V", c // 16) not in num)
                    if len(o) + 1 + len(n_in) + need_i > 28:
                        break
                    if it[0] == "T":
                        s = it[1]
                        num[("T", s)] = ("o", len(o))
                        o.append(f'"=&v"(T{k}_{s})')
                        use_in(("hm", s), f'"v"(hm{k}_{s})')
                        use_in("nd", f'"v"(nd{k})')
                    elif it[0] == "P":
                        _, pp, s = it
                        num[("t", pp, s)] = ("o", len(o))
                        o.append(f'"=&v"(t{k}_{pp}_{s})')
                        use_in(("h", pp // 16), f'"v"(h{k}_{pp // 16})')
                        use_in(("h", s), f'"v"(h{k}_{s})')
                    else:
                        _, s = it
                        if ("V", s) not in num:
                            num[("V", s)] = ("o", len(o))
                            o.append(f'"+v"({vec(s)})')
                        if ("V", c // 16) not in num:
                            num[("V", c // 16)] = ("o", len(o))
                            o.append(f'"+v"({vec(c // 16)})')
                        if ("T", s) not in num:
                            use_in(("Tin", s), f'"v"(T{k}_{s})')
                    items.append(it)
                    pos += 1

                def r_(tag):
                    kind, n = num[tag]
                    return f"%{n}" if kind == "o" else f"%{len(o) + n}"

                body = []
                for it in items:
                    if it[0] == "T":
                        body.append(f"v_mul_f32 {r_(('T', it[1]))}, {r_(('hm', it[1]))}, {r_('nd')}")
                    elif it[0] == "P":
                        _, pp, s = it
                        body.append(f"v_mul_f32_dpp {r_(('t', pp, s))}, {r_(('h', pp // 16))}, {r_(('h', s))} row_newbcast:{pp % 16} {DPP}")
                    else:
                        _, s = it
                        tsrc = ("T", s) if ("T", s) in num else ("Tin", s)
                        # entry of dof k (lane c of its set, untouched by this update) times T, added per lane
                        body.append(f"v_fmac_f32_dpp {r_(('V', s))}, {r_(('V', c // 16))}, {r_(tsrc)} row_newbcast:{c % 16} {DPP}")
                if weave:
                    # estimate first, the residual after four products, the correction after two more;
                    # a transcendental's result needs two instructions' distance before its first use
                    n_e, n_r = min(4, len(body)), min(6, len(body))
                    # of the negated pivot: -1 / pivot is what the updates multiply with
                    body[n_r:n_r] = [f"v_fma_f32 {r_('df')}, {r_('de')}, {r_('df')}, {r_('df')}"]
                    body[n_e:n_e] = (["s_nop 1"] if n_e < 2 else []) + [f"v_fma_f32 {r_('de')}, {r_('piv')}, {r_('df')}, 1.0"]
                    body.insert(0, f"v_rcp_f32_e64 {r_('df')}, -{r_('piv')}")
                lines += body
                text = "\\n\\t".join(lines)
                emit(f'    asm("{text}" : {", ".join(o)} : {", ".join(n_in)});')

        emit(f"    float df{k}, de{k};")
        # eight products at a time, each batch followed by its updates: the temporaries of a deep
        # row would otherwise all be live at once
        BATCH = 8
        pack([("P", pp, s) for pp, s, _ in prods[:BATCH]], weave_reciprocal=True)
        emit(f"    nd{k} = im_negative_reciprocal_checked(piv{k}, df{k});")
        for pp, s, tgt in prods[:BATCH]:
            emit(f"    {tgt} = IM_FMA(t{k}_{pp}_{s}, nd{k}, {tgt});")
        for b0 in range(BATCH, len(prods), BATCH):
            pack([("P", pp, s) for pp, s, _ in prods[b0 : b0 + BATCH]])
            for pp, s, tgt in prods[b0 : b0 + BATCH]:
                emit(f"    {tgt} = IM_FMA(t{k}_{pp}_{s}, nd{k}, {tgt});")
        # T = h * nd and the right-hand side update
        pack([("T", s) for s in range(nsv)] + [("R", s) for s in range(nsv)])

    def backsub_many(dofs):
        """Solutions of `dofs` (ancestors first): u_b = u_b d_b, then u_b += T_b[p] u_anc_p for p
        ascending (tree_ldl.py:298-304); the entry of dof b is lane c of its chain's right-hand side
        vector.  A dof's sum is a chain of dependent instructions, so the chains of all dofs are
        emitted interleaved, a term as soon as the ancestor it needs is complete: the order of
        each dof's own terms is untouched."""
        dofs = list(dofs)
        inset = set(dofs)
        emitted = {b: -1 for b in dofs}  # -1: the product with d_b is still to come
        complete, seq = set(), []
        while len(complete) < len(dofs):
            newly, before = [], len(seq)
            for b in dofs:
                if b in complete or b in newly:
                    continue
                if emitted[b] == -1:
                    seq.append((b, None))
                    emitted[b] = 0
                else:
                    a_ = t.anc[b][emitted[b]]
                    if a_ in inset and a_ not in complete:
                        continue
                    seq.append((b, emitted[b]))
                    emitted[b] += 1
                if emitted[b] == t.depth[b]:
                    newly.append(b)
            _require(bool(newly) or len(seq) > before, "back-substitution order does not close")
            complete.update(newly)

        def src_of(b_):
            c_ = t.depth[b_]
            return sv(seg_of[b_][0], home[seg_of[b_][0]]["g", b_], c_ // 16) if b_ in seg_of else sv("T", 0, c_ // 16)

        pos, first_stmt = 0, True
        while pos < len(seq):
            outs, ins, lines = {}, {}, (["s_nop 1"] if first_stmt else [])
            first_stmt = False

            def need(b_, pp):
                names = [("o", f"S{b_}")]
                if pp is None:
                    names += [("i", src_of(b_)), ("i", f"nd{b_}")]
                else:
                    names += [("i", f"T{b_}_{pp // 16}"), ("oi", f"S{t.anc[b_][pp]}")]
                return names

            while pos < len(seq):
                b_, pp = seq[pos]
                extra = 0
                for kind, nm in need(b_, pp):
                    if nm in outs or nm in ins:
                        continue
                    extra += 1
                if len(outs) + len(ins) + extra > 26 and (outs or ins):
                    break
                for kind, nm in need(b_, pp):
                    if nm in outs or nm in ins:
                        continue
                    if kind == "o":
                        outs[nm] = None
                    else:
                        ins[nm] = None
                pos += 1
                lines.append((b_, pp))
            # an S read before this statement writes it is an input-output as well: "+v" covers both
            olist = list(outs)
            ilist = [nm for nm in ins if nm not in outs]
            ref = {nm: f"%{n}" for n, nm in enumerate(olist)}
            ref.update({nm: f"%{len(olist) + n}" for n, nm in enumerate(ilist)})
            text = []
            for item in lines:
                if isinstance(item, str):
                    text.append(item)
                    continue
                b_, pp = item
                if pp is None:
                    text.append(f"v_mul_f32_dpp {ref[f'S{b_}']}, {ref[src_of(b_)]}, -{ref[f'nd{b_}']} row_newbcast:{t.depth[b_] % 16} {DPP}")
                else:
                    text.append(f"v_fmac_f32_dpp {ref[f'S{b_}']}, {ref[f'T{b_}_{pp // 16}']}, {ref[f'S{t.anc[b_][pp]}']} row_newbcast:{pp % 16} {DPP}")
            joined = "\\n\\t".join(text)
            o_txt = ", ".join('"+v"(%s)' % nm for nm in olist)
            i_txt = ", ".join('"v"(%s)' % nm for nm in ilist)
            emit(f'    asm("{joined}" : {o_txt} : {i_txt});')

    def store_x(dofs):
        emit("    if (live && p == 0) {")
        emit("      float *xw = x + (int64_t)w * ldx;")
        emit("      if (flags & IM_FLAG_NEGATE) {")
        for b in dofs:
            emit(f"        xw[{b}] = -S{b};")
        emit("      } else {")
        for b in dofs:
            emit(f"        xw[{b}] = S{b};")
        emit("      }")
        emit("    }")

    # ---- phase 1: the groups, each into its own zero-initialised trunk accumulators
    # Each role's work is a lambda per phase, called from one branch per wavefront below: a
    # wavefront's path through the kernel then holds its own role's values only (with the roles
    # as guarded blocks one after the other, every role's values stay allocated across the others' code).
    LAMBDA = "[&]() __attribute__((always_inline))"
    for j, g in enumerate(groups):
        emit(f"  auto phase1_{j} = {LAMBDA} {{  // group {j}")
        emit("    if (ASM) {")
        for i in range(len(segs[j])):
            for s_ in range(vsets[j]):
                take_rhs(j, i, s_, sv(j, 0, s_) if i == 0 else f"SY{j}_{i}_{s_}")
        emit("    } else {")
        for i in range(len(segs[j])):
            for s_ in range(vsets[j]):
                load_sv(j, i, s_, sv(j, 0, s_) if i == 0 else f"SY{j}_{i}_{s_}")
        emit("    }")
        fetch_rows(sorted(g))
        if j == 0:
            emit("    STAMP();  // group 0: rows fetched")
        for k in g:
            eliminate(k, j)
        if j == 0:
            emit("    STAMP();  // group 0: eliminated")
        for s_ in range(vsets[j]):
            expr = sv(j, len(segs[j]) - 1, s_)
            by_src = {}
            for a_ in touched[j]:
                if t.depth[a_] // 16 == s_ and home[j]["t", a_] != len(segs[j]) - 1:
                    by_src.setdefault(home[j]["t", a_], 0)
                    by_src[home[j]["t", a_]] |= 1 << (t.depth[a_] % 16)
            for src, mask in sorted(by_src.items()):
                expr = f"im_lane_select2({sv(j, src, s_)}, {expr}, IM_ROW_MASK(0x{mask:x}))"
            emit(f"    SP{j}_{s_} = {expr};")
        emit("    if (SPLIT) {")
        for (a, s_), off in xslots[j].items():
            src = f"SP{j}_{s_}" if a == "S" else f"ga{j}_{a}_{s_}"
            emit(f"      xlds[{xo(off)} + lane] = {src};")
        emit("    }")
        emit("  };")
    # ---- phase 2: trunk rows = own value plus the groups' contributions in group order
    # (tree_ldl.py:274-289), eliminated in reverse, then solved root first
    emit(f"  auto phase2 = {LAMBDA} {{  // trunk")
    emit("    if (ASM) {")
    for s_ in range(tsets):
        take_rhs("T", 0, s_, f"SVT_{s_}")
    emit("    } else {")
    for s_ in range(tsets):
        load_sv("T", 0, s_, f"SVT_{s_}")
    emit("    }")
    fetch_rows(list(trunk))
    for a in trunk:
        for j in range(ngroups):
            if a in touched[j]:
                for s in range(t.sets(a)):
                    emit(f"    h{a}_{s} = h{a}_{s} + (SPLIT ? xlds[{xo(xslots[j][a, s])} + lane] : ga{j}_{a}_{s});")
    # right-hand side: the lanes a group touched take its sums, in group order
    for j in range(ngroups):
        for s_ in range(min(tsets, vsets[j])):
            mask = sum(1 << p for p in range(16) if any(t.depth[a] == 16 * s_ + p for a in touched[j]))
            if mask:
                emit(f"    SVT_{s_} = im_lane_select2(SVT_{s_} + (SPLIT ? xlds[{xo(xslots[j]['S', s_])} + lane] : SP{j}_{s_}), SVT_{s_}, IM_ROW_MASK(0x{mask:x}));")
    emit("    STAMP();  // trunk: rows fetched and merged")
    for k in reversed(trunk):
        eliminate(k, None)
    emit("    STAMP();  // trunk: eliminated")
    backsub_many(trunk)
    emit("    STAMP();  // trunk: solved")
    emit("    if (SPLIT && p == 0) {")
    for b in trunk:
        emit(f"      xlds[{xo(xs_off)} + (lane >> 4) * {nv} + {b}] = S{b};")
    emit("    }")
    store_x(list(trunk))
    emit("  };")
    # ---- phase 3: the groups' solutions, ancestors first
    for j, g in enumerate(groups):
        emit(f"  auto phase3_{j} = {LAMBDA} {{")
        if j != 0:
            emit("    if (SPLIT) {")
            for a in sorted(touched[j]):
                emit(f"      S{a} = xlds[{xo(xs_off)} + (lane >> 4) * {nv} + {a}];")
            emit("    }")
        backsub_many(list(reversed(g)))
        store_x(sorted(g))
        emit("  };")
    emit("  if (SPLIT) {")
    for j in range(max(ngroups, 1)):
        emit(("    if" if j == 0 else "    } else if") + f" (wv == {j}) {{")
        if j < ngroups:
            emit(f"      phase1_{j}();")
        emit("      IM_BLOCK_SYNC();")
        if j == 0:
            emit("      STAMP();  // groups eliminated")
            emit("      phase2();")
        emit("      IM_BLOCK_SYNC();")
        if j == 0:
            emit("      STAMP();  // trunk solved")
        if j < ngroups:
            emit(f"      phase3_{j}();")
    emit("    } else {  // a wavefront without a group only keeps the barriers' count")
    emit("      IM_BLOCK_SYNC();")
    emit("      IM_BLOCK_SYNC();")
    emit("    }")
    emit("  } else {")
    for j in range(ngroups):
        emit(f"    phase1_{j}();")
    emit("    phase2();")
    for j in range(ngroups):
        emit(f"    phase3_{j}();")
    emit("  }")
    emit("  STAMP();")
    emit("  #undef STAMP")
    emit("}")
    args = "M, ldM, J, njmax, D, state, nefc_p, quad, y, ldy, x, ldx, Hout, nworld, flags, niter, state_it, y_it, x_it, skip"
    # The resident Newton loop with this tree's fused kernel as its factor stage: search = -H^-1 grad
    # for the workgroup's four worlds, those whose `unchanged` byte is set left alone.  The line
    # search keeps a lane's two rows in registers up to 64 rows (the short kernel) and reads the rows
    # from LDS at every evaluation beyond.
    emit("template <bool LONG>")
    emit(f"__device__ __forceinline__ void newton_row16_body_{name}(const im::resident::NewtonArgs &a) {{")
    emit("  extern __shared__ float xlds[];")
    emit("  const int *worlds = (const int *)(xlds + a.stage_lds_floats) + 4;  // behind the four votes (coop_layout)")
    emit("  auto stage = [&]() __attribute__((always_inline)) {")
    emit("    const im::resident::NewtonArgs &a = im::resident::kernel_args(0);  // the kernel's only argument")
    emit(f"    tree_row16_body_{name}<true, LONG>(a.M, a.ldM, a.J, a.njmax, a.D, a.state, a.nefc, a.quad, a.grad, a.ld_grad, a.search,")
    emit("        (int64_t)a.nv, nullptr, a.nworld, IM_FLAG_NEGATE, 1, 0, 0, 0, a.unchanged, worlds);")
    emit("  };")
    emit("  const im::resident::LoopLds L = im::resident::coop_layout(a, xlds);")
    emit("  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);")
    emit("  im::resident::block_sync();")
    # rows a lane keeps in registers during the line search: two up to 64 rows, four up to 128 (the
    # same for the whole launch), beyond that the rows are read from LDS at every evaluation
    emit("  if (!LONG)")
    emit("    im::resident::newton_loop<2, 0, true>(0, L, w, stage);")
    emit("  else if (a.njmax <= 128)")
    emit("    im::resident::newton_loop<4, 0, true>(0, L, w, stage);")
    emit("  else")
    emit("    im::resident::newton_loop<0, 0, true>(0, L, w, stage);")
    emit("}")
    if module:
        emit("} }  // namespace im::gen")
        for kernel, asm_, long_, bounds in (("fused", "true", "false", f"256, IM_OCC_{name}"), ("fused_long", "true", "true", f"256, IM_OCC_{name}"),
                                            ("solve", "false", "false", f"256, IM_NOCC_{name}")):  # fmt: skip
            emit(f'extern "C" __global__ __launch_bounds__({bounds}) void im_row16_{kernel}(IM_ROW16_PARAMS) {{')
            emit(f"  im::gen::tree_row16_body_{name}<{asm_}, {long_}, true>({args}, nullptr);")
            emit("}")
        for kernel, long_ in (("newton", "false"), ("newton_long", "true")):
            emit(f'extern "C" __global__ __launch_bounds__(256, IM_NOCC_{name}) void im_row16_{kernel}(im::resident::NewtonArgs a) {{')
            emit(f"  im::gen::newton_row16_body_{name}<{long_}>(a);")
            emit("}")
        emit(f'extern "C" __device__ const unsigned long long im_row16_key = 0x{key:016x}ull;')
        emit(f'extern "C" __device__ const int im_row16_info[5] = {{{nv}, {nM}, {lds_floats * 4}, {4 * PD}, {(lds_floats - 4 * TW) * 4}}};  // nv, nM, LDS bytes, short rows, LDS bytes of the solve-only kernel')
    else:
        emit("template <bool ASM, bool LONG>")
        # (the solve-only kernel fetches a group's rows of H from memory at once and holds a few values
        # more than the fused one: it shares the Newton kernels' occupancy)
        emit(f"__global__ __launch_bounds__(256, ASM ? IM_OCC_{name} : IM_NOCC_{name}) void tree_row16_{name}(IM_ROW16_PARAMS) {{")
        emit(f"  tree_row16_body_{name}<ASM, LONG, true>({args}, nullptr);")
        emit("}")
        emit("template <bool LONG>")
        emit(f"__global__ __launch_bounds__(256, IM_NOCC_{name}) void newton_row16_{name}(im::resident::NewtonArgs a) {{")
        emit(f"  newton_row16_body_{name}<LONG>(a);")
        emit("}")
        emit(f"static const Row16Entry entry_{name} = {{0x{key:016x}ull, {nv}, {nM}, {lds_floats * 4}, {4 * PD}, \"{name}\",")
        emit(f"    (const void *)tree_row16_{name}<true, false>, (const void *)tree_row16_{name}<true, true>,")
        emit(f"    (const void *)tree_row16_{name}<false, false>, (const void *)newton_row16_{name}<false>,")
        emit(f"    (const void *)newton_row16_{name}<true>, {(lds_floats - 4 * TW) * 4}}};")
        emit(f"static const Row16Register reg_{name}(&entry_{name});")
        emit("} }  // namespace im::gen")
    # workgroups per CU that the fused kernel is compiled for: what the 160 KB of LDS admit (with
    # the lists of 128 constraint rows), at most 4 -- fewer workgroups leave each wavefront more
    # registers, which the larger trees need
    asked = int(os.environ.get("IMHIP_OCC", "4"))
    if not 1 <= asked <= 4:
        # a workgroup is four wavefronts, one per SIMD, so this is also the wavefronts per SIMD whose
        # register budget the compiler keeps to: beyond 4 (fewer than 128 registers) the larger trees
        # spill to memory, and such a build once ended in a GPU memory fault
        raise ValueError(f"IMHIP_OCC={asked}: the generated kernels are built for 1 to 4 workgroups per CU")
    occ = max(1, min(asked, (160 * 1024) // (lds_floats * 4 + 32 * 128)))
    text = "\n".join(out) + "\n"
    header = '#include "tree_row16.h"' if module else '#include "../tree_row16.h"'  # a module is built with -I csrc
    # the resident Newton kernels carry the loop's state on top of the stage's rows: whoever compiles
    # the source may give them fewer workgroups per CU (more registers) with -DIM_NOCC_<name>=n
    # where they would otherwise spill
    defines = f"#define IM_OCC_{name} {occ}\n#ifndef IM_NOCC_{name}\n#define IM_NOCC_{name} IM_OCC_{name}\n#endif"
    return text.replace('#include "../tree_row16.h"', f"{header}\n{defines}", 1)


def occupancy_of(source: str) -> tuple[str, int]:
    """(kernel set name, workgroups per CU) that a generated source was written for."""
    import re

    m = re.search(r"#define IM_OCC_(\w+) (\d+)", source)
    if not m:
        raise ValueError("not a generated tree kernel source")
    return m.group(1), int(m.group(2))
