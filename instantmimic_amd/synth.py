"""Seeded synthetic batches for the five benchmark shapes.

There is no network and no MuJoCo in the build image, so every shape is
generated: a dof tree (MuJoCo dof order, parent < child), a tree-sparse SPD
``M`` in MuJoCo's CSR (row = ancestors root-first, diagonal last), constraint
rows ``J`` supported on one root-to-leaf chain each, regularisers ``D``, a
constraint ``state`` array (QUADRATIC = active) and a gradient.

All draws use ``numpy.random.default_rng([seed, block])`` in fp64 over blocks of
``BLOCK`` worlds and are cast to fp32, so the first ``n`` worlds of a batch do
not depend on the batch size.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace

import numpy as np

QUADRATIC = 1  # mjtConstraintState.mjCNSTRSTATE_QUADRATIC
BLOCK = 256


def _chain(parent_of_first: int, first: int, n: int) -> list[int]:
    return [parent_of_first] + list(range(first, first + n - 1))


def ant_parents() -> list[int]:
    # free joint (0..5) + four legs of two hinges hanging off dof 5
    return [-1, 0, 1, 2, 3, 4, 5, 6, 5, 8, 5, 10, 5, 12]


def humanoid_parents() -> list[int]:
    # MuJoCo humanoid.xml order: root 6, abdomen z/y/x, right leg 6, left leg 6,
    # right arm 3, left arm 3
    return [-1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 8, 15, 16, 17, 18, 19, 5, 21, 22, 5, 24, 25]


def g1_parents() -> list[int]:
    p = [-1, 0, 1, 2, 3, 4]
    p += _chain(5, 6, 6)  # left leg 6..11
    p += _chain(5, 12, 6)  # right leg 12..17
    p += _chain(5, 18, 3)  # waist 18..20
    p += _chain(20, 21, 7)  # left arm 21..27
    p += _chain(20, 28, 7)  # right arm 28..34
    return p


def snu_parents() -> list[int]:
    # pelvis 6; legs (hip ball, knee, ankle ball, 3 foot hinges) 10 dofs each off
    # dof 5; spine two balls (26..31) off dof 5; neck ball + head hinge off the
    # spine end; arms (clavicle, shoulder balls, elbow, wrist ball) 10 each.
    p = [-1, 0, 1, 2, 3, 4]
    p += _chain(5, 6, 10)
    p += _chain(5, 16, 10)
    p += _chain(5, 26, 6)
    p += _chain(31, 32, 4)
    p += _chain(31, 36, 10)
    p += _chain(31, 46, 10)
    return p


def stress_parents() -> list[int]:
    # serial trunk of 64 dofs, an 8-dof side chain off trunk dofs 7, 15, ..., 63
    p = [-1] + list(range(63))
    first = 64
    for t in range(7, 64, 8):
        p += _chain(t, first, 8)
        first += 8
    return p


def limbs_parents(limbs: int = 4, links: int = 6) -> list[int]:
    """Free torso with ``limbs`` hinge chains (the reference's test model,
    tests/test_tree_ldl.py:49-60)."""
    p = [-1, 0, 1, 2, 3, 4]
    for n in range(limbs):
        p += _chain(5, 6 + n * links, links)
    return p


def branched_parents() -> list[int]:
    """Free root with a hinge-hinge branch and a ball-slide branch, plus a second
    free body (the reference's test model, tests/test_tree_ldl.py:22-36)."""
    return [-1, 0, 1, 2, 3, 4, 5, 6, 5, 8, 9, 10, -1, 12, 13, 14, 15, 16]


def chain_parents(hinges: int = 30) -> list[int]:
    return [-1] + list(range(5 + hinges))


def extra_trees() -> dict[str, list[int]]:
    """Dof trees beside the five benchmark shapes that the tests and the per-kernel timings run the
    generated kernels on: the reference's test models, torsos with limbs of 62, 70 and 78 dofs, the contact
    model's tree and the SNU-like tree with a second free body."""
    snu_free = snu_parents()
    n0 = len(snu_free)
    snu_free += [-1] + list(range(n0, n0 + 5))
    return {
        "limbs": limbs_parents(), "branched": branched_parents(), "limbs62": limbs_parents(8, 7),
        "limbs70": limbs_parents(8, 8), "limbs78": limbs_parents(6, 12),
        "contact": [int(p) for p in contact_model()[0].dof_parentid], "snu_free": snu_free,
    }  # fmt: skip


def csr_from_parents(parent) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """MuJoCo's M CSR for a dof tree: ``rowadr, rownnz, colind`` (int32)."""
    rowadr, rownnz, colind = [], [], []
    for k in range(len(parent)):
        chain = []
        p = k
        while p >= 0:
            chain.append(p)
            p = parent[p]
        rowadr.append(len(colind))
        rownnz.append(len(chain))
        colind += chain[::-1]
    return (np.asarray(rowadr, np.int32), np.asarray(rownnz, np.int32), np.asarray(colind, np.int32))


@dataclass(frozen=True)
class Shape:
    name: str
    parents: tuple
    nefc: int
    worlds: int
    mass: tuple
    armature: float
    logd: tuple
    p_active: float
    iterations: int
    seed: int
    dense_rows: bool = False
    nmuscle: int = 0
    extra: dict = field(default_factory=dict)

    @property
    def nv(self) -> int:
        return len(self.parents)


SHAPES = {
    "ant": Shape("ant", tuple(ant_parents()), 32, 64, (0.1, 2.0), 0.01, (-3.0, 3.0), 0.5, 1, 1000),
    "humanoid": Shape("humanoid", tuple(humanoid_parents()), 64, 4096, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 3, 1001),
    "g1": Shape("g1", tuple(g1_parents()), 96, 8192, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 1, 1002),
    "snu": Shape("snu", tuple(snu_parents()), 128, 4096, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 1, 1003, nmuscle=284),
    "stress": Shape("stress", tuple(stress_parents()), 256, 16384, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.5, 3, 1004, dense_rows=True),
}


@dataclass
class Batch:
    shape: Shape
    rowadr: np.ndarray
    rownnz: np.ndarray
    colind: np.ndarray
    M: np.ndarray  # (nworld, nM) fp32, CSR values
    J: np.ndarray  # (nworld, nefc, nv) fp32
    D: np.ndarray  # (nworld, nefc) fp32
    state: np.ndarray  # (iterations, nworld, nefc) int32
    nefc: np.ndarray  # (nworld,) int32
    grad: np.ndarray  # (nworld, nv) fp32

    @property
    def nworld(self) -> int:
        return self.M.shape[0]


def chain_mask(parent) -> np.ndarray:
    """mask[k, i] = 1 when i is k or one of k's ancestors."""
    nv = len(parent)
    mask = np.zeros((nv, nv), dtype=bool)
    for k in range(nv):
        p = k
        while p >= 0:
            mask[k, p] = True
            p = parent[p]
    return mask


def make_batch(shape: Shape | str, nworld: int | None = None, *, ragged_nefc: bool = False, supports=None) -> Batch:
    """``supports`` (optional, (nsup, nv) bool): the dof sets a constraint row may be
    supported on, instead of single root-to-leaf chains."""
    if isinstance(shape, str):
        shape = SHAPES[shape]
    nworld = shape.worlds if nworld is None else int(nworld)
    nv, nefc = shape.nv, shape.nefc
    parent = list(shape.parents)
    rowadr, rownnz, colind = csr_from_parents(parent)
    rowi = np.repeat(np.arange(nv), rownnz)
    mask = chain_mask(parent)
    nM = colind.size
    M = np.empty((nworld, nM), np.float32)
    J = np.empty((nworld, nefc, nv), np.float32)
    D = np.empty((nworld, nefc), np.float32)
    state = np.empty((shape.iterations, nworld, nefc), np.int32)
    grad = np.empty((nworld, nv), np.float32)
    nefc_w = np.full((nworld,), nefc, np.int32)
    for b0 in range(0, nworld, BLOCK):
        rng = np.random.default_rng([shape.seed, b0 // BLOCK])
        nb = BLOCK
        mass = rng.uniform(shape.mass[0], shape.mass[1], (nb, nv))
        V = rng.standard_normal((nb, nv, nv)) * mask[None]
        dense = np.einsum("wk,wki,wkj->wij", mass, V, V, optimize=True)
        dense[:, np.arange(nv), np.arange(nv)] += shape.armature
        body = rng.integers(0, nv, (nb, nefc))
        rows = rng.standard_normal((nb, nefc, nv))
        if supports is not None:
            sup = np.asarray(supports, bool)
            rows *= sup[body % sup.shape[0]]
        elif not shape.dense_rows:
            rows *= mask[body]
        logd = rng.uniform(shape.logd[0], shape.logd[1], (nb, nefc))
        act = rng.random((shape.iterations, nb, nefc)) < shape.p_active
        g = rng.standard_normal((nb, nv))
        ragged = rng.integers(0, nefc + 1, (nb,))
        n = min(nb, nworld - b0)
        M[b0 : b0 + n] = dense[:n, rowi, colind]
        J[b0 : b0 + n] = rows[:n]
        D[b0 : b0 + n] = 10.0 ** logd[:n]
        state[:, b0 : b0 + n] = np.where(act[:, :n], QUADRATIC, 0)
        grad[b0 : b0 + n] = g[:n]
        if ragged_nefc:
            nefc_w[b0 : b0 + n] = ragged[:n]
    return Batch(shape, rowadr, rownnz, colind, M, J, D, state, nefc_w, grad)


def dense_from_csr(values: np.ndarray, rowadr, rownnz, colind) -> np.ndarray:
    """Symmetric dense (nworld, nv, nv) fp64 matrix from CSR lower-triangle values."""
    nv = len(rowadr)
    rowi = np.repeat(np.arange(nv), rownnz)
    out = np.zeros((values.shape[0], nv, nv), np.float64)
    out[:, rowi, colind] = values
    out[:, colind, rowi] = values
    return out


# ------------------------------------------------------------------ muscles (SNU-like shape)


def snu_joint_chains() -> list[list[list[int]]]:
    """Root-to-leaf joint chains of the SNU-like tree below the pelvis; a joint is the
    list of its dofs (ball = 3 chained dofs, hinge = 1)."""

    def leg(b):
        return [[b, b + 1, b + 2], [b + 3], [b + 4, b + 5, b + 6], [b + 7], [b + 8], [b + 9]]

    def arm(b):
        return [[b, b + 1, b + 2], [b + 3, b + 4, b + 5], [b + 6], [b + 7, b + 8, b + 9]]

    spine = [[26, 27, 28], [29, 30, 31]]
    return [leg(6), leg(16), spine + [[32, 33, 34], [35]], spine + arm(36), spine + arm(46)]


@dataclass
class MuscleBatch:
    nmuscle: int
    root_dof_count: int
    muscle_dofs: np.ndarray  # (nentry, 2) (muscle, torque dof), sorted by muscle then dof
    moment: np.ndarray  # (nworld, nentry) fp32
    force: np.ndarray  # (nworld, nmuscle) fp32
    slope: np.ndarray  # (nworld, nmuscle) fp32
    timestep: float


def make_muscles(nworld: int, nmuscle: int = 284, seed: int = 1003) -> MuscleBatch:
    """284 muscles, each spanning 1-3 adjacent joints of one chain; moment-arm entries
    ~N(0, 0.05); f = a f_max l + f_passive; slope = df/dl ~ U[0, 1e3]."""
    rng = np.random.default_rng([seed, 77])
    chains = snu_joint_chains()
    root = 6
    pairs = []
    for m in range(nmuscle):
        chain = chains[int(rng.integers(len(chains)))]
        span = int(rng.integers(1, 4))
        first = int(rng.integers(0, len(chain) - span + 1))
        for joint in chain[first : first + span]:
            pairs += [(m, d - root) for d in joint]
    md = np.unique(np.asarray(pairs, np.int64), axis=0)
    nentry = md.shape[0]
    moment = np.empty((nworld, nentry), np.float32)
    force = np.empty((nworld, nmuscle), np.float32)
    slope = np.empty((nworld, nmuscle), np.float32)
    for b0 in range(0, nworld, BLOCK):
        r = np.random.default_rng([seed, 78, b0 // BLOCK])
        a = r.normal(0.0, 0.05, (BLOCK, nentry))
        act = r.uniform(0, 1, (BLOCK, nmuscle))
        fmax = r.uniform(100, 3000, (BLOCK, nmuscle))
        lf = r.uniform(0.5, 1.0, (BLOCK, nmuscle))
        fp = r.uniform(0, 50, (BLOCK, nmuscle))
        sl = r.uniform(0, 1e3, (BLOCK, nmuscle))
        n = min(BLOCK, nworld - b0)
        moment[b0 : b0 + n] = a[:n]
        force[b0 : b0 + n] = (act * fmax * lf + fp)[:n]
        slope[b0 : b0 + n] = sl[:n]
    return MuscleBatch(nmuscle, root, md, moment, force, slope, 1.0 / 480.0)


def matrix_elemid(rowadr, rownnz, colind) -> np.ndarray:
    """(nv, nv) table: CSR index of M's element (i, j), either order, -1 off the pattern."""
    nv = len(rowadr)
    out = np.full((nv, nv), -1, np.int32)
    rowi = np.repeat(np.arange(nv), rownnz)
    out[rowi, colind] = np.arange(len(colind))
    out[colind, rowi] = np.arange(len(colind))
    return out


def model_from_parents(parent, joints: list[list[int]] | None = None):
    """A minimal model namespace (the fields the planners read) for a dof tree.  Bodies:
    one per joint (``joints`` lists each joint's dofs; default one dof per body); body 0 is
    the world."""
    from types import SimpleNamespace

    parent = list(parent)
    nv = len(parent)
    if joints is None:
        joints = [[d] for d in range(nv)]
    body_of_dof = {}
    for b, dofs in enumerate(joints, start=1):
        for d in dofs:
            body_of_dof[d] = b
    body_parentid, body_dofadr, body_dofnum = [0], [-1], [0]
    for dofs in joints:
        p = parent[dofs[0]]
        body_parentid.append(body_of_dof[p] if p >= 0 else 0)
        body_dofadr.append(dofs[0])
        body_dofnum.append(len(dofs))
    rowadr, rownnz, colind = csr_from_parents(parent)
    return SimpleNamespace(
        nv=nv, nv_pad=((nv + 1 + 15) // 16) * 16, dof_parentid=np.asarray(parent, np.int32),
        body_parentid=np.asarray(body_parentid, np.int32), body_dofadr=np.asarray(body_dofadr, np.int32),
        body_dofnum=np.asarray(body_dofnum, np.int32), M_rowadr=rowadr, M_rownnz=rownnz, M_colind=colind,
        M_hinit_i=np.repeat(np.arange(nv), rownnz).astype(np.int32), neq=0, nflex=0, ntendon=0,
        nxn_geom_pair_filtered=np.zeros((0, 2), np.int32), geom_bodyid=np.zeros(0, np.int32),
        # what the fused Newton's eligibility test reads: Newton solver (mjSOL_NEWTON = 2), pyramidal cone
        # (mjCONE_PYRAMIDAL = 0), implicitfast integrator (3), dense Jacobian, 32-lane line search
        opt=SimpleNamespace(solver=2, cone=0, integrator=3, iterations=100), is_sparse=False,
        block_dim=SimpleNamespace(linesearch_iterative=32),
    )  # fmt: skip


def contact_model():
    """The structure of the reference's sparse-Hessian test model
    (tests/test_mjw_sparse_hessian.py:14-53): torso (6 dofs), two legs (ball, hinge, two
    hinges on the foot), two arms (hinge, two hinges), two free boxes; nv = 36.  Returns the
    model namespace and body ids by name."""
    parent = [-1, 0, 1, 2, 3, 4]
    joints = [[0, 1, 2, 3, 4, 5]]
    names = ["torso"]

    def add(body_name, ndof, parent_dof):
        first = len(parent)
        parent.extend([parent_dof] + list(range(first, first + ndof - 1)))
        joints.append(list(range(first, first + ndof)))
        names.append(body_name)
        return first + ndof - 1

    for s in "LR":
        last = add("thigh" + s, 3, 5)
        last = add("shin" + s, 1, last)
        add("foot" + s, 2, last)
    for s in "LR":
        last = add("arm" + s, 1, 5)
        add("fore" + s, 2, last)
    for s in "AB":
        first = len(parent)
        parent.extend([-1] + list(range(first, first + 5)))
        joints.append(list(range(first, first + 6)))
        names.append("box" + s)
    m = model_from_parents(parent, joints)
    return m, {n: i + 1 for i, n in enumerate(names)}


# ------------------------------------------------------------------ muscle rig with path geometry


def make_implicit_case(nworld: int, timestep: float = 0.004, seed: int = 3):
    """A model and data for the implicit-fast integrator matrix: the SNU-like tree with a second,
    free-floating body of six dofs appended, 40 affine actuators over one to three dofs of a chain,
    12 damped tendons.  Returns (m, d, (rowadr, rownnz, colind), dofs of the first tree); arrays are NumPy."""
    rng = np.random.default_rng(seed)
    parents = list(snu_parents())
    nv0 = len(parents)
    parents += [-1, nv0, nv0 + 1, nv0 + 2, nv0 + 3, nv0 + 4]  # a free body: rows reset to M
    nv = len(parents)
    m = model_from_parents(parents)
    rowadr, rownnz, colind = csr_from_parents(parents)
    # bodies: model_from_parents makes one body per dof; body k + 1 holds dof k
    m.body_freeadr = np.array([nv0 + 1], np.int32)
    m.body_dofadr[nv0 + 1] = nv0
    m.dof_damping = rng.uniform(0.0, 2.0, nv).astype(np.float32)
    m.dof_damping[::7] = 0.0
    m.opt.timestep = timestep
    m.opt.disableflags = 0
    chain = chain_mask(parents)

    def rows(n, kmax):
        nnz, adr, col = [], [], []
        for _ in range(n):
            leaf = int(rng.integers(6, nv))
            support = np.flatnonzero(chain[leaf])
            k = int(rng.integers(1, kmax + 1))
            dofs = np.sort(rng.choice(support, min(k, len(support)), replace=False))
            adr.append(len(col))
            nnz.append(len(dofs))
            col += dofs.tolist()
        return np.array(nnz, np.int32), np.array(adr, np.int32), np.array(col, np.int32)

    nu, nt = 40, 12
    m.nactuator = nu
    m.actuator_gaintype = rng.integers(0, 2, nu).astype(np.int32)
    m.actuator_biastype = rng.integers(0, 2, nu).astype(np.int32)
    m.actuator_gainprm = rng.normal(size=(nu, 10)).astype(np.float32)
    m.actuator_biasprm = rng.normal(size=(nu, 10)).astype(np.float32) * 5
    m.actuator_forcelimited = (rng.random(nu) < 0.3).astype(np.uint8)
    m.actuator_forcerange = np.stack([-np.ones(nu), np.ones(nu)], 1).astype(np.float32)
    m.ntendon = nt
    m.ten_J_rownnz, m.ten_J_rowadr, m.ten_J_colind = rows(nt, 4)
    m.tendon_damping = rng.uniform(0.0, 3.0, nt).astype(np.float32)
    mom = rows(nu, 3)
    b = make_batch(Shape("snu+free", tuple(parents), 8, nworld, (0.5, 8.0), 0.02, (-3.0, 3.0), 0.6, 1, seed), nworld)
    d = SimpleNamespace(
        nworld=nworld, M=b.M, moment_rownnz=mom[0], moment_rowadr=mom[1], moment_colind=mom[2],
        actuator_moment=rng.normal(scale=0.3, size=(nworld, len(mom[2]))).astype(np.float32),
        ten_J=rng.normal(scale=0.5, size=(nworld, len(m.ten_J_colind))).astype(np.float32),
        ctrl=rng.uniform(-1, 1, (nworld, nu)).astype(np.float32),
        actuator_force=rng.uniform(-1.5, 1.5, (nworld, nu)).astype(np.float32),
        efc=SimpleNamespace(Ma=b.grad),
    )  # fmt: skip
    return m, d, (rowadr, rownnz, colind), nv0


@dataclass
class MuscleRig:
    """Waypoint muscles routed over the SNU-like tree: the arrays a MuscleDynamicsLayer is
    built from plus the model dimensions."""

    topology: object  # muscle.muscle_dynamics.MuscleTopology
    body_count: int
    full_torque_dim: int
    torque_dim: int
    muscle_count: int

    def dims(self) -> dict:
        return dict(body_count=self.body_count, full_torque_dim=self.full_torque_dim, torque_dim=self.torque_dim,
                    muscle_count=self.muscle_count)  # fmt: skip


def make_muscle_rig(nmuscle: int = 284, seed: int = 1003) -> MuscleRig:
    """Each muscle runs over 1-3 adjacent joints of one chain with one or two waypoints on
    every body it passes (local offsets ~U(-0.08, 0.08) m); the applied segments are the
    ones whose ends sit on different bodies.  f0 ~ U[100, 3000] N, l_m0 ~ U[0.4, 0.9],
    l_t0 ~ U[0.1, 0.5], pennation ~ U[0, 0.4] rad, rest length = 0.5 m."""
    from .muscle.muscle_dynamics import MuscleTopology

    rng = np.random.default_rng([seed, 91])
    chains = snu_joint_chains()
    parent = snu_parents()
    joints = [[0, 1, 2, 3, 4, 5]]
    for chain in chains:
        for j in chain:
            if j not in joints:
                joints.append(j)
    joints.sort(key=lambda j: j[0])
    model = model_from_parents(parent, joints)
    body_of_dof = {d: b for b, dofs in enumerate(joints, start=1) for d in dofs}
    nbody = len(joints) + 1
    wp_body, wp_local, wp_muscle = [], [], []
    for m in range(nmuscle):
        chain = chains[int(rng.integers(len(chains)))]
        span = int(rng.integers(1, 4))
        first = int(rng.integers(0, len(chain) - span + 1))
        bodies = [int(model.body_parentid[body_of_dof[chain[first][0]]])]
        bodies += [body_of_dof[j[0]] for j in chain[first : first + span]]
        for b in bodies:
            for _ in range(int(rng.integers(1, 3))):
                wp_body.append(b)
                wp_local.append(rng.uniform(-0.08, 0.08, 3))
                wp_muscle.append(m)
    wp_body, wp_muscle = np.asarray(wp_body), np.asarray(wp_muscle)
    start = np.flatnonzero(wp_muscle[:-1] == wp_muscle[1:])
    crossing = start[wp_body[start] != wp_body[start + 1]]
    nv = len(parent)
    dof_bodyid = np.asarray([body_of_dof[d] for d in range(nv)])
    dof_bodyid[:6] = 0  # the free root's dofs move every body, as world-body dofs do
    topo = MuscleTopology(
        muscle_params=np.stack(
            [rng.uniform(100, 3000, nmuscle), rng.uniform(0.4, 0.9, nmuscle), rng.uniform(0.1, 0.5, nmuscle),
             rng.uniform(0, 0.4, nmuscle), np.ones(nmuscle)], axis=1).astype(np.float32),
        muscle_rest_length=np.full(nmuscle, 0.5, np.float32),
        muscle_waypoints_local=np.asarray(wp_local, np.float32),
        muscle_waypoint_body=wp_body,
        all_segment_muscle_idx=wp_muscle[start],
        all_segment_start_idx=start,
        apply_segment_muscle_idx=wp_muscle[crossing],
        apply_segment_start_idx=crossing,
        apply_segment_end_idx=crossing + 1,
        apply_segment_body_start_idx=wp_body[crossing],
        apply_segment_body_end_idx=wp_body[crossing + 1],
        body_parentid=model.body_parentid,
        body_rootid=np.asarray([0] + [1] * (nbody - 1)),
        dof_bodyid=dof_bodyid,
    )  # fmt: skip
    return MuscleRig(topo, nbody, nv, nv - 6, nmuscle)


def make_muscle_context(rig: MuscleRig, nworld: int, seed: int = 1003) -> np.ndarray:
    """raw_context (nworld, 13 nbody + 6 nv) = xpos | xquat | xipos | subtree_com | cdof with
    body positions ~N(0, 0.3) m, quaternions ~N(0, 1) (unnormalised on purpose), subtree
    centres ~N(0, 0.2), cdof ~N(0, 1)."""
    nb, nv = rig.body_count, rig.full_torque_dim
    out = np.empty((nworld, 13 * nb + 6 * nv), np.float32)
    for b0 in range(0, nworld, BLOCK):
        r = np.random.default_rng([seed, 92, b0 // BLOCK])
        n = min(BLOCK, nworld - b0)
        parts = [r.normal(0, 0.3, (BLOCK, 3 * nb)), r.normal(0, 1, (BLOCK, 4 * nb)), r.normal(0, 0.3, (BLOCK, 3 * nb)),
                 r.normal(0, 0.2, (BLOCK, 3 * nb)), r.normal(0, 1, (BLOCK, 6 * nv))]  # fmt: skip
        out[b0 : b0 + n] = np.concatenate(parts, axis=1)[:n]
    return out
