"""Writes the committed golden fixtures from the CPU oracle.

    python tests/golden/make_fixtures.py

* tree_plans.json   integer plans of the benchmark trees and of the reference's
                    test trees (spans per group count, chosen plan, elimination order).
                    The spans and chosen plans were checked by hand against the planner rule
                    (src/instantmimic/utils/mjw_kernels/tree_ldl.py:66-193).
* tree_small.npz    4 worlds of the ant shape: inputs, assembled H and solve result of
                    the oracle (fp32), for comparing the HIP path against stored vectors.
"""

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from instantmimic_amd import synth  # noqa: E402
from oracle import planner as P  # noqa: E402
from oracle import ref as R  # noqa: E402


def main():
    trees = {name: list(s.parents) for name, s in synth.SHAPES.items()}
    trees["limbs4x6"] = synth.limbs_parents()
    trees["chain30"] = synth.chain_parents()
    trees["branched"] = synth.branched_parents()
    plans = {}
    for name, parent in trees.items():
        st = P.csr_from_parents(parent)
        best = P.best_tree_ldl_plan(*st)
        plans[name] = {
            "parents": parent,
            "nM": len(st[2]),
            "spans": [P.plan_tree_ldl(*st, g).span for g in (1, 2, 3, 4)],
            "groups": [list(g) for g in best.groups],
            "trunk": list(best.trunk),
            "span": best.span,
            "dense_cost": best.dense_cost,
            "shared_bytes": P.shared_bytes(st[0], st[1], len(best.groups), best.trunk),
            "eligible": bool(P.tree_ldl_beats_dense(best)),
            "elimination_order": P.elimination_order(best),
        }
    with open(os.path.join(HERE, "tree_plans.json"), "w") as f:
        json.dump(plans, f, indent=1)
    b = synth.make_batch("ant", 4)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    x, H = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[0], b.nefc, b.grad, want_h=True)
    np.savez_compressed(
        os.path.join(HERE, "tree_small.npz"), M=b.M, J=b.J, D=b.D, state=b.state[0], nefc=b.nefc, grad=b.grad, H=H, x=x
    )


if __name__ == "__main__":
    main()
