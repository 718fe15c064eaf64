"""CPU oracle for the batched assemble + L'DL + solve path (TEST INFRASTRUCTURE ONLY).

Nothing under this package is part of the shipped product.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and there only as the checker.  The product path
(``instantmimic_amd``) never falls back to it.

Contents

* ``planner``     integer restatement of the reference planner
                  (src/instantmimic/utils/mjw_kernels/tree_ldl.py:66-193) and of the
                  static-pattern symbolic factor
                  (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:192-345).
* ``cpu_ref.c``   fp32 C restatement of the numeric statements (explicit ``fmaf``,
                  compiled with ``-ffp-contract=off``), OpenMP over worlds.
* ``ref``         ctypes front end of ``cpu_ref.c`` plus fp64 dense NumPy solves.

Pinning status of each function is listed in the header of ``ref.py``.
"""
