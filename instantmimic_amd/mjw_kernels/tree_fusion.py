"""Bottom-up accumulation of per-body quantities along the body tree on MI355X.

Drop-in for ``create_tree_reduction_scratch`` / ``accumulate`` of the reference module
``instantmimic.utils.mjw_kernels.tree_fusion``
(src/instantmimic/utils/mjw_kernels/tree_fusion.py:27-51, 137-167): same names and arguments,
arrays are torch tensors on the GPU.  One launch walks every level; a parent adds its children
in the order the level lists them, which is the reference's ``deterministic`` kernel (:82-113).
Its default kernel (:54-80) adds the same children with atomics, in no fixed order: the two
differ in the last bits only where a body has several children.

The reference's ``crb`` and ``rne`` wrap this step between upstream mujoco_warp kernels and
are not part of this module.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import numpy as np

from .. import _lib


@dataclass(frozen=True)
class TreeReductionScratch:
    """Same fields as the reference's scratch (tree_fusion.py:27-33) plus the parent table."""

    bodies: Any
    offsets: Any
    levels: int
    deterministic: bool = False
    cooperative: bool = True
    parent: Any = None
    nbody: int = 0


def _host(a) -> np.ndarray:
    if hasattr(a, "detach"):
        a = a.detach().cpu()
    if hasattr(a, "numpy"):
        a = a.numpy()
    return np.asarray(a)


def create_tree_reduction_scratch(m: Any, *, deterministic: bool = False, cooperative: bool = True, device="cuda"):
    """``m.body_tree`` (one array of body ids per depth) and ``m.body_parentid``; ``None`` for a
    model without a body tree, as the reference (tree_fusion.py:35-51)."""
    import torch

    if not getattr(m, "body_tree", None):
        return None
    levels = [_host(level).astype(np.int32).reshape(-1) for level in m.body_tree]
    parent = _host(m.body_parentid).astype(np.int32)
    bodies = np.concatenate(levels)
    if bodies.size and (bodies.min() < 0 or bodies.max() >= parent.size):
        raise ValueError("body_tree names a body outside body_parentid")
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(device)  # noqa: E731
    offsets = np.cumsum([0] + [len(level) for level in levels])
    return TreeReductionScratch(up(bodies), up(offsets), len(levels), deterministic, cooperative, up(parent), int(parent.size))


def accumulate(m: Any, d: Any, values, components: int, skip_root_parent: bool, scratch: TreeReductionScratch) -> None:
    """In place on ``values`` (nworld, nbody, components) float32: every body ends with the
    sum over its subtree (``skip_root_parent``: the children of body 0 are not added)."""
    import torch

    if scratch is None:
        raise ValueError("accumulate needs the scratch of create_tree_reduction_scratch (no per-level fallback here)")
    if values.dtype != torch.float32 or not values.is_cuda:
        raise TypeError("accumulate needs a float32 CUDA tensor")
    nworld = values.shape[0]
    flat = values.reshape(nworld, -1) if values.is_contiguous() else None
    if flat is None or flat.shape[1] != scratch.nbody * components:
        raise ValueError("values must be a contiguous (nworld, nbody, components) tensor")
    with torch.cuda.device(values.device):
        status = _lib.lib().im_tree_accumulate(
            scratch.parent.data_ptr(), scratch.bodies.data_ptr(), scratch.offsets.data_ptr(), scratch.levels,
            int(components), 1 if skip_root_parent else 0, values.data_ptr(), flat.stride(0) if nworld > 1 else flat.shape[1],
            scratch.nbody, int(nworld), int(torch.cuda.current_stream(values.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_tree_accumulate")


def subtree_com_accumulate(m: Any, d: Any, scratch: TreeReductionScratch) -> None:
    """``d.subtree_com`` (nworld, nbody, 3): mass-weighted positions summed up the tree
    (tree_fusion.py:170-181)."""
    accumulate(m, d, d.subtree_com, 3, False, scratch)
