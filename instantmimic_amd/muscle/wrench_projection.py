"""Body wrenches onto joint torques with a reduction along the body tree, on MI355X.

Drop-in for the reference module ``instantmimic.muscle.wrench_projection``
(src/instantmimic/muscle/wrench_projection.py): :func:`tree_levels`,
:func:`build_wrench_projection_topology` and :func:`launch_project_body_wrench_to_torque`
keep their names and arguments.  Per world a workgroup keeps each body's force and its moment
about the root's subtree centre in LDS, folds the six components bottom-up and takes one dot
product per dof with its ``cdof`` row.  The reference folds siblings with atomics; here a
parent adds its children in level order, so a result is reproducible (and equal to the
reference's up to that order).  There is no per-dof masked-sum kernel here: a topology is
always built on a GPU, for any body count whose wrenches fit 64 KiB of LDS.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any

import numpy as np

from .. import _lib

MAX_BODY_COUNT = 64 * 1024 // (6 * 4)


@dataclass(frozen=True)
class WrenchProjectionTopology:
    """Same fields as the reference's (wrench_projection.py:145-155)."""

    dof_bodyid: Any
    body_parentid: Any
    level_bodies: Any
    level_offsets: Any
    levels: int
    body_count: int
    body_cap: int


def body_cap_for(body_count: int):
    """The reference returns its shared-memory tile (64 or 256 bodies) or None; here any
    count up to MAX_BODY_COUNT is its own cap."""
    return int(body_count) if 0 < int(body_count) <= MAX_BODY_COUNT else None


def tree_levels(body_parentid):
    """``(level_bodies, level_offsets, child_bodies, child_offsets)`` of a body tree whose
    parents precede their children: the bodies grouped by depth (ascending id inside a depth)
    with the depths' start offsets, and every body's children (ascending) behind one another
    with per-body offsets -- the four arrays of the reference's function of this name
    (wrench_projection.py:166-184)."""
    parent = [int(p) for p in np.asarray(body_parentid).reshape(-1)]
    nbody = len(parent)
    depth = [0] * nbody
    children: list[list[int]] = [[] for _ in range(nbody)]
    for body in range(1, nbody):
        if parent[body] >= body:
            raise ValueError("body_parentid must reference an earlier body")
        depth[body] = depth[parent[body]] + 1
        children[parent[body]].append(body)
    by_depth: list[list[int]] = [[] for _ in range(max(depth, default=0) + 1)]
    for body in range(nbody):
        by_depth[depth[body]].append(body)
    i32 = lambda values: np.asarray(values, dtype=np.int32)  # noqa: E731
    level_bodies = i32([body for level in by_depth for body in level])
    level_offsets = i32(np.cumsum([0] + [len(level) for level in by_depth]))
    child_bodies = i32([c for kids in children for c in kids])
    child_offsets = i32(np.cumsum([0] + [len(kids) for kids in children]))
    return level_bodies, level_offsets, child_bodies, child_offsets


def build_wrench_projection_topology(body_parentid, dof_bodyid, body_count: int, device):
    """Device tables of the projection, or None off the GPU or beyond the LDS limit."""
    import torch

    dev = torch.device(device)
    if dev.type != "cuda" or body_cap_for(body_count) is None:
        return None
    parents = body_parentid.detach().cpu().numpy().astype(np.int32)
    order, offsets, _, _ = tree_levels(parents)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)  # noqa: E731
    return WrenchProjectionTopology(
        dof_bodyid=up(dof_bodyid.detach().cpu().numpy()), body_parentid=up(parents), level_bodies=up(order),
        level_offsets=up(offsets), levels=int(offsets.shape[0] - 1), body_count=int(body_count), body_cap=int(body_count),
    )  # fmt: skip


def _rows(t, width: int, name: str):
    import torch

    if t.dtype != torch.float32 or not t.is_cuda:
        raise TypeError(f"{name} must be a float32 CUDA tensor")
    flat = t.reshape(t.shape[0], -1) if t.is_contiguous() else t
    if flat.dim() != 2 or flat.shape[1] < width or (flat.shape[1] > 1 and flat.stride(1) != 1):
        raise ValueError(f"{name} must hold {width} contiguous floats per world")
    return flat.data_ptr(), (flat.stride(0) if flat.shape[0] > 1 else flat.shape[1])


def launch_project_body_wrench_to_torque(
    topology: WrenchProjectionTopology | None, *, body_force, body_torque, xipos, subtree_com, cdof, body_rootid,
    dof_subtree_mask=None, mean, body_count: int, torque_dim: int, root_dof_count: int, output_dof_offset: int,
    batch_size: int, device=None,
) -> None:  # fmt: skip
    """Argument list of the reference's launcher (wrench_projection.py:222-284);
    ``dof_subtree_mask`` is what its per-dof kernel reads and is not used here."""
    import torch

    if topology is None:
        raise RuntimeError("no wrench projection topology: build_wrench_projection_topology returned None (no CPU path)")
    if body_rootid.dtype != torch.int32 or not body_rootid.is_cuda or body_rootid.numel() < body_count:
        raise TypeError("body_rootid must be an int32 CUDA tensor with one element per body")
    if int(body_count) != topology.body_count:
        raise ValueError("body_count differs from the topology's")
    nvfull = int(root_dof_count) + int(torque_dim)
    if topology.dof_bodyid.numel() < nvfull:
        raise ValueError("dof_bodyid is shorter than root_dof_count + torque_dim")
    w = _lib.BodyWrenches()
    for name, t, width in (("body_force", body_force, 3 * body_count), ("body_torque", body_torque, 3 * body_count),
                           ("xipos", xipos, 3 * body_count), ("subtree_com", subtree_com, 3 * body_count),
                           ("cdof", cdof, 6 * nvfull)):  # fmt: skip
        if t.shape[0] < batch_size:
            raise ValueError(f"{name} has fewer than batch_size rows")
        ptr, ld = _rows(t, width, name)
        setattr(w, name, ptr)
        setattr(w, "ld_" + name, ld)
    w.body_rootid = body_rootid.data_ptr()
    topo = _lib.WrenchTopology(
        topology.dof_bodyid.data_ptr(), topology.body_parentid.data_ptr(), topology.level_bodies.data_ptr(),
        topology.level_offsets.data_ptr(), topology.levels, topology.body_count,
    )  # fmt: skip
    if mean.dtype != torch.float32 or not mean.is_cuda or mean.dim() != 2 or (mean.shape[1] > 1 and mean.stride(1) != 1):
        raise TypeError("mean must be a float32 CUDA tensor with contiguous rows")
    if mean.shape[0] < batch_size or mean.shape[1] < output_dof_offset + torque_dim:
        raise ValueError("mean is smaller than (batch_size, output_dof_offset + torque_dim)")
    with torch.cuda.device(mean.device):
        status = _lib.lib().im_project_body_wrenches(
            C.byref(w), C.byref(topo), int(root_dof_count), int(torque_dim), int(output_dof_offset), mean.data_ptr(),
            mean.stride(0) if mean.shape[0] > 1 else mean.shape[1], int(batch_size),
            int(torch.cuda.current_stream(mean.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_project_body_wrenches")
