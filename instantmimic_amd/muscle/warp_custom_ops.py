"""Opaque torch.library operators of the muscle activation-to-torque path.

The operator names and schemas (``instantmimic_muscle::torque_forward`` and its four
siblings), the Python callables that wrap them and the two registry functions are those of the
reference's ``instantmimic.muscle.warp_custom_ops``
(src/instantmimic/muscle/warp_custom_ops.py:41-319), so a compiled loss that calls
``torch.ops.instantmimic_muscle.torque_forward`` needs no change; the module keeps that file's
name for the same reason although nothing here uses Warp.  The operator bodies launch
``libimhip`` kernels on the current torch stream: there is no stream registry to maintain, and
the launches are capturable as they are.

An operator knows its layer through an integer handle only; tensors are the whole data
interface.  Handles resolve through a weak table, and an autograd node holds its layer strongly
until its backward has run.
"""

from __future__ import annotations

import itertools
import weakref
from typing import Any, Callable

import torch

NAMESPACE = "instantmimic_muscle"


class _Handles:
    """Weak table handle -> layer.  A handle belongs to the instance it was issued to: a shallow
    copy of a layer carries the original's ``_warp_op_key`` attribute but is another object and
    is issued a handle of its own the first time it asks."""

    def __init__(self) -> None:
        self._next = itertools.count(1)
        self._entries: dict[int, tuple[weakref.ReferenceType[Any], int]] = {}

    def issue(self, layer: Any) -> int:
        handle = next(self._next)
        self._entries[handle] = (weakref.ref(layer), id(layer))
        layer._warp_op_key = handle
        return handle

    def handle_of(self, layer: Any) -> int:
        handle = getattr(layer, "_warp_op_key", None)
        entry = self._entries.get(int(handle)) if handle is not None else None
        if entry is not None and entry[1] == id(layer):
            return int(handle)
        return self.issue(layer)

    def resolve(self, handle: int) -> Any:
        entry = self._entries.get(int(handle))
        layer = entry[0]() if entry is not None else None
        if layer is None:
            raise RuntimeError(
                f"Warp custom-op layer key {handle} is not registered; the muscle layer "
                "was released while a compiled loss still referenced it."
            )
        return layer


_HANDLES = _Handles()


def register_warp_op_layer(layer: Any) -> int:
    """A fresh dispatcher handle for ``layer`` (warp_custom_ops.py:46-58)."""
    return _HANDLES.issue(layer)


def warp_op_key(layer: Any) -> int:
    """The layer's handle, issued on first use (warp_custom_ops.py:61-68)."""
    return _HANDLES.handle_of(layer)


def _layer_for(key: int) -> Any:
    return _HANDLES.resolve(key)


def _operator(name: str, schema: str, body: Callable, shape: Callable):
    """Registers ``instantmimic_muscle::<name>`` with ``schema``; ``body(layer, *args)`` runs
    it, ``shape(layer, *args)`` gives the float32 output shapes for the fake kernel (a tuple of
    shapes for several outputs).  ``layer_key`` is looked for by position in the schema."""
    arg_names = [part.split()[-1] for part in schema[1 : schema.index(")")].split(",")]
    where = arg_names.index("layer_key")

    def run(*args):
        return body(_layer_for(args[where]), *args)

    def fake(*args):
        shapes = shape(_layer_for(args[where]), *args)
        device = args[0].device
        if isinstance(shapes[0], tuple):
            return tuple(torch.empty(s, dtype=torch.float32, device=device) for s in shapes)
        return torch.empty(shapes, dtype=torch.float32, device=device)

    op = torch.library.custom_op(f"{NAMESPACE}::{name}", run, mutates_args=(), schema=schema)
    op.register_fake(fake)
    return op


def _differentiable(forward_op, backward_op, saved: tuple[int, ...], key_at: int, nargs: int) -> None:
    """Autograd of ``forward_op`` with respect to its first argument: the inputs at ``saved`` are
    kept for ``backward_op(*saved, grad_output, layer_key)``."""

    def setup(ctx: Any, inputs: tuple[Any, ...], output: torch.Tensor) -> None:
        ctx.save_for_backward(*(inputs[i] for i in saved))
        ctx.layer_key = int(inputs[key_at])
        ctx.layer = _layer_for(ctx.layer_key)  # the table is weak: keep the layer until backward has run

    def backward(ctx: Any, grad_output: torch.Tensor):
        grad = backward_op(*ctx.saved_tensors, grad_output, ctx.layer_key)
        return (grad,) + (None,) * (nargs - 1)

    forward_op.register_autograd(backward, setup_context=setup)


# activation -> joint torque of one layer, geometry taken from raw_context (:97-127)
muscle_torque_forward = _operator(
    "torque_forward",
    "(Tensor activation, Tensor raw_context, SymInt layer_key, bool include_passive_force) -> Tensor",
    lambda layer, activation, raw_context, layer_key, include_passive_force: layer._warp_muscle_dynamics_from_activation_forward(
        activation=activation, raw_context=raw_context, include_passive_force=include_passive_force
    )[0],
    lambda layer, activation, *rest: (activation.shape[0], layer.torque_dim),
)

# its activation gradient; the geometry is rebuilt from the context, so no view of another
# forward's scratch is held (:130-160)
muscle_torque_backward = _operator(
    "torque_backward",
    "(Tensor raw_context, Tensor grad_output, SymInt layer_key) -> Tensor",
    lambda layer, raw_context, grad_output, layer_key: layer._warp_muscle_dynamics_from_activation_backward(
        raw_context=raw_context, grad_output=grad_output
    ),
    lambda layer, raw_context, *rest: (raw_context.shape[0], layer.muscle_count),
)
_differentiable(muscle_torque_forward, muscle_torque_backward, saved=(1,), key_at=2, nargs=4)

# the same pair with the per-muscle force magnitudes computed outside the call (:187-258)
muscle_torque_cached_lbs_forward = _operator(
    "torque_cached_lbs_forward",
    "(Tensor activation, Tensor raw_context, Tensor unit_force_magnitude, Tensor passive_force_magnitude, "
    "SymInt layer_key, bool include_passive_force) -> Tensor",
    lambda layer, activation, raw_context, unit, passive, layer_key, include_passive_force: (
        layer._warp_muscle_dynamics_from_activation_forward_cached_lbs_force(
            activation=activation, raw_context=raw_context, unit_force_magnitude=unit,
            passive_force_magnitude=passive, include_passive_force=include_passive_force,
        )  # fmt: skip
    ),
    lambda layer, activation, *rest: (activation.shape[0], layer.torque_dim),
)
muscle_torque_cached_lbs_backward = _operator(
    "torque_cached_lbs_backward",
    "(Tensor raw_context, Tensor unit_force_magnitude, Tensor grad_output, SymInt layer_key) -> Tensor",
    lambda layer, raw_context, unit, grad_output, layer_key: layer._warp_muscle_dynamics_from_activation_backward(
        raw_context=raw_context, grad_output=grad_output, unit_force_magnitude=unit
    ),
    lambda layer, raw_context, *rest: (raw_context.shape[0], layer.muscle_count),
)
_differentiable(muscle_torque_cached_lbs_forward, muscle_torque_cached_lbs_backward, saved=(1, 2), key_at=4, nargs=6)


def _bounds(layer, raw_context, layer_key, select_active):
    # data, not differentiable outputs; owned copies, so nothing a later call does rewrites them
    lower, upper = layer._compute_activation_torque_bounds_warp(raw_context, select_active=select_active)
    return lower.contiguous(), upper.contiguous()


def _bounds_shape(layer, raw_context, layer_key, select_active):
    shape = (raw_context.shape[0], layer.active_output_dim if select_active else layer.torque_dim)
    return shape, shape


# feasible torque box at the current geometry (:285-319)
muscle_torque_bounds = _operator(
    "torque_bounds", "(Tensor raw_context, SymInt layer_key, bool select_active) -> (Tensor, Tensor)", _bounds, _bounds_shape
)

__all__ = [
    "muscle_torque_backward",
    "muscle_torque_bounds",
    "muscle_torque_cached_lbs_backward",
    "muscle_torque_cached_lbs_forward",
    "muscle_torque_forward",
    "register_warp_op_layer",
    "warp_op_key",
]
