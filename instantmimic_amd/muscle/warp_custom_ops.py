"""Opaque torch.library operators of the muscle activation-to-torque path.

Same operator names, schemas, registry functions and autograd wiring as the reference's
``instantmimic.muscle.warp_custom_ops`` (src/instantmimic/muscle/warp_custom_ops.py:41-190),
so a compiled loss that calls ``torch.ops.instantmimic_muscle.torque_forward`` needs no
change; the module keeps that file's name for the same reason although nothing here uses
Warp.  The operator bodies launch ``libimhip`` kernels on the current torch stream: there
is no stream registry to maintain, and the launches are capturable as they are.

Operators are generic over layers: ``layer_key`` resolves the owning layer through a weak
registry, tensors are the whole data interface.
"""

from __future__ import annotations

import itertools
import weakref
from typing import Any

import torch

_LAYERS: dict[int, weakref.ReferenceType[Any]] = {}
_LAYER_OWNERS: dict[int, int] = {}
_LAYER_KEYS = itertools.count(1)


def register_warp_op_layer(layer: Any) -> int:
    """Give ``layer`` a fresh dispatcher handle (warp_custom_ops.py:46-58)."""
    key = next(_LAYER_KEYS)
    layer._warp_op_key = key
    _LAYERS[key] = weakref.ref(layer)
    _LAYER_OWNERS[key] = id(layer)
    return int(key)


def warp_op_key(layer: Any) -> int:
    """The layer's handle; a copy that carries another instance's key gets its own
    (warp_custom_ops.py:61-68)."""
    key = getattr(layer, "_warp_op_key", None)
    if key is not None and _LAYER_OWNERS.get(int(key)) == id(layer):
        return int(key)
    return register_warp_op_layer(layer)


def _layer_for(key: int) -> Any:
    reference = _LAYERS.get(int(key))
    layer = None if reference is None else reference()
    if layer is None:
        raise RuntimeError(
            f"Warp custom-op layer key {key} is not registered; the muscle layer "
            "was released while a compiled loss still referenced it."
        )
    return layer


@torch.library.custom_op("instantmimic_muscle::torque_forward", mutates_args=())
def muscle_torque_forward(
    activation: torch.Tensor,
    raw_context: torch.Tensor,
    layer_key: int,
    include_passive_force: bool,
) -> torch.Tensor:
    """Differentiable activation-to-torque projection of one layer."""
    layer = _layer_for(layer_key)
    mean, _, _ = layer._warp_muscle_dynamics_from_activation_forward(
        activation=activation,
        raw_context=raw_context,
        include_passive_force=include_passive_force,
    )
    return mean


@muscle_torque_forward.register_fake
def _muscle_torque_forward_fake(activation, raw_context, layer_key, include_passive_force):
    layer = _layer_for(layer_key)
    return torch.empty((activation.shape[0], layer.torque_dim), dtype=torch.float32, device=activation.device)


@torch.library.custom_op("instantmimic_muscle::torque_backward", mutates_args=())
def muscle_torque_backward(
    raw_context: torch.Tensor,
    grad_output: torch.Tensor,
    layer_key: int,
) -> torch.Tensor:
    """Activation gradient of muscle_torque_forward; geometry is rebuilt from the context,
    so no view of another forward's scratch is held."""
    layer = _layer_for(layer_key)
    return layer._warp_muscle_dynamics_from_activation_backward(raw_context=raw_context, grad_output=grad_output)


@muscle_torque_backward.register_fake
def _muscle_torque_backward_fake(raw_context, grad_output, layer_key):
    layer = _layer_for(layer_key)
    return torch.empty((raw_context.shape[0], layer.muscle_count), dtype=torch.float32, device=raw_context.device)


def _torque_forward_setup_context(ctx: Any, inputs: tuple[Any, ...], output: torch.Tensor) -> None:
    ctx.save_for_backward(inputs[1])
    ctx.layer_key = int(inputs[2])
    # the registry is weak; the node keeps the layer alive until its backward has run
    ctx.layer = _layer_for(ctx.layer_key)


def _torque_forward_backward(ctx: Any, grad_output: torch.Tensor):
    (raw_context,) = ctx.saved_tensors
    return muscle_torque_backward(raw_context, grad_output, ctx.layer_key), None, None, None


muscle_torque_forward.register_autograd(_torque_forward_backward, setup_context=_torque_forward_setup_context)


@torch.library.custom_op("instantmimic_muscle::torque_cached_lbs_forward", mutates_args=())
def muscle_torque_cached_lbs_forward(
    activation: torch.Tensor,
    raw_context: torch.Tensor,
    unit_force_magnitude: torch.Tensor,
    passive_force_magnitude: torch.Tensor,
    layer_key: int,
    include_passive_force: bool,
) -> torch.Tensor:
    """Projection whose per-muscle forces were precomputed outside this call
    (warp_custom_ops.py:187-209)."""
    layer = _layer_for(layer_key)
    return layer._warp_muscle_dynamics_from_activation_forward_cached_lbs_force(
        activation=activation,
        raw_context=raw_context,
        unit_force_magnitude=unit_force_magnitude,
        passive_force_magnitude=passive_force_magnitude,
        include_passive_force=include_passive_force,
    )


@muscle_torque_cached_lbs_forward.register_fake
def _muscle_torque_cached_lbs_forward_fake(
    activation, raw_context, unit_force_magnitude, passive_force_magnitude, layer_key, include_passive_force
):
    layer = _layer_for(layer_key)
    return torch.empty((activation.shape[0], layer.torque_dim), dtype=torch.float32, device=activation.device)


@torch.library.custom_op("instantmimic_muscle::torque_cached_lbs_backward", mutates_args=())
def muscle_torque_cached_lbs_backward(
    raw_context: torch.Tensor,
    unit_force_magnitude: torch.Tensor,
    grad_output: torch.Tensor,
    layer_key: int,
) -> torch.Tensor:
    """Activation gradient of muscle_torque_cached_lbs_forward (warp_custom_ops.py:230-246)."""
    layer = _layer_for(layer_key)
    return layer._warp_muscle_dynamics_from_activation_backward(
        raw_context=raw_context, grad_output=grad_output, unit_force_magnitude=unit_force_magnitude
    )


@muscle_torque_cached_lbs_backward.register_fake
def _muscle_torque_cached_lbs_backward_fake(raw_context, unit_force_magnitude, grad_output, layer_key):
    layer = _layer_for(layer_key)
    return torch.empty((raw_context.shape[0], layer.muscle_count), dtype=torch.float32, device=raw_context.device)


def _cached_lbs_forward_setup_context(ctx: Any, inputs: tuple[Any, ...], output: torch.Tensor) -> None:
    ctx.save_for_backward(inputs[1], inputs[2])
    ctx.layer_key = int(inputs[4])
    ctx.layer = _layer_for(ctx.layer_key)


def _cached_lbs_forward_backward(ctx: Any, grad_output: torch.Tensor):
    raw_context, unit_force_magnitude = ctx.saved_tensors
    grad = muscle_torque_cached_lbs_backward(raw_context, unit_force_magnitude, grad_output, ctx.layer_key)
    return grad, None, None, None, None, None


muscle_torque_cached_lbs_forward.register_autograd(
    _cached_lbs_forward_backward, setup_context=_cached_lbs_forward_setup_context
)


@torch.library.custom_op("instantmimic_muscle::torque_bounds", mutates_args=())
def muscle_torque_bounds(
    raw_context: torch.Tensor,
    layer_key: int,
    select_active: bool,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Feasible torque box at the current geometry; data, not differentiable outputs.  The
    results are freshly allocated, so nothing a later call does can rewrite them
    (warp_custom_ops.py:285-303)."""
    layer = _layer_for(layer_key)
    lower, upper = layer._compute_activation_torque_bounds_warp(raw_context, select_active=select_active)
    return lower.contiguous(), upper.contiguous()


@muscle_torque_bounds.register_fake
def _muscle_torque_bounds_fake(raw_context, layer_key, select_active):
    layer = _layer_for(layer_key)
    width = layer.active_output_dim if select_active else layer.torque_dim
    lower = torch.empty((raw_context.shape[0], width), dtype=torch.float32, device=raw_context.device)
    return lower, torch.empty_like(lower)


__all__ = [
    "muscle_torque_backward",
    "muscle_torque_bounds",
    "muscle_torque_cached_lbs_backward",
    "muscle_torque_cached_lbs_forward",
    "muscle_torque_forward",
    "register_warp_op_layer",
    "warp_op_key",
]
