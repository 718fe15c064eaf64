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
