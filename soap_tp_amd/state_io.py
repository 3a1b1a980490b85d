"""Saving and restoring a ``soap_step`` state dictionary.

The state holds eight strided column-major matrices (``zeros((cols, ld)).T`` views,
src/soap_tp/ops/_utils.py:159-189) and the integer step (src/soap_tp/soap.py:166-175).  Serialisers
that only keep contiguous data (safetensors, ``tensor.contiguous()`` round trips, dtype casts) lose
that layout, and ``soap_step`` rejects buffers that are not column-major.  ``pack_state`` therefore
stores every buffer as the contiguous ``(cols, rows)`` transpose together with its logical shape (the
Gram matrices symmetrised from their lower triangle, the one ``soap_step`` keeps current), and
``unpack_state`` rebuilds the exact layout (``stride == (1, max(1, rows))``) on the target device and
checks shapes, dtype and mutual consistency before the state is used again.  The reference has no
such helper; its .gitignore:18-20 only anticipates ``.pt`` checkpoints.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, MutableMapping, Optional, Tuple

import torch
from torch import Tensor

STATE_BUFFERS = (
    "left_preconditioner",
    "right_preconditioner",
    "left_basis",
    "right_basis",
    "left_work",
    "right_work",
    "momentum",
    "variance",
)
FORMAT_VERSION = 1

__all__ = ["pack_state", "unpack_state", "save_state", "load_state", "validate_state"]


def _expected_shapes(rows: int, columns: int) -> Dict[str, Tuple[int, int]]:
    square = {"left": (rows, rows), "right": (columns, columns)}
    return {name: square.get(name.split("_", 1)[0], (rows, columns)) for name in STATE_BUFFERS}


def validate_state(state: Mapping[str, Any], global_shape: Optional[Tuple[int, int]] = None) -> Tuple[int, int]:
    """Check an initialised state: all buffers present, fp32, column-major with ``ld >= rows``, shapes
    consistent with one ``(rows, columns)`` parameter (and with ``global_shape`` when given), a
    non-negative integer step.  Returns ``(rows, columns)``; raises ``ValueError`` otherwise."""
    missing = [name for name in STATE_BUFFERS + ("step",) if name not in state]
    if missing:
        raise ValueError(f"state is missing {missing}.")
    momentum = state["momentum"]
    if not isinstance(momentum, Tensor) or momentum.ndim != 2:
        raise ValueError("state['momentum'] must be a 2D tensor.")
    rows, columns = momentum.shape
    if global_shape is not None and tuple(global_shape) != (rows, columns):
        raise ValueError(f"state is for a {(rows, columns)} parameter, expected {tuple(global_shape)}.")
    for name, shape in _expected_shapes(rows, columns).items():
        tensor = state[name]
        if not isinstance(tensor, Tensor):
            raise ValueError(f"state[{name!r}] must be a tensor.")
        if tuple(tensor.shape) != shape:
            raise ValueError(f"state[{name!r}] has shape {tuple(tensor.shape)}, expected {shape}.")
        if tensor.dtype != torch.float32:
            raise ValueError(f"state[{name!r}] must use float32, got {tensor.dtype}.")
        if tensor.stride(0) != 1 or tensor.stride(1) < max(1, shape[0]):
            raise ValueError(f"state[{name!r}] must be column-major with a leading dimension of at least "
                             f"{max(1, shape[0])}, got strides {tuple(tensor.stride())}.")
        if tensor.device != momentum.device:
            raise ValueError("all state buffers must live on one device.")
    step = state["step"]
    if isinstance(step, bool) or not isinstance(step, int) or step < 0:
        raise ValueError(f"state['step'] must be a non-negative int, got {step!r}.")
    status = state.get("status")
    if isinstance(status, Tensor) and int(status[0]) != 0:
        raise ValueError("a factorisation of this state failed on the device (state['status'] is raised): its "
                         "bases are NaN-poisoned.")
    return rows, columns


def pack_state(state: Mapping[str, Any]) -> Dict[str, Any]:
    """Layout-free copy of a state: contiguous ``(cols, rows)`` transposes, shapes, step.  An empty
    (not yet initialised) state packs to a marker and unpacks to ``{}``."""
    if "left_basis" not in state:
        return {"format_version": FORMAT_VERSION, "initialised": False}
    rows, columns = validate_state(state)
    packed: Dict[str, Any] = {"format_version": FORMAT_VERSION, "initialised": True, "rows": rows,
                              "columns": columns, "step": int(state["step"])}
    for name in STATE_BUFFERS:
        buffer = state[name].detach()
        if name.endswith("_preconditioner"):
            # soap_step keeps only the lower triangle of a Gram matrix up to date between refreshes
            # (preconditioner_storage="lower"); a saved state has both triangles valid, as the
            # reference's state contract asks (src/soap_tp/ops/factorizations.py:378)
            packed[name] = (torch.tril(buffer) + torch.tril(buffer, -1).T).contiguous()
        else:
            packed[name] = buffer.T.contiguous()
    return packed


def unpack_state(packed: Mapping[str, Any], device=None) -> Dict[str, Any]:
    """Inverse of ``pack_state``: rebuilds the column-major buffers (``ld = max(1, rows)``) on
    ``device`` (default: where the packed tensors are) and validates the result."""
    version = packed.get("format_version")
    if version != FORMAT_VERSION:
        raise ValueError(f"unsupported SOAP state format version {version!r}.")
    if not packed.get("initialised", False):
        return {}
    rows, columns = int(packed["rows"]), int(packed["columns"])
    state: Dict[str, Any] = {}
    for name, shape in _expected_shapes(rows, columns).items():
        if name not in packed:
            raise ValueError(f"packed state is missing {name!r}.")
        stored = packed[name]
        if tuple(stored.shape) != (shape[1], shape[0]):
            raise ValueError(f"packed {name!r} has shape {tuple(stored.shape)}, expected {(shape[1], shape[0])}.")
        if stored.dtype != torch.float32:
            raise ValueError(f"packed {name!r} must use float32, got {stored.dtype}.")
        target = device if device is not None else stored.device
        buffer = torch.empty((shape[1], max(1, shape[0])), dtype=torch.float32, device=target)
        buffer[:, : shape[0]].copy_(stored)
        state[name] = buffer.T[: shape[0], :]
    state["step"] = int(packed["step"])
    validate_state(state, (rows, columns))
    return state


def save_state(state: Mapping[str, Any], path) -> None:
    """``torch.save`` of the packed state (tensors, ints and bools only, so it loads with
    ``weights_only=True``)."""
    packed = pack_state(state)
    torch.save({key: (value.cpu() if isinstance(value, Tensor) else value) for key, value in packed.items()}, path)


def load_state(path, device=None, into: Optional[MutableMapping[str, Any]] = None) -> Dict[str, Any]:
    """Load a file written by ``save_state`` (nothing in the file is executed) and rebuild the state
    on ``device``; with ``into`` the given dictionary is cleared and filled instead of a new one."""
    packed = torch.load(path, map_location="cpu", weights_only=True)
    state = unpack_state(packed, device=device)
    if into is not None:
        into.clear()
        into.update(state)
        return into  # type: ignore[return-value]
    return state
