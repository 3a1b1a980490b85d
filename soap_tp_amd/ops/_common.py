"""Shared argument checks and launch helpers for the ops."""
from __future__ import annotations

from typing import Any, Optional, Tuple

import torch
from torch import Tensor

from .. import _native
from ..binding import default_binding
from ._utils import validate_2d_block_cyclic_buffer


def stream_of(tensor: Tensor) -> int:
    return torch.cuda.current_stream(tensor.device).cuda_stream


def scratch(nbytes: int, device) -> Tensor:
    """Workspace from torch's caching allocator (stream-ordered, so no synchronisation)."""
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def raise_on_device_error(device) -> None:
    """Raise if a factorisation enqueued earlier on ``device`` has since failed there.

    The persistent panel kernels of the QR and of the tridiagonalisation bound their waits for
    other workgroups' messages; a kernel that gives up NaN-poisons its output and raises a word of
    pinned host memory, which is read here without synchronising.  The reference's bindings throw
    from inside the call (src/soap_tp/csrc/elpa_bindings.cpp:77-91); here the kernels are still
    queued when the call returns, so the failure surfaces at the next call on that device."""
    with torch.cuda.device(device):
        if _native.device_error_flag(clear=True):
            raise RuntimeError(
                "a QR or eigensolver kernel enqueued earlier on this device gave up waiting for a message "
                "from another workgroup; the bases it produced are NaN-poisoned and the optimizer state "
                "that used them is invalid. Re-initialise the state (or restore a checkpoint)."
            )


def new_status_word() -> Tensor:
    """One zeroed int32 of pinned host memory: kernels raise it, the host reads it without synchronising."""
    return torch.zeros(1, dtype=torch.int32, pin_memory=True)


class reporting_to:
    """While active, factorisations enqueued by this thread report a failure on the device in the
    given pinned int32 tensor instead of the device-wide flag (``None``: no change)."""

    def __init__(self, status: Optional[Tensor]):
        if status is not None and (status.dtype != torch.int32 or status.numel() < 1 or not status.is_pinned()):
            raise ValueError("status must be a pinned int32 tensor with at least one element.")
        self.status = status

    def __enter__(self):
        if self.status is not None:
            _native.call("soapmi_set_status_word", self.status.data_ptr())
        return self

    def __exit__(self, *exc):
        if self.status is not None:
            _native.call("soapmi_set_status_word", 0)
        return False


def raise_on_state_error(state) -> None:
    """Raise if a factorisation of THIS state (its initialisation or one of its refreshes) failed on
    the device: the state's status word stays raised, so every later step of the state raises too,
    while other states on the device go on.  Reads pinned host memory, no synchronisation."""
    status = state.get("status") if hasattr(state, "get") else None
    if isinstance(status, Tensor) and int(status[0]) != 0:
        raise RuntimeError(
            "a QR or eigensolver kernel of this optimizer state gave up waiting for a message from another "
            "workgroup; its bases are NaN-poisoned and the state is invalid. Re-initialise the state (or "
            "restore a checkpoint)."
        )


def require_device_tensor(name: str, tensor: Tensor) -> None:
    """The kernels run on the GPU only; same rule and wording as the reference's backend check
    (src/soap_tp/ops/factorizations.py:33-48 with backend 'rocm')."""
    if tensor.device.type != "cuda":
        raise ValueError(
            f"native backend 'rocm' requires cuda buffers, got {tensor.device.type} for {name}."
        )


def validate_float_buffer(
    name: str,
    matrix: Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    rank: int,
) -> Tuple[int, int]:
    if matrix.dtype != torch.float32:
        raise ValueError(f"{name} must use float32, got {matrix.dtype}.")
    return validate_2d_block_cyclic_buffer(
        name, matrix, global_shape, block_size, process_grid_shape, rank
    )


def validated_binding(binding: Optional[Any], device: torch.device, rank: int, world_size: int) -> Any:
    """Resolve and check a binding object the way the reference does
    (src/soap_tp/ops/factorizations.py:85-101)."""
    if binding is None:
        binding = default_binding()
    mpi_rank, mpi_world_size = binding.mpi_world_rank_and_size()
    if (mpi_rank, mpi_world_size) != (rank, world_size):
        raise RuntimeError(
            "Torch and MPI worlds must have identical ranks and sizes; "
            f"got Torch {(rank, world_size)} and MPI {(mpi_rank, mpi_world_size)}."
        )
    backend = binding.compiled_gpu_backend()
    if backend not in {"none", "cuda", "rocm"}:
        raise RuntimeError(f"unsupported native backend {backend!r}.")
    expected_device = "cpu" if backend == "none" else "cuda"
    if device.type != expected_device:
        raise ValueError(
            f"native backend {backend!r} requires {expected_device} buffers, got {device.type}."
        )
    if backend == "cuda" and (torch.version.cuda is None or torch.version.hip is not None):
        raise RuntimeError("the CUDA binding requires a CUDA PyTorch build.")
    if backend == "rocm" and torch.version.hip is None:
        raise RuntimeError("the ROCm binding requires a ROCm PyTorch build.")
    return binding


native_call = _native.call
native_library = _native.library
