"""EMA Gram preconditioners ``L <- beta L + (1-beta) G G^T`` and ``R <- beta R + (1-beta) G^T G``.

Same entry points as the reference (src/soap_tp/ops/preconditioners.py:678-777).  There the
update is a Python loop over block tiles (``mm`` + ``reduce`` + ``lerp_`` per tile, :339-406
and :523-623); here it is one launch of the MFMA kernel that walks the tiles on or below the
diagonal and applies the ``lerp`` in its epilogue.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ._common import native_call, require_device_tensor, stream_of
from ._utils import current_world, validate_2d_block_cyclic_buffer


def _update(
    side: int,
    name: str,
    G_local: Tensor,
    preconditioner: Tensor,
    beta: float,
    block_size: int,
    process_grid_shape: tuple[int, int],
    shard_dim: int,
    mirror: bool,
) -> Tensor:
    if G_local.ndim != 2:
        raise ValueError(f"G_local must be 2D, got {G_local.ndim}D.")
    if shard_dim not in (0, 1):
        raise ValueError(f"shard_dim must be 0 or 1, got {shard_dim}.")
    if not 0.0 <= beta <= 1.0:
        raise ValueError(f"beta must be in [0, 1], got {beta}.")
    rank, _ = current_world(process_grid_shape)
    if preconditioner.dtype != torch.float32:
        raise ValueError(
            f"{name} must use float32 for ELPA and SLATE, got {preconditioner.dtype}."
        )
    if preconditioner.device != G_local.device:
        raise ValueError(f"{name} is on {preconditioner.device}, expected {G_local.device}.")
    rows, columns = G_local.shape
    size = rows if side == 0 else columns
    validate_2d_block_cyclic_buffer(
        "matrix", preconditioner, (size, size), block_size, process_grid_shape, rank
    )
    require_device_tensor("G_local", G_local)
    gradient = G_local.detach().to(dtype=torch.float32)
    if gradient.stride(1) == 1 and gradient.stride(0) >= max(1, columns):
        row_major, ldg = 1, gradient.stride(0)
    elif gradient.stride(0) == 1 and gradient.stride(1) >= max(1, rows):
        row_major, ldg = 0, gradient.stride(1)
    else:
        gradient = gradient.contiguous()
        row_major, ldg = 1, max(1, columns)
    if size == 0:
        return preconditioner
    with torch.cuda.device(gradient.device):
        native_call(
            "soapmi_gram_ema_f32",
            gradient.data_ptr(), rows, columns, ldg, row_major, side,
            preconditioner.data_ptr(), preconditioner.stride(1), float(beta), 1 if mirror else 0,
            stream_of(gradient),
        )
    return preconditioner


@torch.no_grad()
def update_left_preconditioner_2d_block_cyclic_(
    G_local: Tensor,
    left_preconditioner: Tensor,
    beta: float,
    block_size: int,
    process_grid_shape: tuple[int, int],
    *,
    shard_dim: Literal[0, 1],
    mirror: bool = True,
) -> Tensor:
    """Update packed ``L = beta * L + (1 - beta) * G @ G.T`` in place.

    ``mirror=False`` (an extension) writes only the lower triangle; the reference always keeps
    both triangles (tile mode "full", src/soap_tp/ops/preconditioners.py:709-716).
    """
    return _update(0, "left_preconditioner", G_local, left_preconditioner, beta, block_size,
                   process_grid_shape, shard_dim, mirror)


@torch.no_grad()
def update_right_preconditioner_2d_block_cyclic_(
    G_local: Tensor,
    right_preconditioner: Tensor,
    beta: float,
    block_size: int,
    process_grid_shape: tuple[int, int],
    *,
    shard_dim: Literal[0, 1],
    mirror: bool = True,
) -> Tensor:
    """Update packed ``R = beta * R + (1 - beta) * G.T @ G`` in place."""
    return _update(1, "right_preconditioner", G_local, right_preconditioner, beta, block_size,
                   process_grid_shape, shard_dim, mirror)
