"""Layout helpers for packed buffers on a 1x1 process grid.

On one rank a 2-D block-cyclic buffer is simply a dense column-major matrix
(``block_cyclic_indices(size, bs, 0, 1) == range(size)`` in the reference,
src/soap_tp/ops/_utils.py:47-71), so ``block_size`` only has to be positive and the
local shape equals the global one.  The validators keep the reference's checks and
messages (src/soap_tp/ops/_utils.py:74-189) so callers see the same errors.
"""
from __future__ import annotations

from typing import Tuple

import torch
import torch.distributed as dist


def ceil_div(a: int, b: int) -> int:
    if b <= 0:
        raise ValueError(f"b must be positive, got {b}.")
    return -(-a // b)


def block_cyclic_indices(size: int, block_size: int, process: int, process_count: int) -> Tuple[int, ...]:
    """Global indices owned by ``process`` (src/soap_tp/ops/_utils.py:47-71)."""
    if size < 0:
        raise ValueError(f"size must be non-negative, got {size}.")
    if block_size <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}.")
    if process_count <= 0:
        raise ValueError(f"process_count must be positive, got {process_count}.")
    if not 0 <= process < process_count:
        raise ValueError(f"process must be in [0, {process_count}), got {process}.")
    if process_count == 1:
        return tuple(range(size))
    owned = []
    for start in range(process * block_size, size, process_count * block_size):
        owned.extend(range(start, min(start + block_size, size)))
    return tuple(owned)


def validate_process_grid(process_grid_shape: Tuple[int, int], world_size: int) -> None:
    process_rows, process_columns = process_grid_shape
    if process_rows <= 0 or process_columns <= 0:
        raise ValueError(
            f"process_grid_shape must contain positive dimensions, got {process_grid_shape}."
        )
    if process_rows * process_columns != world_size:
        raise ValueError(
            f"process_grid_shape={process_grid_shape} does not match world_size={world_size}."
        )


def current_world(process_grid_shape: Tuple[int, int]) -> Tuple[int, int]:
    """Return (rank, world_size) after checking the grid against the world.

    ``torch.distributed`` may be left uninitialised (then the world is one rank); a grid that
    does not match the world raises the reference's ``ValueError``; a world of more than one
    rank is outside what this one-GPU implementation covers.
    """
    if dist.is_available() and dist.is_initialized():
        rank, world_size = dist.get_rank(), dist.get_world_size()
    else:
        rank, world_size = 0, 1
    validate_process_grid(tuple(process_grid_shape), world_size)
    if world_size != 1:
        raise RuntimeError(
            "soap_tp_amd implements one GPU's share of the SOAP step: it requires "
            f"world_size == 1 and process_grid_shape == (1, 1), got world_size={world_size}."
        )
    return rank, world_size


def local_2d_block_cyclic_shape(
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    rank: int,
) -> Tuple[int, int]:
    rows, columns = global_shape
    process_rows, process_columns = process_grid_shape
    validate_process_grid(process_grid_shape, process_rows * process_columns)
    if not 0 <= rank < process_rows * process_columns:
        raise ValueError(f"rank must be in [0, {process_rows * process_columns}), got {rank}.")
    if block_size <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}.")
    if rows < 0:
        raise ValueError(f"size must be non-negative, got {rows}.")
    if columns < 0:
        raise ValueError(f"size must be non-negative, got {columns}.")
    if process_rows == 1 and process_columns == 1:
        return rows, columns
    process_row, process_column = divmod(rank, process_columns)
    return (
        len(block_cyclic_indices(rows, block_size, process_row, process_rows)),
        len(block_cyclic_indices(columns, block_size, process_column, process_columns)),
    )


def validate_2d_block_cyclic_buffer(
    name: str,
    matrix: torch.Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    rank: int,
) -> Tuple[int, int]:
    """Check a packed buffer and return its logical (rows, columns)
    (src/soap_tp/ops/_utils.py:120-156)."""
    if matrix.ndim != 2:
        raise ValueError(f"{name} must be 2D, got {matrix.ndim}D.")
    if matrix.stride(0) != 1:
        raise ValueError(
            f"{name} must use column-major local storage, got stride {matrix.stride()}."
        )
    local_rows, local_columns = local_2d_block_cyclic_shape(
        global_shape, block_size, process_grid_shape, rank
    )
    if matrix.size(0) < max(1, local_rows):
        raise ValueError(
            f"{name} has {matrix.size(0)} storage rows, expected at least {max(1, local_rows)}."
        )
    if matrix.size(1) < max(1, local_columns):
        raise ValueError(
            f"{name} has {matrix.size(1)} storage columns, expected at least "
            f"{max(1, local_columns)}."
        )
    if matrix.stride(1) < max(1, matrix.size(0)):
        raise ValueError(f"{name} has invalid leading dimension {matrix.stride(1)}.")
    return local_rows, local_columns


def allocate_2d_block_cyclic(
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    dtype: torch.dtype = torch.float32,
    device: torch.device | str | None = None,
) -> torch.Tensor:
    """Zeroed column-major buffer: a ``(columns, ld)`` allocation viewed transposed
    (src/soap_tp/ops/_utils.py:159-189)."""
    rank, _ = current_world(process_grid_shape)
    local_rows, local_columns = local_2d_block_cyclic_shape(
        global_shape, block_size, process_grid_shape, rank
    )
    return torch.zeros(
        (max(1, local_columns), max(1, local_rows)), dtype=dtype, device=device
    ).T


def empty_column_major(rows: int, columns: int, *, dtype: torch.dtype, device) -> torch.Tensor:
    return torch.empty((max(1, columns), max(1, rows)), dtype=dtype, device=device).T
