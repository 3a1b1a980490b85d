"""Adam in the eigenbasis, permutations and layout changes of packed matrices.

Mirrors src/soap_tp/ops/optimizer.py.  On one rank the two ``redistribute_*`` functions are
layout copies (row-major shard <-> column-major packed buffer) and ``permute_2d_block_cyclic_``
is a gather; the reference's all-to-all machinery (:130-219, :282-392, :476-566) has nothing
left to do.
"""
from __future__ import annotations

from typing import Literal, Optional, Sequence, Tuple

import torch
from torch import Tensor

from ._common import native_call, native_library, require_device_tensor, scratch, stream_of
from ._utils import current_world, empty_column_major


def _column_major_view(tensor: Tensor) -> Optional[Tuple[Tensor, int]]:
    if tensor.ndim == 2 and tensor.stride(0) == 1 and tensor.stride(1) >= max(1, tensor.size(0)):
        return tensor, tensor.stride(1)
    return None


@torch.no_grad()
def adam_update(
    gradient: Tensor,
    momentum: Tensor,
    variance: Tensor,
    step: int,
    beta1: float = 0.9,
    beta2: float = 0.999,
    eps: float = 1e-8,
) -> Tensor:
    """Update local Adam state and return the bias-corrected update
    (src/soap_tp/ops/optimizer.py:12-44); one fused kernel instead of seven passes."""
    if step < 1:
        raise ValueError(f"step must be positive, got {step}.")
    if not 0.0 <= beta1 < 1.0:
        raise ValueError(f"beta1 must be in [0, 1), got {beta1}.")
    if not 0.0 <= beta2 < 1.0:
        raise ValueError(f"beta2 must be in [0, 1), got {beta2}.")
    if eps <= 0.0:
        raise ValueError(f"eps must be positive, got {eps}.")
    if gradient.shape != momentum.shape or gradient.shape != variance.shape:
        raise ValueError("gradient, momentum, and variance must have identical shapes.")
    if gradient.ndim != 2:
        raise ValueError(f"gradient must be 2D, got {gradient.ndim}D.")
    for name, tensor in (("gradient", gradient), ("momentum", momentum), ("variance", variance)):
        require_device_tensor(name, tensor)
        if tensor.dtype != torch.float32:
            raise ValueError(f"{name} must use float32, got {tensor.dtype}.")
    rows, columns = gradient.shape
    # The kernel addresses element (i, j) at base + i + j*ld.  Column-major tensors are used as
    # they are; row-major ones are handled as the transposed problem.
    views = [_column_major_view(t) for t in (gradient, momentum, variance)]
    if all(view is not None for view in views):
        update = torch.empty_strided(variance.shape, variance.stride(), dtype=torch.float32, device=variance.device)
        g, m, v, u = gradient, momentum, variance, update
        kernel_rows, kernel_columns = rows, columns
    else:
        transposed = [_column_major_view(t.T) for t in (gradient, momentum, variance)]
        if not all(view is not None for view in transposed):
            raise ValueError(
                "gradient, momentum, and variance must all be column-major or all row-major matrices."
            )
        update = torch.empty_strided(variance.shape, variance.stride(), dtype=torch.float32, device=variance.device)
        g, m, v, u = gradient.T, momentum.T, variance.T, update.T
        kernel_rows, kernel_columns = columns, rows
    if rows == 0 or columns == 0:
        return update
    with torch.cuda.device(gradient.device):
        native_call(
            "soapmi_adam_f32",
            g.data_ptr(), g.stride(1), m.data_ptr(), m.stride(1), v.data_ptr(), v.stride(1),
            u.data_ptr(), u.stride(1), kernel_rows, kernel_columns, int(step),
            float(beta1), float(beta2), float(eps), stream_of(gradient),
        )
    return update


def _checked_order(order: Sequence[int] | Tensor, size: int, name: str, device) -> Tensor:
    """Device int64 copy of ``order`` after the reference's permutation check
    (src/soap_tp/ops/optimizer.py:47-61)."""
    if isinstance(order, Tensor):
        if order.ndim != 1:
            raise ValueError(f"{name} must be 1D, got {order.ndim}D.")
        order_tensor = order.to(device=device, dtype=torch.int64).contiguous()
    else:
        order_tensor = torch.tensor([int(index) for index in order], dtype=torch.int64, device=device)
    if order_tensor.numel() != size:
        raise ValueError(f"{name} must be a permutation of range({size}).")
    if size:
        work = scratch((size + 1) * 4 + 512, device)
        with torch.cuda.device(device):
            verdict = native_library().soapmi_is_permutation(
                order_tensor.data_ptr(), size, work.data_ptr(), work.numel(),
                torch.cuda.current_stream(device).cuda_stream,
            )
        if verdict < 0:
            raise RuntimeError("permutation check failed to run")
        if verdict == 0:
            raise ValueError(f"{name} must be a permutation of range({size}).")
    return order_tensor


@torch.no_grad()
def permute_2d_block_cyclic_(
    matrix: Tensor,
    global_shape: Tuple[int, int],
    row_order: Sequence[int] | Tensor,
    column_order: Sequence[int] | Tensor,
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    group=None,
    validate: bool = True,
) -> Tensor:
    """Apply ``matrix[row_order][:, column_order]`` to a packed matrix in place
    (src/soap_tp/ops/optimizer.py:395-567).  ``validate=False`` (an extension) skips the
    permutation check, which has to synchronise with the device."""
    if matrix.ndim != 2:
        raise ValueError(f"matrix must be 2D, got {matrix.ndim}D.")
    if block_size <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}.")
    rows, columns = global_shape
    if rows < 0 or columns < 0:
        raise ValueError(f"global_shape must be non-negative, got {global_shape}.")
    require_device_tensor("matrix", matrix)
    if matrix.dtype != torch.float32:
        raise ValueError(f"matrix must use float32, got {matrix.dtype}.")
    device = matrix.device
    if validate:
        row_index = _checked_order(row_order, rows, "row_order", device)
        column_index = _checked_order(column_order, columns, "column_order", device)
    else:
        row_index = torch.as_tensor(row_order, dtype=torch.int64, device=device).contiguous()
        column_index = torch.as_tensor(column_order, dtype=torch.int64, device=device).contiguous()
    process_rows, process_columns = process_grid_shape
    if process_rows <= 0 or process_columns <= 0:
        raise ValueError(
            f"process_grid_shape must contain positive dimensions, got {process_grid_shape}."
        )
    if process_rows * process_columns != 1:
        raise ValueError("process grid must contain every process-group rank.")
    if matrix.size(0) < rows or matrix.size(1) < columns:
        raise ValueError(
            f"matrix shape {tuple(matrix.shape)} is smaller than its logical "
            f"block-cyclic shape {(rows, columns)}."
        )
    if rows == 0 or columns == 0:
        return matrix
    logical = matrix[:rows, :columns]
    if logical.stride(0) == 1:
        target, kernel_rows, kernel_columns, first, second = logical, rows, columns, row_index, column_index
    elif logical.stride(1) == 1:
        target, kernel_rows, kernel_columns, first, second = logical.T, columns, rows, column_index, row_index
    else:
        raise ValueError(f"matrix must be column-major or row-major, got stride {matrix.stride()}.")
    nbytes = native_library().soapmi_permute_workspace_bytes(kernel_rows, kernel_columns)
    work = scratch(nbytes, device)
    with torch.cuda.device(device):
        native_call(
            "soapmi_permute_f32", target.data_ptr(), target.stride(1), kernel_rows, kernel_columns,
            first.data_ptr(), second.data_ptr(), work.data_ptr(), work.numel(), stream_of(matrix),
        )
    return matrix


def _check_redistribution(matrix, global_shape, block_size, process_grid_shape, shard_dim):
    if matrix.ndim != 2:
        raise ValueError(f"matrix must be 2D, got {matrix.ndim}D.")
    if shard_dim not in (0, 1):
        raise ValueError(f"shard_dim must be 0 or 1, got {shard_dim}.")
    if block_size <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}.")
    rows, columns = global_shape
    if rows < 0 or columns < 0:
        raise ValueError(f"global_shape must be non-negative, got {global_shape}.")
    process_rows, process_columns = process_grid_shape
    if process_rows <= 0 or process_columns <= 0:
        raise ValueError(
            f"process_grid_shape must contain positive dimensions, got {process_grid_shape}."
        )
    if process_rows * process_columns != 1:
        raise ValueError("process grid must contain every process-group rank.")
    current_world(process_grid_shape)
    return rows, columns


def redistribute_2d_block_cyclic_to_tp_shard(
    matrix: Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    shard_dim: Literal[0, 1],
    group=None,
) -> Tensor:
    """Packed column-major matrix -> contiguous (row-major) TP shard, which on one rank is the
    whole matrix (src/soap_tp/ops/optimizer.py:64-219)."""
    rows, columns = _check_redistribution(matrix, global_shape, block_size, process_grid_shape, shard_dim)
    if matrix.size(0) < rows or matrix.size(1) < columns:
        raise ValueError(
            f"matrix shape {tuple(matrix.shape)} is smaller than its logical "
            f"block-cyclic shape {(rows, columns)}."
        )
    require_device_tensor("matrix", matrix)
    if matrix.dtype != torch.float32 or matrix.stride(0) != 1:
        return matrix[:rows, :columns].contiguous()
    output = matrix.new_empty((rows, columns))
    if rows and columns:
        with torch.cuda.device(matrix.device):
            native_call("soapmi_col_major_to_row_major_f32", matrix.data_ptr(), matrix.stride(1),
                        output.data_ptr(), columns, rows, columns, stream_of(matrix))
    return output


def redistribute_tp_shard_to_2d_block_cyclic(
    matrix: Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    shard_dim: Literal[0, 1],
    group=None,
) -> Tensor:
    """TP shard -> new packed column-major buffer (src/soap_tp/ops/optimizer.py:222-392)."""
    rows, columns = _check_redistribution(matrix, global_shape, block_size, process_grid_shape, shard_dim)
    if tuple(matrix.shape) != (rows, columns):
        raise ValueError(
            f"matrix has shape {tuple(matrix.shape)}, expected {(rows, columns)} for shard_dim={shard_dim}."
        )
    require_device_tensor("matrix", matrix)
    output = empty_column_major(rows, columns, dtype=matrix.dtype, device=matrix.device)
    if rows == 0 or columns == 0:
        return output
    if matrix.dtype != torch.float32 or matrix.stride(1) != 1:
        output[:rows, :columns].copy_(matrix)
        return output
    with torch.cuda.device(matrix.device):
        native_call("soapmi_row_major_to_col_major_f32", matrix.data_ptr(), matrix.stride(0),
                    output.data_ptr(), output.stride(1), rows, columns, stream_of(matrix))
    return output
