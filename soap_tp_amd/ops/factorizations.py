"""Rotations, eigenbasis initialisation and refresh of packed SOAP state.

Function names, argument order and error behaviour follow
src/soap_tp/ops/factorizations.py.  With no binding injected, each function is one call into
``libsoap_mi355.so``.  With a binding object (``slate_binding=`` / ``elpa_binding=``, the
reference's injection seam, :18-30) the reference's own call sequence runs against that
object's methods, so a counting or delegating proxy observes the same calls as it would around
the SLATE/ELPA modules.  Nothing here synchronises the device; the reference's
``torch.cuda.synchronize`` brackets (:169,183,234,245,308,319,530,543) existed because SLATE and
ELPA run on their own streams.
"""
from __future__ import annotations

from typing import Any, Literal, Optional, Tuple

import torch
from torch import Tensor

from ._common import (
    native_call,
    native_library,
    scratch,
    stream_of,
    validate_float_buffer,
    validated_binding,
)
from ._utils import current_world
from .optimizer import permute_2d_block_cyclic_


@torch.no_grad()
def rotate_2d_block_cyclic_(
    matrix: Tensor,
    Q_left: Tensor,
    Q_right: Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    direction: Literal["forward", "backward"],
    slate_binding: Optional[Any] = None,
) -> Tensor:
    """Rotate a packed matrix in place: ``forward`` is ``Q_left.T @ matrix @ Q_right``,
    ``backward`` is ``Q_left @ matrix @ Q_right.T`` (reference :104-184)."""
    if direction not in {"forward", "backward"}:
        raise ValueError(f"direction must be 'forward' or 'backward', got {direction!r}.")
    rank, world_size = current_world(process_grid_shape)
    rows, columns = global_shape
    validate_float_buffer("matrix", matrix, global_shape, block_size, process_grid_shape, rank)
    validate_float_buffer("Q_left", Q_left, (rows, rows), block_size, process_grid_shape, rank)
    validate_float_buffer("Q_right", Q_right, (columns, columns), block_size, process_grid_shape, rank)
    if len({matrix.device, Q_left.device, Q_right.device}) != 1:
        raise ValueError("matrix and bases must share a device.")
    if len({matrix.data_ptr(), Q_left.data_ptr(), Q_right.data_ptr()}) != 3:
        raise ValueError("matrix and basis buffers must not overlap.")
    binding = validated_binding(slate_binding, matrix.device, rank, world_size)
    process_rows, process_columns = process_grid_shape
    with torch.cuda.device(matrix.device):
        if slate_binding is None:
            work = scratch(native_library().soapmi_rotate_workspace_bytes(rows, columns), matrix.device)
            native_call(
                "soapmi_rotate_f32", Q_left.data_ptr(), matrix.data_ptr(), Q_right.data_ptr(), rows, columns,
                Q_left.stride(1), matrix.stride(1), Q_right.stride(1), 1 if direction == "forward" else 0,
                work.data_ptr(), work.numel(), stream_of(matrix),
            )
        else:
            function = (
                binding.slate_forward_rotation_float
                if direction == "forward"
                else binding.slate_backward_rotation_float
            )
            # an injected binding may work on streams of its own (SLATE does): the call is
            # bracketed by synchronisations, as in the reference (:169,:183)
            torch.cuda.synchronize(matrix.device)
            function(
                Q_left.data_ptr(), matrix.data_ptr(), Q_right.data_ptr(), rows, columns,
                Q_left.stride(1), matrix.stride(1), Q_right.stride(1), block_size,
                process_rows, process_columns,
            )
            torch.cuda.synchronize(matrix.device)
    return matrix


def _validate_square_triple(preconditioner, Q, work, size, block_size, process_grid_shape, rank):
    for name, matrix in (("preconditioner", preconditioner), ("Q", Q), ("work", work)):
        validate_float_buffer(name, matrix, (size, size), block_size, process_grid_shape, rank)
        if matrix.device != preconditioner.device:
            raise ValueError("preconditioner, Q, and work must share a device.")
    if len({preconditioner.data_ptr(), Q.data_ptr(), work.data_ptr()}) != 3:
        raise ValueError("preconditioner, Q, and work must not overlap.")


@torch.no_grad()
def estimated_eigenvalue_order_2d_block_cyclic_(
    preconditioner: Tensor,
    Q: Tensor,
    work: Tensor,
    size: int,
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    slate_binding: Optional[Any] = None,
) -> Tensor:
    """Return the descending order of ``diag(Q.T @ P @ Q)``; ``work`` is overwritten with
    ``P @ Q`` (reference :187-271).  Both triangles of ``preconditioner`` are read."""
    rank, world_size = current_world(process_grid_shape)
    _validate_square_triple(preconditioner, Q, work, size, block_size, process_grid_shape, rank)
    if not (preconditioner.stride(1) == Q.stride(1) == work.stride(1)):
        raise ValueError("preconditioner, Q, and work LDAs must match.")
    binding = validated_binding(slate_binding, preconditioner.device, rank, world_size)
    device = preconditioner.device
    process_rows, process_columns = process_grid_shape
    estimates = torch.empty(size, dtype=torch.float32, device=device)
    order = torch.empty(size, dtype=torch.int64, device=device)
    with torch.cuda.device(device):
        stream = stream_of(preconditioner)
        if slate_binding is None:
            native_call("soapmi_symm_f32", preconditioner.data_ptr(), Q.data_ptr(), work.data_ptr(), size,
                        preconditioner.stride(1), Q.stride(1), work.stride(1), stream)
        else:
            torch.cuda.synchronize(device)  # reference :234,:245
            binding.slate_symmetric_multiply_float(
                preconditioner.data_ptr(), Q.data_ptr(), work.data_ptr(), size,
                preconditioner.stride(1), block_size, process_rows, process_columns,
            )
            torch.cuda.synchronize(device)
        native_call("soapmi_column_dots_f32", Q.data_ptr(), Q.stride(1), work.data_ptr(), work.stride(1),
                    size, size, estimates.data_ptr(), stream)
        sort_work = scratch(native_library().soapmi_argsort_workspace_bytes(size), device)
        native_call("soapmi_argsort_desc_f32", estimates.data_ptr(), size, order.data_ptr(),
                    sort_work.data_ptr(), sort_work.numel(), stream)
    return order


@torch.no_grad()
def qr_2d_block_cyclic_(
    matrix: Tensor,
    Q: Tensor,
    size: int,
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    slate_binding: Optional[Any] = None,
) -> Tensor:
    """Overwrite ``Q`` with the orthogonal QR factor of ``matrix`` (destroyed) (reference :274-320)."""
    rank, world_size = current_world(process_grid_shape)
    for name, buffer in (("matrix", matrix), ("Q", Q)):
        validate_float_buffer(name, buffer, (size, size), block_size, process_grid_shape, rank)
    if matrix.device != Q.device:
        raise ValueError("matrix and Q must share a device.")
    if matrix.data_ptr() == Q.data_ptr():
        raise ValueError("matrix and Q must not overlap.")
    binding = validated_binding(slate_binding, matrix.device, rank, world_size)
    process_rows, process_columns = process_grid_shape
    with torch.cuda.device(matrix.device):
        if slate_binding is None:
            work = scratch(native_library().soapmi_qr_workspace_bytes(size), matrix.device)
            native_call("soapmi_qr_f32", matrix.data_ptr(), Q.data_ptr(), size, matrix.stride(1), Q.stride(1),
                        work.data_ptr(), work.numel(), stream_of(matrix))
        else:
            torch.cuda.synchronize(matrix.device)  # reference :308,:319
            binding.slate_qr_float(
                matrix.data_ptr(), Q.data_ptr(), size, matrix.stride(1), Q.stride(1), block_size,
                process_rows, process_columns,
            )
            torch.cuda.synchronize(matrix.device)
    return Q


@torch.no_grad()
def power_iteration_qr_2d_block_cyclic_(
    preconditioner: Tensor,
    Q: Tensor,
    work: Tensor,
    size: int,
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    slate_binding: Optional[Any] = None,
    symmetrize: bool = False,
) -> Tensor:
    """Sort one power iterate, QR it into ``Q``, and return the sort order (reference :323-360).

    ``symmetrize=True`` (an extension) first copies the lower triangle of ``preconditioner`` onto
    its upper one, for preconditioners kept with ``mirror=False``.
    """
    if slate_binding is not None:
        if symmetrize:
            _symmetrize(preconditioner, size)
        order = estimated_eigenvalue_order_2d_block_cyclic_(
            preconditioner, Q, work, size, block_size, process_grid_shape, slate_binding=slate_binding
        )
        permute_2d_block_cyclic_(
            work, (size, size), torch.arange(size, device=work.device), order, block_size,
            process_grid_shape, validate=False,
        )
        qr_2d_block_cyclic_(work, Q, size, block_size, process_grid_shape, slate_binding=slate_binding)
        return order
    rank, world_size = current_world(process_grid_shape)
    _validate_square_triple(preconditioner, Q, work, size, block_size, process_grid_shape, rank)
    validated_binding(None, preconditioner.device, rank, world_size)
    device = preconditioner.device
    order = torch.empty(size, dtype=torch.int64, device=device)
    with torch.cuda.device(device):
        buffer = scratch(native_library().soapmi_power_iteration_qr_workspace_bytes(size), device)
        native_call(
            "soapmi_power_iteration_qr_f32", preconditioner.data_ptr(), Q.data_ptr(), work.data_ptr(), size,
            preconditioner.stride(1), Q.stride(1), work.stride(1), 1 if symmetrize else 0,
            order.data_ptr(), None, buffer.data_ptr(), buffer.numel(), stream_of(preconditioner),
        )
    return order


def _symmetrize(preconditioner: Tensor, size: int) -> None:
    with torch.cuda.device(preconditioner.device):
        native_call("soapmi_symmetrize_lower_f32", preconditioner.data_ptr(), size, preconditioner.stride(1),
                    stream_of(preconditioner))


@torch.no_grad()
def initialize_basis_2d_block_cyclic_(
    preconditioner: Tensor,
    Q: Tensor,
    work: Tensor,
    eigenvalues: Tensor,
    size: int,
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    implementation: Literal["elpa", "eigh"] = "elpa",
    elpa_binding: Optional[Any] = None,
) -> Tensor:
    """Initialize a descending eigenbasis (reference :363-547).

    ``"elpa"`` solves ``-P`` in float64 and overwrites ``work``, as the ELPA path does
    (:497-546); ``"eigh"`` solves ``P + 1e-30 I`` in float32 and flips the result (:446-469).
    Both run the library's Householder / divide-and-conquer eigensolver on the GPU.  Only the
    lower triangle of ``preconditioner`` is read.
    """
    if implementation not in {"elpa", "eigh"}:
        raise ValueError(f"implementation must be 'elpa' or 'eigh', got {implementation!r}.")
    rank, world_size = current_world(process_grid_shape)
    _validate_square_triple(preconditioner, Q, work, size, block_size, process_grid_shape, rank)
    if eigenvalues.shape != (size,) or eigenvalues.dtype != torch.float32:
        raise ValueError(
            f"eigenvalues must be float32 with shape {(size,)}, got "
            f"{eigenvalues.dtype} {tuple(eigenvalues.shape)}."
        )
    if not eigenvalues.is_contiguous():
        raise ValueError("eigenvalues must be contiguous.")
    if eigenvalues.device != preconditioner.device:
        raise ValueError("eigenvalues must share the matrix device.")
    device = preconditioner.device
    if implementation == "elpa":
        for name, matrix in (("preconditioner", preconditioner), ("Q", Q), ("work", work)):
            if matrix.stride(1) != max(1, size):
                raise ValueError(
                    f"{name} must use the exact ELPA leading dimension {max(1, size)}, "
                    f"got {matrix.stride(1)}."
                )
        if size == 0:
            raise ValueError(
                "ELPA initialization requires every rank to own at least one local row and column."
            )
    binding = validated_binding(elpa_binding, device, rank, world_size)
    with torch.cuda.device(device):
        if elpa_binding is not None and implementation == "elpa":
            # the reference's staging (:500-546) around the injected solver; the preconditioner
            # itself is left untouched, only its lower triangle is read
            work.copy_(torch.tril(preconditioner))
            work.add_(torch.tril(preconditioner, -1).T).neg_()
            work_double = torch.empty_strided(work.size(), work.stride(), dtype=torch.float64, device=device)
            work_double.copy_(work)
            Q_double = torch.empty_strided(Q.size(), Q.stride(), dtype=torch.float64, device=device)
            eigenvalues_double = torch.empty_like(eigenvalues, dtype=torch.float64)
            gpu_id = device.index if device.index is not None else torch.cuda.current_device()
            process_rows, process_columns = process_grid_shape
            # an injected binding may run on a stream of its own (ELPA does): bracket the call with
            # synchronisations, as the reference does (:530,:543)
            torch.cuda.synchronize(device)
            binding.elpa_eigenvectors_2d_block_cyclic_double(
                work_double.data_ptr(), eigenvalues_double.data_ptr(), Q_double.data_ptr(), size, size, size,
                block_size, process_rows, process_columns, gpu_id,
            )
            torch.cuda.synchronize(device)
            Q.copy_(Q_double)
            eigenvalues.copy_(eigenvalues_double).neg_()
            return Q
        code = 0 if implementation == "elpa" else 1
        buffer = scratch(native_library().soapmi_initialize_basis_workspace_bytes(size, code), device)
        native_call(
            "soapmi_initialize_basis_f32", preconditioner.data_ptr(), Q.data_ptr(), work.data_ptr(),
            eigenvalues.data_ptr(), size, preconditioner.stride(1), Q.stride(1), work.stride(1), code,
            buffer.data_ptr(), buffer.numel(), stream_of(preconditioner),
        )
    return Q


@torch.no_grad()
def refresh_bases_and_transport_optimizer_state_(
    momentum: Tensor,
    variance: Tensor,
    left_preconditioner: Tensor,
    right_preconditioner: Tensor,
    Q_left: Tensor,
    Q_right: Tensor,
    left_work: Tensor,
    right_work: Tensor,
    global_shape: Tuple[int, int],
    block_size: int,
    process_grid_shape: Tuple[int, int],
    *,
    slate_binding: Optional[Any] = None,
    symmetrize: bool = False,
) -> tuple[Tensor, Tensor]:
    """Refresh both bases while preserving SOAP optimizer-state semantics (reference :550-614)."""
    rows, columns = global_shape
    if slate_binding is not None:
        rotate_2d_block_cyclic_(momentum, Q_left, Q_right, global_shape, block_size, process_grid_shape,
                                direction="backward", slate_binding=slate_binding)
        left_order = power_iteration_qr_2d_block_cyclic_(
            left_preconditioner, Q_left, left_work, rows, block_size, process_grid_shape,
            slate_binding=slate_binding, symmetrize=symmetrize)
        right_order = power_iteration_qr_2d_block_cyclic_(
            right_preconditioner, Q_right, right_work, columns, block_size, process_grid_shape,
            slate_binding=slate_binding, symmetrize=symmetrize)
        permute_2d_block_cyclic_(variance, global_shape, left_order, right_order, block_size,
                                 process_grid_shape, validate=False)
        rotate_2d_block_cyclic_(momentum, Q_left, Q_right, global_shape, block_size, process_grid_shape,
                                direction="forward", slate_binding=slate_binding)
        return left_order, right_order

    rank, world_size = current_world(process_grid_shape)
    validate_float_buffer("matrix", momentum, global_shape, block_size, process_grid_shape, rank)
    validate_float_buffer("matrix", variance, global_shape, block_size, process_grid_shape, rank)
    _validate_square_triple(left_preconditioner, Q_left, left_work, rows, block_size, process_grid_shape, rank)
    _validate_square_triple(right_preconditioner, Q_right, right_work, columns, block_size, process_grid_shape, rank)
    device = momentum.device
    if len({t.device for t in (momentum, variance, left_preconditioner, right_preconditioner)}) != 1:
        raise ValueError("matrix and bases must share a device.")
    if len({momentum.data_ptr(), variance.data_ptr(), Q_left.data_ptr(), Q_right.data_ptr()}) != 4:
        raise ValueError("matrix and basis buffers must not overlap.")
    validated_binding(None, device, rank, world_size)
    left_order = torch.empty(rows, dtype=torch.int64, device=device)
    right_order = torch.empty(columns, dtype=torch.int64, device=device)
    with torch.cuda.device(device):
        buffer = scratch(native_library().soapmi_refresh_workspace_bytes(rows, columns), device)
        native_call(
            "soapmi_refresh_f32",
            momentum.data_ptr(), momentum.stride(1), variance.data_ptr(), variance.stride(1),
            left_preconditioner.data_ptr(), left_preconditioner.stride(1),
            right_preconditioner.data_ptr(), right_preconditioner.stride(1),
            Q_left.data_ptr(), Q_left.stride(1), Q_right.data_ptr(), Q_right.stride(1),
            left_work.data_ptr(), left_work.stride(1), right_work.data_ptr(), right_work.stride(1),
            rows, columns, 1 if symmetrize else 0, left_order.data_ptr(), right_order.data_ptr(),
            buffer.data_ptr(), buffer.numel(), stream_of(momentum),
        )
    return left_order, right_order
