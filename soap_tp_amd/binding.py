"""The binding object that stands where ``soap_tp.slate_bindings`` and
``soap_tp.elpa_bindings`` stand in the reference.

The reference's ops take an injectable binding (``slate_binding=``, ``elpa_binding=``;
src/soap_tp/ops/factorizations.py:18-30,85-101) whose methods receive raw buffer addresses,
sizes and leading dimensions.  ``NativeBinding`` offers the same method names and argument
order (src/soap_tp/csrc/slate_bindings.cpp:317-389, elpa_bindings.cpp:200-236) on top of
``libsoap_mi355.so``; ``block_size`` and the process grid are accepted and checked but have no
effect on one rank.  Work is enqueued on torch's current stream of the current device and is
not synchronised.
"""
from __future__ import annotations

import torch

from . import _native


def _current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _workspace(query: str, *sizes):
    """Scratch for one call from torch's caching allocator: stream-ordered, so the call neither
    allocates through the runtime nor synchronises, and concurrent streams do not share it."""
    nbytes = getattr(_native.library(), query)(*sizes)
    buffer = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=torch.device("cuda", torch.cuda.current_device()))
    return buffer


def _check_grid(process_rows: int, process_cols: int) -> None:
    if process_rows <= 0 or process_cols <= 0 or process_rows * process_cols != 1:
        raise ValueError("process grid must be positive and contain every MPI world rank")


class NativeBinding:
    """Drop-in for both reference binding modules on a 1x1 process grid."""

    def compiled_gpu_backend(self) -> str:
        return _native.compiled_gpu_backend()

    def mpi_world_rank_and_size(self):
        return _native.world_rank_and_size()

    # ---- SLATE replacements -------------------------------------------------------------
    def slate_symmetric_multiply_float(self, a, q, work, n, lda, block_size, process_rows, process_cols):
        _check_grid(process_rows, process_cols)
        if a == 0 or q == 0 or work == 0:
            raise ValueError("SLATE buffer addresses must be nonzero")
        if n <= 0 or lda <= 0 or block_size <= 0:
            raise ValueError("matrix size, leading dimension, and block size must be positive")
        _native.call("soapmi_symm_f32", a, q, work, n, lda, lda, lda, _current_stream())

    def slate_qr_float(self, matrix, q, n, ldmatrix, ldq, block_size, process_rows, process_cols):
        _check_grid(process_rows, process_cols)
        if matrix == 0 or q == 0:
            raise ValueError("SLATE buffer addresses must be nonzero")
        if n <= 0 or ldmatrix <= 0 or ldq <= 0 or block_size <= 0:
            raise ValueError("matrix size, leading dimensions, and block size must be positive")
        work = _workspace("soapmi_qr_workspace_bytes", n)
        _native.call("soapmi_qr_f32", matrix, q, n, ldmatrix, ldq, work.data_ptr(), work.numel(), _current_stream())

    def _rotation(self, forward, q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix, ldq_right,
                  block_size, process_rows, process_cols):
        _check_grid(process_rows, process_cols)
        if q_left == 0 or matrix == 0 or q_right == 0:
            raise ValueError("SLATE buffer addresses must be nonzero")
        if min(rows, columns, ldq_left, ldmatrix, ldq_right, block_size) <= 0:
            raise ValueError("matrix dimensions, leading dimensions, and block size must be positive")
        work = _workspace("soapmi_rotate_workspace_bytes", rows, columns)
        _native.call("soapmi_rotate_f32", q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix,
                     ldq_right, 1 if forward else 0, work.data_ptr(), work.numel(), _current_stream())

    def slate_forward_rotation_float(self, q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix,
                                     ldq_right, block_size, process_rows, process_cols):
        self._rotation(True, q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix, ldq_right,
                       block_size, process_rows, process_cols)

    def slate_backward_rotation_float(self, q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix,
                                      ldq_right, block_size, process_rows, process_cols):
        self._rotation(False, q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix, ldq_right,
                       block_size, process_rows, process_cols)

    # ---- ELPA replacement ---------------------------------------------------------------
    def initialize_basis_2d_block_cyclic_(self, a, eigenvalues, q, n, local_rows, local_columns, block_size,
                                          process_rows, process_columns, gpu_id=-1):
        """Ascending eigenpairs of the float64 matrix at ``a`` (destroyed)."""
        if a == 0 or eigenvalues == 0 or q == 0:
            raise ValueError("ELPA buffer addresses must be nonzero")
        if n <= 0 or local_rows <= 0 or local_columns <= 0 or block_size <= 0:
            raise ValueError("matrix dimensions and block size must be positive")
        if process_rows <= 0 or process_columns <= 0 or process_rows * process_columns != 1:
            raise ValueError("the process grid must be positive and contain every MPI rank")
        if gpu_id < 0:
            raise ValueError("a nonnegative GPU device index is required by this ELPA build")
        if local_rows != n or local_columns != n:
            raise ValueError("on a 1x1 process grid the local shape must equal the matrix size")
        with torch.cuda.device(gpu_id):
            work = _workspace("soapmi_eigh_workspace_bytes", n, 8)
            _native.call("soapmi_eigh_f64", a, eigenvalues, q, n, local_rows, local_rows, work.data_ptr(),
                         work.numel(), _current_stream())

    elpa_eigenvectors_2d_block_cyclic_double = initialize_basis_2d_block_cyclic_


_default_binding = None


def default_binding() -> NativeBinding:
    global _default_binding
    if _default_binding is None:
        _native.library()  # fail loudly if the kernels were never built
        _default_binding = NativeBinding()
    return _default_binding
