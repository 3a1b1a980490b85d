"""Stands where the reference's ``soap_tp.slate_bindings`` extension module stands
(src/soap_tp/csrc/slate_bindings.cpp:317-389): the same six module-level functions with the same
argument names, served by ``libsoap_mi355.so`` on a 1x1 process grid."""
from soap_tp_amd.binding import default_binding as _binding


def compiled_gpu_backend():
    """Return the GPU backend selected when the binding was compiled."""
    return _binding().compiled_gpu_backend()


def mpi_world_rank_and_size():
    """Return the (rank, size) of the single-process world."""
    return _binding().mpi_world_rank_and_size()


def slate_symmetric_multiply_float(a, q, work, n, lda, block_size, process_rows, process_cols):
    """Compute work = A @ Q for a symmetric A."""
    return _binding().slate_symmetric_multiply_float(a, q, work, n, lda, block_size, process_rows, process_cols)


def slate_qr_float(matrix, q, n, ldmatrix, ldq, block_size, process_rows, process_cols):
    """Overwrite q with the QR factor of matrix."""
    return _binding().slate_qr_float(matrix, q, n, ldmatrix, ldq, block_size, process_rows, process_cols)


def slate_forward_rotation_float(q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix, ldq_right,
                                 block_size, process_rows, process_cols):
    return _binding().slate_forward_rotation_float(q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix,
                                                   ldq_right, block_size, process_rows, process_cols)


def slate_backward_rotation_float(q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix, ldq_right,
                                  block_size, process_rows, process_cols):
    return _binding().slate_backward_rotation_float(q_left, matrix, q_right, rows, columns, ldq_left, ldmatrix,
                                                    ldq_right, block_size, process_rows, process_cols)
