"""Stands where the reference's ``soap_tp.elpa_bindings`` extension module stands
(src/soap_tp/csrc/elpa_bindings.cpp:198-236): the same functions and argument names, served by
``libsoap_mi355.so`` on a 1x1 process grid."""
from soap_tp_amd.binding import default_binding as _binding


def compiled_gpu_backend():
    return _binding().compiled_gpu_backend()


def mpi_world_rank_and_size():
    return _binding().mpi_world_rank_and_size()


def initialize_basis_2d_block_cyclic_(a, eigenvalues, q, n, local_rows, local_columns, block_size, process_rows,
                                      process_columns, gpu_id=-1):
    """Ascending eigenpairs of the float64 matrix at address ``a`` (destroyed)."""
    return _binding().initialize_basis_2d_block_cyclic_(a, eigenvalues, q, n, local_rows, local_columns,
                                                        block_size, process_rows, process_columns, gpu_id)


elpa_eigenvectors_2d_block_cyclic_double = initialize_basis_2d_block_cyclic_
