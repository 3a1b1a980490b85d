"""Composable single-GPU operations of the SOAP step (the names exported by
src/soap_tp/ops/__init__.py:23-37 of the reference)."""

from ._utils import allocate_2d_block_cyclic
from .factorizations import (
    estimated_eigenvalue_order_2d_block_cyclic_,
    initialize_basis_2d_block_cyclic_,
    power_iteration_qr_2d_block_cyclic_,
    qr_2d_block_cyclic_,
    refresh_bases_and_transport_optimizer_state_,
    rotate_2d_block_cyclic_,
)
from .optimizer import (
    adam_update,
    permute_2d_block_cyclic_,
    redistribute_2d_block_cyclic_to_tp_shard,
    redistribute_tp_shard_to_2d_block_cyclic,
)
from .preconditioners import (
    update_left_preconditioner_2d_block_cyclic_,
    update_right_preconditioner_2d_block_cyclic_,
)

__all__ = [
    "adam_update",
    "allocate_2d_block_cyclic",
    "estimated_eigenvalue_order_2d_block_cyclic_",
    "initialize_basis_2d_block_cyclic_",
    "permute_2d_block_cyclic_",
    "power_iteration_qr_2d_block_cyclic_",
    "qr_2d_block_cyclic_",
    "redistribute_2d_block_cyclic_to_tp_shard",
    "redistribute_tp_shard_to_2d_block_cyclic",
    "refresh_bases_and_transport_optimizer_state_",
    "rotate_2d_block_cyclic_",
    "update_left_preconditioner_2d_block_cyclic_",
    "update_right_preconditioner_2d_block_cyclic_",
]
