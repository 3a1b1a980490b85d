"""``soap_step``: one SOAP update of a dense 2-D parameter on one MI355X.

Same signature, state dictionary and sequencing as the reference orchestrator
(src/soap_tp/soap.py:123-506) at ``process_grid_shape == (1, 1)``:

* first call: allocate the eight packed buffers, form both Gram preconditioners from a zero
  state, initialise both eigenbases, set ``state["step"] = 0`` and return exact zeros
  (:163-276);
* later calls: rotate the gradient into the eigenbasis, Adam there, rotate the update back
  (:327-417), then update the preconditioners with the same gradient (:425-448) and, when
  ``step % basis_refresh_interval == 0``, refresh the bases and transport the optimizer state
  (:457-471).

Beyond the reference's keys the state holds ``"status"``: one int32 of pinned host memory that a
factorisation kernel of this state raises if it gives up on the device (see ``soap_tp_amd.ops._common``).

The default path issues three library calls per step (update, left Gram, right Gram; plus one
on refresh steps) on torch's current stream and never synchronises.  When a binding object is
injected (``slate_binding`` / ``elpa_binding``) or ``SOAP_PROFILE`` is set, the step runs op by
op through ``soap_tp_amd.ops`` exactly in the reference's order, so proxies see every call and
every intermediate stage exists to be dumped.
"""
from __future__ import annotations

import math
import threading
from typing import Any, Literal, MutableMapping

import torch
from torch import Tensor

from . import _profile
from .ops import (
    adam_update,
    allocate_2d_block_cyclic,
    initialize_basis_2d_block_cyclic_,
    redistribute_2d_block_cyclic_to_tp_shard,
    redistribute_tp_shard_to_2d_block_cyclic,
    refresh_bases_and_transport_optimizer_state_,
    rotate_2d_block_cyclic_,
    update_left_preconditioner_2d_block_cyclic_,
    update_right_preconditioner_2d_block_cyclic_,
)
from .ops._common import (native_call, native_library, new_status_word, raise_on_device_error,
                          raise_on_state_error, reporting_to, require_device_tensor, scratch, stream_of)
from .ops._utils import current_world

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


_SIDE_STREAMS: dict = {}


def _side_stream(device, main) -> "torch.cuda.Stream":
    """One extra stream (default priority) per device and calling stream, created on first use and
    kept: callers that step parameters on several streams get a side stream for each of them."""
    key = (torch.device(device), main.cuda_stream)
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
    return _SIDE_STREAMS[key]


def _state_shapes(rows: int, columns: int) -> dict:
    square = {"left": (rows, rows), "right": (columns, columns)}
    shapes = {}
    for name in STATE_BUFFERS:
        side = name.split("_", 1)[0]
        shapes[name] = square.get(side, (rows, columns))
    return shapes


def _fused_update(gradient: Tensor, state, rows: int, columns: int, step: int, beta1, beta2, eps) -> Tensor:
    """Forward rotation, Adam and backward rotation as four chained MFMA products."""
    update = torch.empty_like(gradient)
    device = gradient.device
    with torch.cuda.device(device):
        work = scratch(native_library().soapmi_rotate_adam_rotate_workspace_bytes(rows, columns), device)
        native_call(
            "soapmi_rotate_adam_rotate_f32",
            gradient.data_ptr(), gradient.stride(0), update.data_ptr(), update.stride(0),
            state["left_basis"].data_ptr(), state["left_basis"].stride(1),
            state["right_basis"].data_ptr(), state["right_basis"].stride(1),
            state["momentum"].data_ptr(), state["momentum"].stride(1),
            state["variance"].data_ptr(), state["variance"].stride(1),
            rows, columns, step, float(beta1), float(beta2), float(eps),
            work.data_ptr(), work.numel(), stream_of(gradient),
        )
    return update


def _fused_gram_pair(gradient: Tensor, state, rows: int, columns: int, beta: float, mirror: bool) -> None:
    """Both Gram EMAs of a step in one launch (the gradient is the contiguous fp32 copy made by soap_step)."""
    if not 0.0 <= beta <= 1.0:
        raise ValueError(f"beta must be in [0, 1], got {beta}.")
    left, right = state["left_preconditioner"], state["right_preconditioner"]
    with torch.cuda.device(gradient.device):
        native_call(
            "soapmi_gram_ema_pair_f32",
            gradient.data_ptr(), rows, columns, gradient.stride(0), 1,
            left.data_ptr(), left.stride(1), right.data_ptr(), right.stride(1),
            float(beta), 1 if mirror else 0, stream_of(gradient),
        )


@torch.no_grad()
def soap_step(
    gradient_shard: Tensor,
    state: MutableMapping[str, Any],
    *,
    global_shape: tuple[int, int],
    shard_dim: Literal[0, 1],
    block_size: int,
    process_grid_shape: tuple[int, int],
    preconditioner_beta: float = 0.95,
    beta1: float = 0.95,
    beta2: float = 0.95,
    eps: float = 1e-8,
    basis_refresh_interval: int = 10,
    basis_implementation: Literal["elpa", "eigh"] = "elpa",
    elpa_binding: Any | None = None,
    slate_binding: Any | None = None,
    preconditioner_storage: Literal["lower", "full"] = "lower",
) -> Tensor:
    """Run one SOAP update and return the normalized ``float32`` update for the shard.

    ``state`` is a mutable per-parameter dictionary, populated on the first call.  Applying a
    learning rate, weight decay and the update itself stays with the caller.
    ``preconditioner_storage`` is an extension: ``"lower"`` keeps only the lower triangle of the
    Gram matrices up to date between refreshes (the upper one is rebuilt when a refresh reads
    it); ``"full"`` keeps both triangles valid after every call, as the reference does.
    """
    if basis_refresh_interval <= 0:
        raise ValueError("basis_refresh_interval must be positive.")
    if basis_implementation not in {"elpa", "eigh"}:
        raise ValueError(
            f"basis_implementation must be 'elpa' or 'eigh', got {basis_implementation!r}."
        )
    if preconditioner_storage not in {"lower", "full"}:
        raise ValueError(
            f"preconditioner_storage must be 'lower' or 'full', got {preconditioner_storage!r}."
        )
    if shard_dim not in (0, 1):
        raise ValueError(f"shard_dim must be 0 or 1, got {shard_dim}.")
    current_world(process_grid_shape)
    rows, columns = global_shape
    if gradient_shard.ndim != 2:
        raise ValueError(f"matrix must be 2D, got {gradient_shard.ndim}D.")
    if tuple(gradient_shard.shape) != (rows, columns):
        raise ValueError(
            f"matrix has shape {tuple(gradient_shard.shape)}, expected {(rows, columns)} "
            f"for shard_dim={shard_dim}."
        )
    require_device_tensor("gradient_shard", gradient_shard)
    mirror = preconditioner_storage == "full"
    device = gradient_shard.device
    # A factorisation kernel that failed on the device: this state's own word first (set by its
    # initialisation and refreshes, and left raised, so a poisoned state raises on every later step while
    # other states go on), then the device-wide word that factorisations enqueued without one raise.
    raise_on_state_error(state)
    raise_on_device_error(device)
    initializing = "left_basis" not in state
    status = state.get("status")
    if not (isinstance(status, Tensor) and status.dtype == torch.int32 and status.numel() >= 1 and status.is_pinned()):
        # (a state restored from a checkpoint comes without one; a deep copy of a state has one that
        # is no longer pinned memory, which a kernel could not write to)
        state["status"] = new_status_word()

    if initializing:
        for name, shape in _state_shapes(rows, columns).items():
            state[name] = allocate_2d_block_cyclic(shape, block_size, process_grid_shape, device=device)

    gradient = gradient_shard.detach().to(torch.float32).contiguous()
    profile_step = 0 if initializing else int(state["step"]) + 1
    profiling = _profile.enabled(profile_step)
    _profile.dump("gradient", profile_step, gradient)

    def update_preconditioners(suffix: str) -> None:
        if slate_binding is None and not profiling:
            _fused_gram_pair(gradient, state, rows, columns, preconditioner_beta, mirror)
            return
        update_left_preconditioner_2d_block_cyclic_(
            gradient, state["left_preconditioner"], preconditioner_beta, block_size, process_grid_shape,
            shard_dim=shard_dim, mirror=mirror)
        update_right_preconditioner_2d_block_cyclic_(
            gradient, state["right_preconditioner"], preconditioner_beta, block_size, process_grid_shape,
            shard_dim=shard_dim, mirror=mirror)
        if profiling:
            for side in ("left", "right"):
                matrix = state[f"{side}_preconditioner"]
                if not mirror:
                    matrix = torch.tril(matrix) + torch.tril(matrix, -1).T
                _profile.dump(f"{side}_preconditioner{suffix}", profile_step, matrix)

    if initializing:
        update_preconditioners("")

        def initialize(side: str, size: int) -> None:
            with reporting_to(state["status"]):
                initialize_basis_2d_block_cyclic_(
                    state[f"{side}_preconditioner"], state[f"{side}_basis"], state[f"{side}_work"],
                    torch.empty(size, dtype=torch.float32, device=device), size, block_size,
                    process_grid_shape, implementation=basis_implementation, elpa_binding=elpa_binding)

        sides = (("left", rows), ("right", columns))
        if elpa_binding is None and not profiling:
            # The two eigensolves are independent: the smaller one runs on a side stream (default
            # priority) forked from and joined back into the current one, so its latency-bound column
            # steps fill the gaps of the larger one.  An eigensolve is tens of thousands of launches
            # and the host does not run ahead of the device by that many, so the smaller one is
            # enqueued by a helper thread while this one enqueues the larger one (the library calls
            # release the interpreter lock).  Each solve's kernels and their order are what they are
            # alone, so the bases are the same bit for bit.
            small, large = sorted(sides, key=lambda item: item[1])
            main = torch.cuda.current_stream(device)
            side_stream = _side_stream(device, main)
            side_stream.wait_stream(main)
            failures = []

            def enqueue_small() -> None:
                try:
                    with torch.cuda.device(device), torch.cuda.stream(side_stream), torch.no_grad():
                        initialize(*small)
                except BaseException as error:  # re-raised by the calling thread
                    failures.append(error)

            helper = threading.Thread(target=enqueue_small, name="soap-init-small-side")
            helper.start()
            try:
                initialize(*large)
            finally:
                helper.join()
                main.wait_stream(side_stream)
            if failures:
                raise failures[0]
        else:
            for side, size in sides:
                initialize(side, size)
        for side, _ in sides:
            _profile.dump(f"{side}_basis", profile_step, state[f"{side}_basis"])
        state["step"] = 0
        zero_update = torch.zeros_like(gradient)
        _profile.dump("returned_update", profile_step, zero_update)
        return zero_update

    step = int(state["step"]) + 1
    if profiling:
        for name in ("left_basis", "right_basis"):
            _profile.dump(name, profile_step, state[name])
        _profile.dump("momentum_before_adam", profile_step, state["momentum"])
        _profile.dump("variance_before_adam", profile_step, state["variance"])

    if slate_binding is None and not profiling:
        update_shard = _fused_update(gradient, state, rows, columns, step, beta1, beta2, eps)
    else:
        packed = redistribute_tp_shard_to_2d_block_cyclic(
            gradient, global_shape, block_size, process_grid_shape, shard_dim=shard_dim)
        _profile.dump("gradient_2d", profile_step, packed)
        rotate_2d_block_cyclic_(packed, state["left_basis"], state["right_basis"], global_shape, block_size,
                                process_grid_shape, direction="forward", slate_binding=slate_binding)
        _profile.dump("projected_gradient", profile_step, packed)
        packed_update = adam_update(packed, state["momentum"], state["variance"], step, beta1, beta2,
                                    eps / math.sqrt(1.0 - beta2**step))
        _profile.dump("momentum_after_adam", profile_step, state["momentum"])
        _profile.dump("variance_after_adam", profile_step, state["variance"])
        _profile.dump("coordinate_update", profile_step, packed_update)
        rotate_2d_block_cyclic_(packed_update, state["left_basis"], state["right_basis"], global_shape,
                                block_size, process_grid_shape, direction="backward",
                                slate_binding=slate_binding)
        _profile.dump("backrotated_update", profile_step, packed_update)
        update_shard = redistribute_2d_block_cyclic_to_tp_shard(
            packed_update, global_shape, block_size, process_grid_shape, shard_dim=shard_dim)
    _profile.dump("returned_update", profile_step, update_shard)

    update_preconditioners("_after_step")
    if step % basis_refresh_interval == 0:
        with reporting_to(state["status"]):
            refresh_bases_and_transport_optimizer_state_(
                state["momentum"], state["variance"], state["left_preconditioner"],
                state["right_preconditioner"], state["left_basis"], state["right_basis"],
                state["left_work"], state["right_work"], global_shape, block_size, process_grid_shape,
                slate_binding=slate_binding, symmetrize=not mirror)
    if profiling:
        _profile.dump("left_basis_after_step", profile_step, state["left_basis"])
        _profile.dump("right_basis_after_step", profile_step, state["right_basis"])
        _profile.dump("momentum_after_step", profile_step, state["momentum"])
        _profile.dump("variance_after_step", profile_step, state["variance"])
    state["step"] = step
    return update_shard


__all__ = ["soap_step"]
