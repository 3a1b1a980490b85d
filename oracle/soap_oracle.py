"""CPU oracle for the SOAP step: TEST INFRASTRUCTURE ONLY.

A dense, single-process restatement (torch on CPU, LAPACK/MKL underneath) of what soap-tp
computes at ``world_size == 1`` / ``process_grid_shape == (1, 1)``, where every 2-D block-cyclic
buffer is a plain dense matrix and every collective is the identity.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module,
and only as the checker or the timed baseline: the product (``soap_tp_amd``) never does.

Each function cites the reference lines it restates (paths relative to the reference
repository).  What pins each function (see ``tests/test_oracle.py``):

=========================  =======================================================================
function                   pinned by
=========================  =======================================================================
``gram_ema``               float64 closed form ``L + (1-b)(GG^T - L)``; the reference's own test
                           formula (tests/unit/test_preconditioners.py:107-114,604-608); symmetry,
                           beta = 0 / 1 limits, quadratic scaling
``rotate``                 float64 ``QL^T M QR`` / ``QL M QR^T`` (tests/unit/test_factorizations.py:385,398);
                           norm preservation; backward(forward(X)) = X
``adam_update``            closed form of tests/unit/test_optimizer.py:32-49 at its parameters;
                           algebraic equivalence with the original optimizer's update
                           (tests/reference/soap.py:252-273) through the eps rescaling of
                           src/soap_tp/soap.py:367
``eigh_descending``        prescribed spectra ``Q diag(s) Q^T``; diagonal and Wilkinson matrices;
                           residual / orthogonality / trace identities; rank-deficient Gram
                           matrices (tests/unit/test_elpa_bindings.py:341-457); 2x2 closed form
``estimated_order``        ``argsort(diag(Q^T P Q))`` (tests/unit/test_slate_bindings.py:158-159)
``householder_qr``         ``Q^T Q = I``, ``Q^T W`` upper triangular, nested column spans, and an
                           independent unblocked Householder loop written in the test
``permute``                definition ``M[ro][:, co]`` by brute force; inverse round trip
``refresh``                composition formula of tests/unit/test_factorizations.py:550-571
``soap_step``              an independent restatement of the ORIGINAL optimizer's control flow
                           (``original_soap_reference`` below, after tests/reference/soap.py:145-345,
                           401-440,505-562: momentum leaves and re-enters the eigenbasis on every
                           step there) must produce the same updates; the golden trajectory in
                           tests/golden/ made by running that vendored optimizer itself; the
                           invariants of tests/unit/test_soap.py:791-801,844-849
=========================  =======================================================================

No function here is "parity unpinned" at tolerance level.  Bit-level agreement with SLATE and
ELPA themselves cannot be pinned: their sources are absent from the reference checkout (empty
submodules) and the reference's tests hold no stored vectors, only tolerance checks against the
same dense formulas used here.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch
from torch import Tensor


# ---- synthetic gradients ---------------------------------------------------------------------
def low_rank_plus_noise(
    rows: int,
    columns: int,
    rank: int,
    seed: int,
    *,
    noise_std: float = 1e-4,
    spectrum: Tuple[float, float] = (1e-4, 1e-1),
    dtype: torch.dtype = torch.float32,
) -> Tensor:
    """``U diag(s) V^T + noise``: orthonormal U, V, log-uniform ``s``, N(0, noise_std^2) noise.

    The benchmark's gradient family; generated on the CPU from ``seed`` so that the CPU oracle
    and the GPU path consume identical bits.
    """
    generator = torch.Generator().manual_seed(seed)
    U, _ = torch.linalg.qr(torch.randn(rows, rank, generator=generator, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(columns, rank, generator=generator, dtype=torch.float64))
    low, high = math.log(spectrum[0]), math.log(spectrum[1])
    s = torch.exp(torch.rand(rank, generator=generator, dtype=torch.float64) * (high - low) + low)
    noise = torch.randn(rows, columns, generator=generator, dtype=torch.float32)
    return ((U * s) @ V.T).to(dtype) + noise_std * noise.to(dtype)


# ---- single operations -------------------------------------------------------------------------
def gram_ema(preconditioner: Tensor, gradient: Tensor, beta: float, side: str) -> Tensor:
    """``P.lerp_(G G^T or G^T G, 1 - beta)`` (src/soap_tp/ops/preconditioners.py:367,579,688,739)."""
    if not 0.0 <= beta <= 1.0:
        raise ValueError(f"beta must be in [0, 1], got {beta}.")
    gram = gradient @ gradient.T if side == "left" else gradient.T @ gradient
    return preconditioner.lerp_(gram, 1.0 - beta)


def rotate(matrix: Tensor, q_left: Tensor, q_right: Tensor, direction: str) -> Tensor:
    """``Q_L^T X Q_R`` or ``Q_L X Q_R^T`` with the product order of the binding
    (src/soap_tp/csrc/slate_bindings.cpp:257-273; src/soap_tp/ops/factorizations.py:118-119)."""
    if direction == "forward":
        return (q_left.T @ matrix) @ q_right
    if direction == "backward":
        return (q_left @ matrix) @ q_right.T
    raise ValueError(f"direction must be 'forward' or 'backward', got {direction!r}.")


def adam_update(
    gradient: Tensor, momentum: Tensor, variance: Tensor, step: int, beta1: float, beta2: float, eps: float
) -> Tensor:
    """Same in-place operation order as src/soap_tp/ops/optimizer.py:36-44."""
    if step < 1:
        raise ValueError(f"step must be positive, got {step}.")
    momentum.mul_(beta1).add_(gradient, alpha=1.0 - beta1)
    variance.mul_(beta2).addcmul_(gradient, gradient, value=1.0 - beta2)
    bias_correction1 = 1.0 - beta1**step
    bias_correction2 = 1.0 - beta2**step
    denominator = variance.sqrt().div_(math.sqrt(bias_correction2)).add_(eps)
    return denominator.reciprocal_().mul_(momentum).div_(bias_correction1)


def eigh_descending(preconditioner: Tensor, implementation: str = "elpa") -> Tuple[Tensor, Tensor]:
    """Descending eigenpairs as ``initialize_basis_2d_block_cyclic_`` returns them.

    ``"elpa"``: ascending float64 solve of ``-P``, ``Q = float32(Q64)``, ``eig = -lambda``
    (src/soap_tp/ops/factorizations.py:497-546; ELPA's one-stage solver is replaced by LAPACK's
    symmetric eigensolver, which computes the same decomposition).  ``"eigh"``: float32
    ``eigh(P + 1e-30 I)`` flipped (:453-463).
    """
    size = preconditioner.shape[0]
    if implementation == "elpa":
        values, vectors = torch.linalg.eigh(-preconditioner.to(torch.float64))
        return (-values).to(torch.float32), vectors.to(torch.float32)
    if implementation == "eigh":
        shifted = preconditioner + 1e-30 * torch.eye(size, dtype=preconditioner.dtype)
        values, vectors = torch.linalg.eigh(shifted)
        return values.flip(0), vectors.flip(1)
    raise ValueError(f"implementation must be 'elpa' or 'eigh', got {implementation!r}.")


def estimated_order(preconditioner: Tensor, basis: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """``work = P Q``; ``est = (Q * work).sum(0)``; ``argsort(est, descending)``
    (src/soap_tp/ops/factorizations.py:235-271).  Returns (order, estimates, work)."""
    work = preconditioner @ basis
    estimates = (basis * work).sum(dim=0)
    return torch.argsort(estimates, descending=True, stable=True), estimates, work


def householder_qr(matrix: Tensor) -> Tensor:
    """Explicit orthogonal factor with LAPACK's Householder sign convention, which is what
    SLATE's geqrf + unmqr on the identity produce (src/soap_tp/csrc/slate_bindings.cpp:176-185)."""
    return torch.linalg.qr(matrix).Q


def permute(matrix: Tensor, row_order: Tensor, column_order: Tensor) -> Tensor:
    """``matrix[row_order][:, column_order]`` (src/soap_tp/ops/optimizer.py:408)."""
    return matrix.index_select(0, row_order).index_select(1, column_order)


def power_iteration_qr(preconditioner: Tensor, basis: Tensor) -> Tuple[Tensor, Tensor]:
    """src/soap_tp/ops/factorizations.py:323-360: order, permuted power iterate, QR."""
    order, _, work = estimated_order(preconditioner, basis)
    return order, householder_qr(work.index_select(1, order))


def refresh(state: Dict[str, Tensor]) -> Tuple[Tensor, Tensor]:
    """src/soap_tp/ops/factorizations.py:550-614 on dense matrices (updates ``state`` in place)."""
    momentum = rotate(state["momentum"], state["left_basis"], state["right_basis"], "backward")
    left_order, state["left_basis"] = power_iteration_qr(state["left_preconditioner"], state["left_basis"])
    right_order, state["right_basis"] = power_iteration_qr(state["right_preconditioner"], state["right_basis"])
    state["variance"] = permute(state["variance"], left_order, right_order)
    state["momentum"] = rotate(momentum, state["left_basis"], state["right_basis"], "forward")
    return left_order, right_order


# ---- the step ----------------------------------------------------------------------------------
def soap_step(
    gradient: Tensor,
    state: Dict[str, Tensor],
    *,
    preconditioner_beta: float = 0.95,
    beta1: float = 0.95,
    beta2: float = 0.95,
    eps: float = 1e-8,
    basis_refresh_interval: int = 10,
    basis_implementation: str = "elpa",
    bases_override: Optional[Dict[int, Tuple[Tensor, Tensor]]] = None,
) -> Tensor:
    """Dense restatement of src/soap_tp/soap.py:154-506.

    ``bases_override`` maps a step number to ``(Q_left, Q_right)`` that replace the oracle's
    own bases after that step's initialisation or refresh.  Parity tests use it to compare
    update, moment and Gram arithmetic conditionally on the bases, because eigenvectors inside
    a cluster of nearly equal eigenvalues are not determined by the data to working precision.
    """
    if basis_refresh_interval <= 0:
        raise ValueError("basis_refresh_interval must be positive.")
    if basis_implementation not in {"elpa", "eigh"}:
        raise ValueError(f"basis_implementation must be 'elpa' or 'eigh', got {basis_implementation!r}.")
    rows, columns = gradient.shape
    gradient = gradient.detach().to(torch.float32).contiguous()
    initializing = "left_basis" not in state
    if initializing:
        # soap.py:165-182 allocates zeros; :194-225 forms both Gram matrices from that zero state
        state["left_preconditioner"] = torch.zeros(rows, rows)
        state["right_preconditioner"] = torch.zeros(columns, columns)
        state["momentum"] = torch.zeros(rows, columns)
        state["variance"] = torch.zeros(rows, columns)
        gram_ema(state["left_preconditioner"], gradient, preconditioner_beta, "left")
        gram_ema(state["right_preconditioner"], gradient, preconditioner_beta, "right")
        if bases_override and 0 in bases_override:  # the eigensolves would be discarded: skip them
            state["left_basis"], state["right_basis"] = (t.clone() for t in bases_override[0][:2])
        else:
            _, state["left_basis"] = eigh_descending(state["left_preconditioner"], basis_implementation)
            _, state["right_basis"] = eigh_descending(state["right_preconditioner"], basis_implementation)
        state["step"] = 0
        return torch.zeros_like(gradient)  # soap.py:268-276

    step = int(state["step"]) + 1  # soap.py:278
    projected = rotate(gradient, state["left_basis"], state["right_basis"], "forward")  # :342
    coordinate_update = adam_update(  # :360-368, including the eps rescaling
        projected, state["momentum"], state["variance"], step, beta1, beta2,
        eps / math.sqrt(1.0 - beta2**step),
    )
    update = rotate(coordinate_update, state["left_basis"], state["right_basis"], "backward")  # :393
    gram_ema(state["left_preconditioner"], gradient, preconditioner_beta, "left")  # :425
    gram_ema(state["right_preconditioner"], gradient, preconditioner_beta, "right")  # :441
    if step % basis_refresh_interval == 0:  # :457
        if bases_override and step in bases_override:
            # keep the transport semantics, but land on the supplied bases
            momentum = rotate(state["momentum"], state["left_basis"], state["right_basis"], "backward")
            override = bases_override[step]
            if len(override) == 4:  # caller also supplies the orders that were used
                left_order, right_order = override[2], override[3]
            else:
                left_order, _, _ = estimated_order(state["left_preconditioner"], state["left_basis"])
                right_order, _, _ = estimated_order(state["right_preconditioner"], state["right_basis"])
            state["left_basis"], state["right_basis"] = override[0].clone(), override[1].clone()
            state["variance"] = permute(state["variance"], left_order, right_order)
            state["momentum"] = rotate(momentum, state["left_basis"], state["right_basis"], "forward")
        else:
            refresh(state)
    state["step"] = step  # :505
    return update.contiguous()


def original_soap_reference(
    gradients,
    *,
    preconditioner_beta: float,
    beta1: float,
    beta2: float,
    eps: float,
    basis_refresh_interval: int,
):
    """Updates of the ORIGINAL SOAP optimizer for one 2-D parameter, restated from its control
    flow (tests/reference/soap.py:145-345 ``step``, :401-440 ``update_preconditioner``, :470-503
    ``get_orthogonal_matrix``, :505-562 ``get_orthogonal_matrix_QR``) with lr = 1,
    weight_decay = 0, correct_bias, no gradient normalisation, as tests/unit/test_soap.py:417-438
    configures it.  Unlike ``soap_step`` above, momentum is taken out of and put back into the
    eigenbasis on every step, and the refreshed basis is ``qr(P @ Q[:, order])`` computed after
    reordering ``Q``: a different arrangement of the same mathematics, which is what makes
    agreement between the two a meaningful check of the sequencing.
    """
    updates = []
    L = R = QL = QR = exp_avg = exp_avg_sq = None
    step = 0
    for gradient in gradients:
        gradient = gradient.to(torch.float32)
        if QL is None:
            rows, columns = gradient.shape
            L, R = torch.zeros(rows, rows), torch.zeros(columns, columns)
            exp_avg, exp_avg_sq = torch.zeros_like(gradient), torch.zeros_like(gradient)
            L.lerp_(gradient @ gradient.T, 1 - preconditioner_beta)
            R.lerp_(gradient.T @ gradient, 1 - preconditioner_beta)
            QL = torch.linalg.eigh(L + 1e-30 * torch.eye(rows))[1].flip(1)
            QR = torch.linalg.eigh(R + 1e-30 * torch.eye(columns))[1].flip(1)
            updates.append(torch.zeros_like(gradient))
            continue
        projected = QL.T @ gradient @ QR
        step += 1
        exp_avg.mul_(beta1).add_(projected, alpha=1.0 - beta1)
        exp_avg_sq.mul_(beta2).add_(projected.square(), alpha=1.0 - beta2)
        denom = exp_avg_sq.sqrt().add_(eps)
        step_size = math.sqrt(1.0 - beta2**step) / (1.0 - beta1**step)
        updates.append((QL @ (exp_avg / denom) @ QR.T) * step_size)
        # update_preconditioner: momentum leaves the basis, Gram EMA, optional QR refresh, re-entry
        exp_avg = QL @ exp_avg @ QR.T
        L.lerp_(gradient @ gradient.T, 1 - preconditioner_beta)
        R.lerp_(gradient.T @ gradient, 1 - preconditioner_beta)
        if step % basis_refresh_interval == 0:
            new_bases = []
            for dim, (P, Q) in enumerate(((L, QL), (R, QR))):
                estimates = torch.diag(Q.T @ P @ Q)
                order = torch.argsort(estimates, descending=True, stable=True)
                exp_avg_sq = exp_avg_sq.index_select(dim, order)
                new_bases.append(torch.linalg.qr(P @ Q[:, order])[0])
            QL, QR = new_bases
        exp_avg = QL.T @ exp_avg @ QR
    return updates
