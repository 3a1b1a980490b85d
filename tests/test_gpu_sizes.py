"""Parity at the sizes the benchmark runs: 4096 x 4096, 4096 x 11008, 8192 x 3584 (refresh every 5)
and one transformer layer's parameter set (4096 x 4096, 4096 x 14336, 14336 x 4096), the sizes the
reference's own accuracy sweep reaches (scripts/slurm/frontier/soap_accuracy.slurm:62-68: 8 ... 8192,
both ``eigh`` and ``elpa``).

What is compared, and why in this form:

* update, momentum, variance and both Gram matrices against the CPU oracle, conditionally on the
  GPU's bases and sort orders (relative Frobenius error <= 1e-4): eigenvectors inside the noise
  bulk of a low-rank-plus-noise Gram matrix are not determined to working precision by the data,
  and Adam normalises element-wise in that basis, so two correct eigensolvers give different
  updates; conditionally on the bases every product, the Adam arithmetic, the transport and the
  Gram accumulation are pinned;
* the bases themselves on the device, in float64: eigen-residual ``|P Q - Q diag(rho)|_F <=
  1e-5 |P|_F``, Rayleigh quotients against LAPACK's eigenvalues computed on the CPU (error <=
  1e-5 lambda_max, the bar stated for this build), orthogonality, descending order, and the angle
  of the signal subspace bounded through the residual of its block over the spectral gap
  (Davis-Kahan) <= 1e-3;
* the refresh's factorisation on the state the run produced: ``P Q`` against a float64 product,
  the sort order against the estimates it was computed from, and the QR of the permuted power
  iterate by orthogonality, ``Q^T W`` upper triangular, the backward error of ``W = Q R`` (norm-wise
  and per column) and the span of the leading columns.
"""
import pytest
import torch

import soap_tp_amd
from oracle import soap_oracle as oracle
from soap_tp_amd import ops
from soap_tp_amd import soap as soap_module
from tests.helpers import SEED, relative_l2

pytestmark = pytest.mark.gpu
GRID = (1, 1)
BLOCK = 128
TOL = 1e-4
HYPER = dict(preconditioner_beta=0.95, beta1=0.95, beta2=0.95, eps=1e-8)


def _full(lower):
    """Both triangles of a Gram matrix that is kept up to date in its lower triangle only."""
    return torch.tril(lower) + torch.tril(lower, -1).T


def _relative(actual, reference):
    """Relative Frobenius error, computed where ``actual`` lives (float64)."""
    reference = reference.to(actual.device, torch.float64)
    return ((actual.double() - reference).norm() / reference.norm().clamp_min(1e-300)).item()


def check_eigenbasis(gram, basis, signal_rank, cpu_eigenvalues=True, residual_tol=1e-5):
    """Invariants of a descending eigenbasis ``basis`` of the symmetric ``gram`` (device tensors).
    ``residual_tol`` is 1e-5 for the float64 solver; the float32 variant gets 5e-5 (LAPACK's float32
    solver leaves 8e-6 on the 4096 x 4096 matrix of this test, this build's 1.8e-5)."""
    size = gram.shape[0]
    p = gram.double()
    q = basis.double()
    pq = p @ q
    rho = (q * pq).sum(dim=0)
    scale = rho.abs().max().item()
    residual = pq - q * rho
    assert (residual.norm() / p.norm()).item() <= residual_tol
    identity_error = q.T @ q
    identity_error.diagonal().sub_(1.0)
    assert identity_error.abs().max().item() <= 1e-4
    assert torch.all(rho[:-1] >= rho[1:] - 1e-5 * scale)
    # The leading block up to the widest spectral gap among the first `signal_rank` eigenvalues (the
    # weakest signal directions lie inside the noise bulk, so the cut is placed where the spectrum
    # separates): sin(angle to the exact invariant subspace) <= |residual of the block| / gap.
    gaps = rho[:signal_rank] - rho[1:signal_rank + 1]
    cut = int(torch.argmax(gaps).item()) + 1
    gap = gaps[cut - 1].item()
    assert gap > 0
    assert residual[:, :cut].norm().item() / gap <= 1e-3
    del pq, residual, identity_error
    if cpu_eigenvalues:
        if size <= 4096:
            exact, vectors = torch.linalg.eigh(p.cpu())
            exact, vectors = exact.flip(0), vectors.flip(1)
            mine = q[:, :cut].cpu()
            difference = mine @ mine.T - vectors[:, :cut] @ vectors[:, :cut].T
            assert torch.linalg.matrix_norm(difference, ord=2).item() <= 1e-3
        else:
            exact = torch.linalg.eigvalsh(p.cpu()).flip(0)
        assert (rho.cpu() - exact).abs().max().item() <= 1e-5 * exact.abs().max().item()
    return rho


def check_power_iteration_and_qr(gram, basis, signal_rank, device):
    """One power iteration + QR (the refresh of one side) on the given state, step by step."""
    size = gram.shape[0]
    work = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    order = ops.estimated_eigenvalue_order_2d_block_cyclic_(gram, basis, work, size, BLOCK, GRID)
    exact_work = gram.double() @ basis.double()
    assert _relative(work, exact_work) <= 1e-5
    estimates = (basis.double() * exact_work).sum(dim=0)
    del exact_work
    assert torch.equal(torch.sort(order).values, torch.arange(size, device=device))
    sorted_estimates = estimates[order]
    scale = estimates.abs().max().item()
    # the order was computed from float32 estimates: descending up to their rounding error
    assert torch.all(sorted_estimates[:-1] >= sorted_estimates[1:] - 1e-5 * scale)
    ops.permute_2d_block_cyclic_(work, (size, size), torch.arange(size, device=device), order, BLOCK, GRID,
                                 validate=False)
    iterate = work.clone()
    factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    ops.qr_2d_block_cyclic_(work, factor, size, BLOCK, GRID)
    del work
    assert torch.isfinite(factor).all()
    q = factor.double()
    w = iterate.double()
    identity_error = q.T @ q
    identity_error.diagonal().sub_(1.0)
    assert identity_error.abs().max().item() <= 1e-4
    del identity_error
    r = q.T @ w
    assert (torch.tril(r, -1).norm() / w.norm()).item() <= 1e-5  # Q^T W is upper triangular
    backward = w - q @ torch.triu(r)
    assert (backward.norm() / w.norm()).item() <= 1e-5
    column_norms = w.norm(dim=0)
    sizeable = column_norms >= 1e-6 * column_norms.max()
    assert (backward.norm(dim=0)[sizeable] / column_norms[sizeable]).max().item() <= 5e-5
    # span(Q[:, :k]) = span(W[:, :k]) for the signal block
    lead_q, lead_w = q[:, :signal_rank], w[:, :signal_rank]
    outside = lead_w - lead_q @ (lead_q.T @ lead_w)
    assert (outside.norm() / lead_w.norm()).item() <= 1e-5
    return order


def run_recorded(gradients, device, monkeypatch, interval, implementation="elpa", shard_dim=1, shape=None):
    """soap_step over ``gradients`` (CPU tensors); returns updates (CPU), the final state and the
    bases after the initialisation and after every refresh (with that refresh's orders)."""
    original = soap_module.refresh_bases_and_transport_optimizer_state_
    seen = {}

    def recording(*args, **kwargs):
        orders = original(*args, **kwargs)
        seen["orders"] = tuple(order.cpu() for order in orders)
        return orders

    monkeypatch.setattr(soap_module, "refresh_bases_and_transport_optimizer_state_", recording)
    shape = shape or tuple(gradients[0].shape)
    state, updates, bases = {}, [], {}
    for gradient in gradients:
        seen.pop("orders", None)
        update = soap_tp_amd.soap_step(gradient.to(device), state, global_shape=shape, shard_dim=shard_dim,
                                       block_size=BLOCK, process_grid_shape=GRID, basis_refresh_interval=interval,
                                       basis_implementation=implementation, **HYPER)
        updates.append(update.cpu())
        step = int(state["step"])
        if step == 0 or "orders" in seen:
            bases[step] = (state["left_basis"].cpu().clone(), state["right_basis"].cpu().clone()) + seen.get("orders", ())
    return updates, state, bases


def assert_conditional_parity(gradients, updates, state, bases, interval, implementation="elpa"):
    oracle_state = {}
    for iteration, gradient in enumerate(gradients):
        expected = oracle.soap_step(gradient, oracle_state, bases_override=bases, basis_refresh_interval=interval,
                                    basis_implementation=implementation, **HYPER)
        if iteration == 0:
            assert torch.count_nonzero(updates[0]) == 0
        else:
            error = relative_l2(updates[iteration], expected)
            assert error <= TOL, f"update of iteration {iteration}: {error}"
    assert int(state["step"]) == int(oracle_state["step"]) == len(gradients) - 1
    for name in ("momentum", "variance"):
        assert _relative(state[name], oracle_state[name]) <= TOL, name
    for side in ("left", "right"):
        name = f"{side}_preconditioner"
        assert _relative(_full(state[name]), oracle_state[name]) <= TOL, name


@pytest.mark.parametrize("shape,rank,implementation", [
    ((4096, 4096), 64, "elpa"),
    ((4096, 4096), 64, "eigh"),
    ((4096, 11008), 128, "elpa"),
])
def test_step_and_bases_at_benchmark_sizes(shape, rank, implementation, device, monkeypatch):
    """Initialisation, a plain step, a refresh step and a step in the refreshed bases."""
    rows, columns = shape
    gradients = [oracle.low_rank_plus_noise(rows, columns, rank, seed=SEED + t) for t in range(4)]
    # the initial bases against the Gram matrices they were computed from
    state = {}
    soap_tp_amd.soap_step(gradients[0].to(device), state, global_shape=shape, shard_dim=1, block_size=BLOCK,
                          process_grid_shape=GRID, basis_refresh_interval=2, basis_implementation=implementation,
                          **HYPER)
    for side in ("left", "right"):
        check_eigenbasis(_full(state[f"{side}_preconditioner"]), state[f"{side}_basis"], rank,
                         residual_tol=1e-5 if implementation == "elpa" else 5e-5)
    del state
    updates, state, bases = run_recorded(gradients, device, monkeypatch, interval=2, implementation=implementation)
    assert sorted(bases) == [0, 2] and len(bases[2]) == 4
    assert_conditional_parity(gradients, updates, state, bases, 2, implementation)
    for side, size in (("left", rows), ("right", columns)):
        q = state[f"{side}_basis"].double()
        identity_error = q.T @ q
        identity_error.diagonal().sub_(1.0)
        assert identity_error.abs().max().item() <= 1e-4


SWEEP = [(size, implementation) for size in (16, 32, 64, 128, 256, 512, 2048) for implementation in ("elpa", "eigh")]


@pytest.mark.parametrize("size,implementation", SWEEP + [(8192, "elpa"), (8192, "eigh")])
def test_square_sizes_of_the_reference_accuracy_sweep(size, implementation, device, monkeypatch):
    """The square sizes of the reference's accuracy sweep that no other test runs
    (scripts/slurm/frontier/soap_accuracy.slurm:62-68: 8 ... 8192, both variants; 8, 1024 and 4096 are
    covered elsewhere): initialisation, plain steps and a refresh step, conditionally on the bases."""
    rank = max(2, min(64, size // 8))
    count = 3 if size >= 8192 else 5
    gradients = [oracle.low_rank_plus_noise(size, size, rank, seed=SEED + size + t) for t in range(count)]
    updates, state, bases = run_recorded(gradients, device, monkeypatch, interval=2, implementation=implementation)
    assert sorted(bases) == ([0, 2] if count == 3 else [0, 2, 4])
    assert_conditional_parity(gradients, updates, state, bases, 2, implementation)
    for side in ("left", "right"):
        q = state[f"{side}_basis"].double()
        identity_error = q.T @ q
        identity_error.diagonal().sub_(1.0)
        assert identity_error.abs().max().item() <= 1e-4


@pytest.mark.parametrize("shape,rank", [((4096, 4096), 64), ((4096, 11008), 128)])
def test_refresh_factorisation_at_benchmark_sizes(shape, rank, device):
    """P Q, the order and the QR of a refresh, on the state after three Gram updates."""
    rows, columns = shape
    state = {}
    for t in range(3):
        gradient = oracle.low_rank_plus_noise(rows, columns, rank, seed=SEED + t).to(device)
        soap_tp_amd.soap_step(gradient, state, global_shape=shape, shard_dim=1, block_size=BLOCK,
                              process_grid_shape=GRID, basis_refresh_interval=10, **HYPER)
    for side in ("left", "right"):
        gram = ops.allocate_2d_block_cyclic(state[f"{side}_preconditioner"].shape, BLOCK, GRID, device=device)
        gram.copy_(_full(state[f"{side}_preconditioner"]))
        check_power_iteration_and_qr(gram, state[f"{side}_basis"], rank, device)
        del gram


def test_shard_dim_0_equals_shard_dim_1_at_4096x11008(device, monkeypatch):
    """On one rank the shard is the whole matrix whichever dimension it was cut along: the results
    must be the same bit for bit (the benchmark's third configuration asks for both)."""
    shape = (4096, 11008)
    gradients = [oracle.low_rank_plus_noise(*shape, 128, seed=SEED + t) for t in range(3)]
    results = []
    for shard_dim in (1, 0):
        updates, state, _ = run_recorded(gradients, device, monkeypatch, interval=2, shard_dim=shard_dim)
        results.append((updates, {name: state[name].clone() for name in soap_module.STATE_BUFFERS}))
        monkeypatch.undo()
        del state
    for first, second in zip(results[0][0], results[1][0]):
        assert torch.equal(first, second)
    for name in soap_module.STATE_BUFFERS:
        assert torch.equal(results[0][1][name], results[1][1][name]), name


def test_config_8192x3584_refresh_every_5(device, monkeypatch):
    """The refresh-heavy configuration: 8192 x 3584, rank 128, refresh every 5; ten steps, two refreshes."""
    shape = (8192, 3584)
    gradients = [oracle.low_rank_plus_noise(*shape, 128, seed=SEED + t) for t in range(11)]
    updates, state, bases = run_recorded(gradients, device, monkeypatch, interval=5)
    assert sorted(bases) == [0, 5, 10]
    assert_conditional_parity(gradients, updates, state, bases, 5)
    # the initial bases: recompute the first Gram matrices on the device and check the eigenpairs
    first = gradients[0].to(device)
    for side, gram in (("left", 0.05 * (first @ first.T)), ("right", 0.05 * (first.T @ first))):
        index = 0 if side == "left" else 1
        check_eigenbasis(gram, bases[0][index].to(device), 128)
    # and the factorisation of a refresh on the final state
    for side in ("left", "right"):
        gram = ops.allocate_2d_block_cyclic(state[f"{side}_preconditioner"].shape, BLOCK, GRID, device=device)
        gram.copy_(_full(state[f"{side}_preconditioner"]))
        check_power_iteration_and_qr(gram, state[f"{side}_basis"], 128, device)
        del gram


def test_config_4096x4096_full_schedule(device, monkeypatch):
    """The second benchmark configuration at its full length: 4096 x 4096, rank 64, 50 steps after the
    initialising call, a refresh every 10 (five refreshes).  Every iteration's update is compared with
    the oracle given the device's bases, as the reference's end-to-end test follows every iteration
    of its schedule (tests/unit/test_soap.py:715-817); moments and Gram matrices at the end."""
    shape = (4096, 4096)
    gradients = [oracle.low_rank_plus_noise(*shape, 64, seed=SEED + 500 + t) for t in range(51)]
    updates, state, bases = run_recorded(gradients, device, monkeypatch, interval=10)
    assert sorted(bases) == [0, 10, 20, 30, 40, 50]
    assert_conditional_parity(gradients, updates, state, bases, 10)
    for side in ("left", "right"):
        q = state[f"{side}_basis"].double()
        identity_error = q.T @ q
        identity_error.diagonal().sub_(1.0)
        assert identity_error.abs().max().item() <= 1e-4


def test_config_4096x11008_two_refresh_cycles(device, monkeypatch):
    """The third benchmark configuration at its real cadence: 4096 x 11008, rank 128, a refresh every 10,
    twenty steps after the initialising call (two refreshes; the configuration's full fifty would keep the
    CPU oracle busy for several minutes).  Every iteration's update against the oracle given the
    device's bases; moments and Gram matrices at the end."""
    shape = (4096, 11008)
    gradients = [oracle.low_rank_plus_noise(*shape, 128, seed=SEED + 700 + t) for t in range(21)]
    updates, state, bases = run_recorded(gradients, device, monkeypatch, interval=10)
    assert sorted(bases) == [0, 10, 20]
    assert_conditional_parity(gradients, updates, state, bases, 10)


LAYER = (("q", (4096, 4096)), ("k", (4096, 4096)), ("v", (4096, 4096)), ("o", (4096, 4096)),
         ("gate", (4096, 14336)), ("up", (4096, 14336)), ("down", (14336, 4096)))


def test_layer_parameter_set_through_the_optimizer(device, monkeypatch):
    """The benchmark's fifth configuration with fewer steps: seven parameters of one transformer
    layer, a state each, stepped through ``SOAP`` (lr 1, no weight decay, so a parameter moves by
    minus the update); initialisation, a plain step, a refresh step.  One
    parameter of each shape is compared with the oracle conditionally on its bases; all are
    checked for the invariants of their bases."""
    original = soap_module.refresh_bases_and_transport_optimizer_state_
    refreshed = {}

    def recording(momentum, *args, **kwargs):
        orders = original(momentum, *args, **kwargs)
        refreshed[momentum.data_ptr()] = orders
        return orders

    monkeypatch.setattr(soap_module, "refresh_bases_and_transport_optimizer_state_", recording)
    parameters = {name: torch.nn.Parameter(torch.zeros(shape, device=device)) for name, shape in LAYER}
    optimizer = soap_tp_amd.SOAP(parameters.values(), lr=1.0, betas=(0.95, 0.95), eps=1e-8, weight_decay=0.0,
                                 precondition_frequency=2, block_size=BLOCK)
    compared = ("q", "gate", "down")
    gradients = {name: [] for name in compared}
    moved = {name: [] for name in compared}
    bases = {name: {} for name in compared}
    refreshes = 0
    for t in range(3):
        refreshed.clear()
        before = {name: parameters[name].detach().clone() for name in compared}
        for index, (name, shape) in enumerate(LAYER):
            gradient = oracle.low_rank_plus_noise(*shape, 64, seed=SEED + 1000 * index + t)
            if name in compared:
                gradients[name].append(gradient)
            parameters[name].grad = gradient.to(device)
        optimizer.step()
        for name in compared:
            soap_state = optimizer.state[parameters[name]]["soap"]
            moved[name].append((before[name] - parameters[name].detach()).cpu())
            orders = refreshed.get(soap_state["momentum"].data_ptr())
            if t == 0 or orders is not None:
                entry = (soap_state["left_basis"].cpu().clone(), soap_state["right_basis"].cpu().clone())
                if orders is not None:
                    entry = entry + tuple(order.cpu() for order in orders)
                bases[name][int(soap_state["step"])] = entry
        refreshes += len(refreshed)
        del before
    assert refreshes == len(LAYER)  # every parameter refreshed once, on its second step
    for name in compared:
        assert sorted(bases[name]) == [0, 2]
        assert_conditional_parity(gradients[name], moved[name], optimizer.state[parameters[name]]["soap"],
                                  bases[name], 2)
    for name, shape in LAYER:
        soap_state = optimizer.state[parameters[name]]["soap"]
        assert int(soap_state["step"]) == 2
        for side in ("left", "right"):
            q = soap_state[f"{side}_basis"].double()
            identity_error = q.T @ q
            identity_error.diagonal().sub_(1.0)
            assert identity_error.abs().max().item() <= 1e-4
            del q, identity_error


@pytest.mark.parametrize("shape", [(4096, 14336), (14336, 4096)])
def test_bases_and_refresh_at_14336(shape, device):
    """Eigenbasis and refresh factorisation with a 14336-wide side (more than 8192 rows in the
    variance permutation, 56 workgroups in the factorisations' panel kernels)."""
    rows, columns = shape
    state = {}
    for t in range(2):
        gradient = oracle.low_rank_plus_noise(rows, columns, 64, seed=SEED + t).to(device)
        soap_tp_amd.soap_step(gradient, state, global_shape=shape, shard_dim=1, block_size=BLOCK,
                              process_grid_shape=GRID, basis_refresh_interval=10, **HYPER)
        if t == 0:
            side = "left" if rows > columns else "right"
            check_eigenbasis(_full(state[f"{side}_preconditioner"]), state[f"{side}_basis"], 64)
    # variance permutation with more than 8192 rows / columns against index_select
    variance = state["variance"]
    expected = variance.clone()
    generator = torch.Generator().manual_seed(SEED)
    row_order = torch.randperm(rows, generator=generator).to(device)
    column_order = torch.randperm(columns, generator=generator).to(device)
    ops.permute_2d_block_cyclic_(variance, shape, row_order, column_order, BLOCK, GRID)
    assert torch.equal(variance, expected.index_select(0, row_order).index_select(1, column_order))
    del expected
    side = "left" if rows > columns else "right"
    gram = ops.allocate_2d_block_cyclic(state[f"{side}_preconditioner"].shape, BLOCK, GRID, device=device)
    gram.copy_(_full(state[f"{side}_preconditioner"]))
    check_power_iteration_and_qr(gram, state[f"{side}_basis"], 64, device)


def test_two_stage_eigensolver_at_4096(device):
    """The two-stage tridiagonalisation (option "eigh_algorithm" = 2) on the 4096 x 4096 Gram matrix of
    the benchmark's second configuration, through the basis initialisation: the same invariants as the
    default solver has to meet, and the same eigenvalues."""
    from soap_tp_amd import _native

    size, rank = 4096, 64
    gradient = oracle.low_rank_plus_noise(size, size, rank, seed=SEED).to(device)
    gram = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    gram.copy_(0.05 * gradient @ gradient.T)
    spectra = []
    try:
        for algorithm in (1, 2):
            _native.call("soapmi_set_option", b"eigh_algorithm", algorithm)
            basis = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            work = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            values = torch.empty(size, dtype=torch.float32, device=device)
            ops.initialize_basis_2d_block_cyclic_(gram, basis, work, values, size, BLOCK, GRID, implementation="elpa")
            check_eigenbasis(gram, basis, rank, cpu_eigenvalues=(algorithm == 2))
            spectra.append(values.clone())
    finally:
        _native.call("soapmi_set_option", b"eigh_algorithm", 1)
    assert (spectra[0] - spectra[1]).abs().max().item() <= 1e-6 * spectra[0].abs().max().item()


@pytest.mark.parametrize("size,width", [(8192, 1024), (4096, 256)])
def test_qr_blocking_not_chosen_by_default_at_size(size, width, device):
    """The QR blocking the library does not pick by itself at this size (three levels above 4096, two
    up to 4096): orthogonality, triangularity of Q^T W and backward error on a graded matrix."""
    from soap_tp_amd import _native
    generator = torch.Generator().manual_seed(4242 + size)
    matrix = (torch.randn(size, size, generator=generator) * torch.logspace(0, -6, size)[None, :]).to(device)
    iterate = matrix.T.contiguous().T.clone()  # column-major copy
    work = iterate.clone()
    factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    try:
        _native.call("soapmi_set_option", b"qr_super_block", width)
        ops.qr_2d_block_cyclic_(work, factor, size, BLOCK, GRID)
    finally:
        _native.call("soapmi_set_option", b"qr_super_block", 0)
    del work
    assert torch.isfinite(factor).all()
    q, w = factor.double(), iterate.double()
    identity_error = q.T @ q
    identity_error.diagonal().sub_(1.0)
    assert identity_error.abs().max().item() <= 1e-4
    del identity_error
    r = q.T @ w
    assert (torch.tril(r, -1).norm() / w.norm()).item() <= 1e-5
    backward = w - q @ torch.triu(r)
    assert (backward.norm(dim=0) / w.norm(dim=0)).max().item() <= 5e-5


def test_qr_with_more_workgroups_in_a_launch_than_compute_units(device):
    """n = 16640: a panel launch holds 65 panel workgroups and up to 195 workgroups that update the columns
    behind the panel for the previous one, more than the chip's 256 compute units hold at once.  The
    updating workgroups come first in the launch and wait for nobody, so the panel's own workgroups are
    all placed once those have finished.  Checked by properties (a CPU factorisation of this size takes
    minutes): orthogonality on a sample of columns, ``Q^T A`` upper triangular and the backward error of
    the leading columns."""
    size = 16640
    generator = torch.Generator(device=device).manual_seed(SEED + size)
    matrix = torch.randn(size, size, device=device, generator=generator).T  # column-major
    work = matrix.clone()
    factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    ops.qr_2d_block_cyclic_(work, factor, size, BLOCK, GRID)
    torch.cuda.synchronize()
    assert not soap_tp_amd._native.device_error_flag()
    sample = torch.cat([torch.arange(0, 256), torch.arange(size // 2, size // 2 + 256),
                        torch.arange(size - 256, size)]).to(device)
    q_sample = factor[:, sample].double()
    identity = torch.eye(sample.numel(), dtype=torch.float64, device=device)
    assert (q_sample.T @ q_sample - identity).abs().max().item() <= 1e-5
    lead = 512
    r_lead = factor[:, :lead].double().T @ matrix[:, :lead].double()
    assert torch.tril(r_lead, -1).abs().max().item() <= 1e-5 * r_lead.abs().max().item()
    residual = factor[:, :lead].double() @ torch.triu(r_lead) - matrix[:, :lead].double()
    assert residual.norm().item() <= 1e-5 * matrix[:, :lead].double().norm().item()


def test_lost_messages_with_more_than_32_workgroups(device):
    """n = 8704: 34 workgroups per panel launch, the size from which the Gram values travel in two
    levels (shares summed by their owners, totals fetched by everybody).  With no patience for
    another workgroup's message (spin limit 0) every wait of both levels must give up, leave the
    kernel and poison Q, or, if every message happened to be there at the first poll, give a correct
    Q; the next factorisation with the default limit is clean."""
    from soap_tp_amd import _native
    size = 8704
    generator = torch.Generator(device=device).manual_seed(SEED + size)
    matrix = torch.randn(size, size, device=device, generator=generator).T

    def run():
        factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
        ops.qr_2d_block_cyclic_(matrix.clone(), factor, size, BLOCK, GRID)
        torch.cuda.synchronize()
        return factor

    def orthogonality(factor):
        sample = factor[:, -384:].double()
        return (sample.T @ sample - torch.eye(384, dtype=torch.float64, device=device)).abs().max().item()

    assert not _native.device_error_flag(clear=True)
    try:
        _native.call("soapmi_set_option", b"message_spin_limit", 0)
        factor = run()
    finally:
        _native.call("soapmi_set_option", b"message_spin_limit", 1 << 22)
        reported = _native.device_error_flag(clear=True)
    poisoned = bool(torch.isnan(factor).any())
    assert poisoned or orthogonality(factor) <= 1e-5
    assert reported == poisoned
    factor = run()
    assert torch.isfinite(factor).all() and orthogonality(factor) <= 1e-5
    assert not _native.device_error_flag(clear=True)
