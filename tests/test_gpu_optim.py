"""The optimizer wrapper, checkpoint helpers and profile comparer on the GPU.

The wrapper is checked against the golden trajectory of the original optimizer (the reference's
ground truth, tests/reference/soap.py of the reference checkout, lr = 1, weight_decay = 0), against
closed-form AdamW arithmetic for vectors, for independence of the stream pool, and for exact
continuation after a checkpoint round trip.  Bar: relative Frobenius error <= 1e-4."""
import io
import math
from pathlib import Path

import numpy as np
import pytest
import torch

import soap_tp_amd
from oracle import soap_oracle as oracle
from soap_tp_amd import _profile, compare_profiles, state_io
from soap_tp_amd.optim import SOAP
from tests.helpers import SEED, relative_l2

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden" / "soap_trajectory.npz"
TOL = 1e-4


@pytest.mark.parametrize("shape", [(8, 8), (12, 12)])
def test_wrapper_follows_the_original_optimizer(shape, device):
    golden = np.load(GOLDEN)
    gradients = torch.from_numpy(golden[f"gradients_{shape[0]}x{shape[1]}"])
    updates = torch.from_numpy(golden[f"updates_{shape[0]}x{shape[1]}"])
    parameter = torch.nn.Parameter(torch.zeros(shape, device=device))
    optimizer = SOAP([parameter], lr=1.0, betas=(0.8, 0.9), shampoo_beta=0.75, eps=1e-6, weight_decay=0.0,
                     precondition_frequency=2, basis_implementation="eigh", block_size=2)
    expected = torch.zeros(shape, dtype=torch.float64)
    for iteration in range(gradients.shape[0]):
        parameter.grad = gradients[iteration].to(device)
        optimizer.step()
        expected -= updates[iteration].double()
        if iteration == 0:
            assert torch.count_nonzero(parameter) == 0  # the first gradient only initialises state
        if iteration >= 2:
            assert relative_l2(parameter.detach().cpu().double(), expected) <= TOL, f"iteration {iteration}"


def test_learning_rate_and_decoupled_weight_decay(device):
    shape = (8, 8)
    golden = np.load(GOLDEN)
    gradients = torch.from_numpy(golden["gradients_8x8"])
    updates = torch.from_numpy(golden["updates_8x8"]).double()
    lr, decay = 0.05, 0.1
    start = torch.linspace(-1, 1, 64).reshape(shape)
    parameter = torch.nn.Parameter(start.clone().to(device))
    optimizer = SOAP([parameter], lr=lr, betas=(0.8, 0.9), shampoo_beta=0.75, eps=1e-6, weight_decay=decay,
                     precondition_frequency=2, basis_implementation="eigh", block_size=2)
    expected = start.double()
    for iteration in range(6):
        parameter.grad = gradients[iteration].to(device)
        optimizer.step()
        if iteration > 0:  # p -= lr * update, then p -= lr * wd * p
            expected = expected - lr * updates[iteration]
            expected = expected - lr * decay * expected
    assert relative_l2(parameter.detach().cpu().double(), expected) <= TOL


def test_vectors_get_bias_corrected_adam_with_the_first_step_skipped(device):
    generator = torch.Generator().manual_seed(SEED)
    beta1, beta2, eps, lr, decay = 0.9, 0.95, 1e-8, 0.01, 0.1
    start = torch.randn(37, generator=generator)
    parameter = torch.nn.Parameter(start.clone().to(device))
    scalar = torch.nn.Parameter(torch.tensor(0.5, device=device))
    optimizer = SOAP([parameter, scalar], lr=lr, betas=(beta1, beta2), eps=eps, weight_decay=decay)
    p = start.double()
    m = torch.zeros(37, dtype=torch.float64)
    v = torch.zeros(37, dtype=torch.float64)
    for iteration in range(5):
        gradient = torch.randn(37, generator=generator)
        parameter.grad = gradient.to(device)
        scalar.grad = torch.tensor(1.0, device=device)
        optimizer.step()
        if iteration == 0:
            assert torch.equal(parameter.detach().cpu(), start)
            continue
        g = gradient.double()
        m = beta1 * m + (1 - beta1) * g
        v = beta2 * v + (1 - beta2) * g * g
        step_size = lr * math.sqrt(1 - beta2 ** iteration) / (1 - beta1 ** iteration)
        p = p - step_size * m / (v.sqrt() + eps)
        p = p - lr * decay * p
    assert relative_l2(parameter.detach().cpu().double(), p) <= 1e-5
    assert scalar.item() < 0.5  # moved against a positive gradient


def _model(device, seed=3):
    generator = torch.Generator().manual_seed(seed)
    shapes = [(48, 32), (16, 40), (24,), (32, 32), (2, 3, 8)]
    return [torch.nn.Parameter(torch.randn(shape, generator=generator).to(device)) for shape in shapes]


def _gradients(parameters, iteration):
    generator = torch.Generator().manual_seed(100 + iteration)
    return [torch.randn(p.shape, generator=generator).to(p.device) for p in parameters]


def _train(parameters, optimizer, iterations, first=0):
    for iteration in range(first, first + iterations):
        for p, g in zip(parameters, _gradients(parameters, iteration)):
            p.grad = g
        optimizer.step()


def test_stream_pool_does_not_change_results(device):
    serial, pooled = _model(device), _model(device)
    kwargs = dict(lr=0.01, precondition_frequency=3, basis_implementation="eigh", block_size=8, flatten_nd=True)
    _train(serial, SOAP(serial, streams=0, **kwargs), 8)
    _train(pooled, SOAP(pooled, streams=3, **kwargs), 8)
    torch.cuda.synchronize()
    for a, b in zip(serial, pooled):
        assert torch.equal(a.detach().cpu(), b.detach().cpu())


def test_checkpoint_round_trip_continues_bit_exactly(device):
    kwargs = dict(lr=0.01, precondition_frequency=3, basis_implementation="elpa", block_size=8, flatten_nd=True)
    straight = _model(device)
    _train(straight, SOAP(straight, **kwargs), 9)

    resumed = _model(device)
    optimizer = SOAP(resumed, **kwargs)
    _train(resumed, optimizer, 4)
    buffer = io.BytesIO()
    torch.save(optimizer.state_dict(), buffer)
    buffer.seek(0)
    saved = torch.load(buffer, weights_only=True)
    fresh = SOAP(resumed, **kwargs)
    fresh.load_state_dict(saved)
    for p in resumed:
        if p.ndim >= 2:
            state_io.validate_state(fresh.state[p]["soap"])
    _train(resumed, fresh, 5, first=4)
    torch.cuda.synchronize()
    for a, b in zip(straight, resumed):
        assert torch.equal(a.detach().cpu(), b.detach().cpu())


def test_state_helpers_on_device(device, tmp_path):
    shape = (24, 40)
    state = {}
    gradients = [oracle.low_rank_plus_noise(*shape, 4, seed=s).to(device) for s in range(5)]
    kwargs = dict(global_shape=shape, shard_dim=1, block_size=8, process_grid_shape=(1, 1), basis_refresh_interval=2)
    for gradient in gradients[:3]:
        soap_tp_amd.soap_step(gradient, state, **kwargs)
    # saved between two refreshes (step 2 refreshed, step 3 has not happened): the state's upper
    # triangles are stale, the file's Gram matrices must be symmetric all the same
    soap_tp_amd.soap_step(gradients[3], state, **kwargs)
    state_io.save_state(state, tmp_path / "state.pt")
    raw = torch.load(tmp_path / "state.pt", weights_only=True)
    for side in ("left", "right"):
        saved = raw[f"{side}_preconditioner"]
        assert torch.equal(saved, saved.T)
        assert torch.equal(torch.tril(saved), torch.tril(state[f"{side}_preconditioner"].cpu()))
        assert not torch.equal(state[f"{side}_preconditioner"], state[f"{side}_preconditioner"].T)
    clone = state_io.load_state(tmp_path / "state.pt", device=device)
    assert state_io.validate_state(clone, shape) == shape
    a = soap_tp_amd.soap_step(gradients[4], state, **kwargs)  # a refresh step: reads the Gram matrices
    b = soap_tp_amd.soap_step(gradients[4], clone, **kwargs)
    assert torch.equal(a, b) and clone["step"] == state["step"] == 4
    assert torch.equal(clone["left_basis"], state["left_basis"]) and torch.equal(clone["right_basis"], state["right_basis"])


def test_profile_dump_diffs_clean_against_the_oracle(device, monkeypatch, capfd, tmp_path):
    """SOAP_PROFILE lines of a GPU run against the same stages written from the oracle's state."""
    shape = (12, 12)
    config = dict(preconditioner_beta=0.75, beta1=0.8, beta2=0.9, eps=1e-6, basis_refresh_interval=2)
    generator = torch.Generator().manual_seed(SEED + 1)
    gradients = [torch.normal(0, 2, size=shape, generator=generator) for _ in range(5)]
    monkeypatch.setenv("SOAP_PROFILE", "1")
    state = {}
    capfd.readouterr()
    for gradient in gradients:
        soap_tp_amd.soap_step(gradient.to(device), state, global_shape=shape, shard_dim=1, block_size=4,
                              process_grid_shape=(1, 1), basis_implementation="eigh", **config)
    candidate_text = capfd.readouterr().out
    monkeypatch.delenv("SOAP_PROFILE")
    assert candidate_text.count(compare_profiles.MARKER) > 40

    reference_lines = []
    oracle_state = {}

    def emit(stage, step, tensor):
        reference_lines.append(compare_profiles.MARKER + __import__("json").dumps(
            {"impl": "reference", "step": step, "stage": stage, "shape": list(tensor.shape),
             "values": tensor.reshape(-1).tolist()}))

    for gradient in gradients:
        profile_step = 0 if "left_basis" not in oracle_state else int(oracle_state["step"]) + 1
        if profile_step > 0:
            emit("left_basis", profile_step, oracle_state["left_basis"])
            emit("right_basis", profile_step, oracle_state["right_basis"])
            emit("momentum_before_adam", profile_step, oracle_state["momentum"])
        update = oracle.soap_step(gradient, oracle_state, basis_implementation="eigh", **config)
        emit("gradient", profile_step, gradient)
        emit("returned_update", profile_step, update)
        if profile_step > 0:
            for name in ("left_preconditioner", "right_preconditioner", "left_basis", "right_basis", "momentum",
                         "variance"):
                emit(name + "_after_step", profile_step, oracle_state[name])
    (tmp_path / "reference.log").write_text("\n".join(reference_lines))
    (tmp_path / "candidate.log").write_text(candidate_text)
    status = compare_profiles.main([str(tmp_path / "reference.log"), str(tmp_path / "candidate.log"),
                                    "--tolerance", "1e-4", "--steps", "0,2,3,4"])
    report = capfd.readouterr().out
    assert status == 0, report
    assert "sign-flipped" in report or "within" in report
