"""CPU tests of the host-side helpers around the step: state (de)serialisation, the SOAP_PROFILE
comparer and the optimizer wrapper's argument handling (no GPU, no library calls)."""
import json

import pytest
import torch

from soap_tp_amd import compare_profiles, state_io
from soap_tp_amd.optim import SOAP
from tests.helpers import make_orthogonal


def _column_major(rows, columns, seed, pad=0):
    generator = torch.Generator().manual_seed(seed)
    return torch.randn(columns, max(1, rows) + pad, generator=generator).T[:rows, :]


def _state(rows=3, columns=5, pad=0):
    state = {
        "left_preconditioner": _column_major(rows, rows, 1, pad), "right_preconditioner": _column_major(columns, columns, 2),
        "left_basis": _column_major(rows, rows, 3), "right_basis": _column_major(columns, columns, 4, pad),
        "left_work": _column_major(rows, rows, 5), "right_work": _column_major(columns, columns, 6),
        "momentum": _column_major(rows, columns, 7, pad), "variance": _column_major(rows, columns, 8), "step": 4,
    }
    return state


# ---- state_io -----------------------------------------------------------------------------------
@pytest.mark.parametrize("pad", [0, 3])
def test_pack_unpack_round_trip_restores_values_and_layout(pad):
    state = _state(pad=pad)
    packed = state_io.pack_state(state)
    assert all(packed[name].is_contiguous() for name in state_io.STATE_BUFFERS)
    restored = state_io.unpack_state(packed)
    assert restored["step"] == 4
    for name in state_io.STATE_BUFFERS:
        assert torch.equal(restored[name], _saved_form(name, state[name]))
        assert restored[name].stride() == (1, max(1, state[name].size(0)))


def _saved_form(name, tensor):
    """What a saved state holds for a buffer: Gram matrices symmetrised from their lower triangle."""
    if name.endswith("_preconditioner"):
        return torch.tril(tensor) + torch.tril(tensor, -1).T
    return tensor


def test_saved_gram_matrices_are_symmetric_whatever_the_upper_triangle_held():
    """soap_step keeps only the lower triangle of the Gram matrices current between refreshes; a saved
    state must have both triangles valid (src/soap_tp/ops/factorizations.py:378)."""
    state = _state(rows=6, columns=9)
    for side in ("left", "right"):
        matrix = state[f"{side}_preconditioner"]
        matrix.copy_(torch.tril(matrix) + torch.tril(matrix, -1).T)
    expected = {side: state[f"{side}_preconditioner"].clone() for side in ("left", "right")}
    for side in ("left", "right"):  # a stale upper triangle
        state[f"{side}_preconditioner"].add_(torch.triu(torch.full_like(expected[side], 7.0), 1))
    restored = state_io.unpack_state(state_io.pack_state(state))
    for side in ("left", "right"):
        assert torch.equal(restored[f"{side}_preconditioner"], expected[side])
        assert torch.equal(restored[f"{side}_preconditioner"], restored[f"{side}_preconditioner"].T)


def test_save_load_round_trip_uses_a_safe_loader(tmp_path):
    state = _state()
    path = tmp_path / "state.pt"
    state_io.save_state(state, path)
    target = {"stale": 1}
    loaded = state_io.load_state(path, into=target)
    assert loaded is target and "stale" not in target
    assert state_io.validate_state(loaded) == (3, 5)
    for name in state_io.STATE_BUFFERS:
        assert torch.equal(loaded[name], _saved_form(name, state[name]))
    # the file holds tensors and plain scalars only
    raw = torch.load(path, weights_only=True)
    assert raw["rows"] == 3 and raw["columns"] == 5 and raw["step"] == 4


def test_uninitialised_state_round_trips_to_empty():
    assert state_io.unpack_state(state_io.pack_state({})) == {}


def test_validate_state_rejects_broken_states():
    state = _state()
    assert state_io.validate_state(state, (3, 5)) == (3, 5)
    with pytest.raises(ValueError, match="expected"):
        state_io.validate_state(state, (5, 3))
    broken = dict(state)
    del broken["variance"]
    with pytest.raises(ValueError, match="missing"):
        state_io.validate_state(broken)
    broken = dict(state, momentum=state["momentum"].contiguous())  # row-major
    with pytest.raises(ValueError, match="column-major"):
        state_io.validate_state(broken)
    broken = dict(state, left_basis=state["left_basis"].double())
    with pytest.raises(ValueError, match="float32"):
        state_io.validate_state(broken)
    broken = dict(state, right_work=_column_major(4, 4, 9))
    with pytest.raises(ValueError, match="shape"):
        state_io.validate_state(broken)
    broken = dict(state, step=-1)
    with pytest.raises(ValueError, match="step"):
        state_io.validate_state(broken)


def test_unpack_rejects_wrong_version_and_shapes():
    packed = state_io.pack_state(_state())
    with pytest.raises(ValueError, match="version"):
        state_io.unpack_state(dict(packed, format_version=99))
    with pytest.raises(ValueError, match="shape"):
        state_io.unpack_state(dict(packed, momentum=packed["momentum"].T.contiguous()))
    with pytest.raises(ValueError, match="float32"):
        state_io.unpack_state(dict(packed, variance=packed["variance"].double()))


# ---- compare_profiles ----------------------------------------------------------------------------
def _line(impl, step, stage, tensor):
    return "noise before " + compare_profiles.MARKER + json.dumps(
        {"impl": impl, "step": step, "stage": stage, "shape": list(tensor.shape), "values": tensor.reshape(-1).tolist()})


def _logs(perturb=None):
    rows, columns = 4, 6
    q_left, q_right = make_orthogonal(rows, 11).double(), make_orthogonal(columns, 12).double()
    generator = torch.Generator().manual_seed(5)
    gradient = torch.randn(rows, columns, generator=generator, dtype=torch.float64)
    projected = q_left.T @ gradient @ q_right
    variance = projected.square()
    update = q_left @ (projected / (variance.sqrt() + 1e-8)) @ q_right.T
    s_left = torch.tensor([1.0, -1.0, 1.0, -1.0], dtype=torch.float64)
    s_right = torch.tensor([-1.0, 1.0, 1.0, -1.0, 1.0, 1.0], dtype=torch.float64)
    reference = {"gradient": gradient, "left_basis": q_left, "right_basis": q_right, "projected_gradient": projected,
                 "momentum_after_adam": 0.2 * projected, "variance_after_adam": 0.1 * variance,
                 "returned_update": update}
    candidate = {"gradient": gradient, "left_basis": q_left * s_left, "right_basis": q_right * s_right,
                 "projected_gradient": projected * s_left[:, None] * s_right[None, :],
                 "momentum_after_adam": 0.2 * projected * s_left[:, None] * s_right[None, :],
                 "variance_after_adam": 0.1 * variance, "returned_update": update, "gradient_2d": gradient}
    if perturb:
        candidate[perturb] = candidate[perturb] * 1.01
    return ([_line("reference", 1, stage, tensor) for stage, tensor in reference.items()],
            [_line("tp", 1, stage, tensor) for stage, tensor in candidate.items()] + ["unrelated text"])


def test_comparer_aligns_signs_of_bases_and_coordinates():
    reference_lines, candidate_lines = _logs()
    rows = compare_profiles.compare(compare_profiles.read_log(reference_lines, "a"),
                                    compare_profiles.read_log(candidate_lines, "b"))
    assert [row["stage"] for row in rows] == ["gradient", "left_basis", "right_basis", "projected_gradient",
                                              "momentum_after_adam", "variance_after_adam", "returned_update"]
    assert all(row["error"] < 1e-12 for row in rows)
    flipped = {row["stage"]: row["flipped"] for row in rows}
    assert flipped["left_basis"] == 2 and flipped["right_basis"] == 2
    assert compare_profiles.first_divergence(rows, 1e-6) is None


def test_comparer_names_the_first_diverging_stage(tmp_path, capsys):
    reference_lines, candidate_lines = _logs(perturb="momentum_after_adam")
    (tmp_path / "ref.log").write_text("\n".join(reference_lines))
    (tmp_path / "tp.log").write_text("\n".join(candidate_lines))
    status = compare_profiles.main([str(tmp_path / "ref.log"), str(tmp_path / "tp.log"), "--tolerance", "1e-6"])
    output = capsys.readouterr().out
    assert status == 1
    assert "first stage above 1e-06: step 1 momentum_after_adam" in output
    assert "only in" in output and "gradient_2d" in output
    reference_lines, candidate_lines = _logs()
    (tmp_path / "tp.log").write_text("\n".join(candidate_lines))
    assert compare_profiles.main([str(tmp_path / "ref.log"), str(tmp_path / "tp.log")]) == 0


def test_comparer_reports_unusable_input(tmp_path, capsys):
    (tmp_path / "empty.log").write_text("nothing here\n")
    (tmp_path / "bad.log").write_text(compare_profiles.MARKER + '{"step": 1}\n')
    assert compare_profiles.main([str(tmp_path / "empty.log"), str(tmp_path / "empty.log")]) == 2
    assert compare_profiles.main([str(tmp_path / "bad.log"), str(tmp_path / "empty.log")]) == 2
    assert "unusable SOAP_PROFILE line" in capsys.readouterr().err


# ---- optimizer wrapper: argument handling --------------------------------------------------------
def test_optimizer_rejects_bad_hyper_parameters():
    weight = torch.nn.Parameter(torch.zeros(4, 4))
    for kwargs in (dict(lr=-1.0), dict(betas=(1.0, 0.9)), dict(shampoo_beta=1.0), dict(eps=0.0), dict(weight_decay=-0.1),
                   dict(precondition_frequency=0), dict(basis_implementation="jacobi"), dict(streams=99)):
        with pytest.raises(ValueError):
            SOAP([weight], **kwargs)


def test_optimizer_has_the_original_defaults_and_no_cpu_path():
    weight = torch.nn.Parameter(torch.zeros(4, 4))
    optimizer = SOAP([weight])
    group = optimizer.param_groups[0]
    # tests/reference/soap.py:80-94 of the reference checkout
    assert (group["lr"], group["betas"], group["shampoo_beta"], group["eps"], group["weight_decay"],
            group["precondition_frequency"]) == (3e-3, (0.95, 0.95), -1.0, 1e-8, 0.01, 10)
    weight.grad = torch.ones(4, 4)
    with pytest.raises(ValueError, match="GPU"):
        optimizer.step()
    assert torch.count_nonzero(weight) == 0


def test_optimizer_rejects_higher_rank_parameters_unless_flattening_is_requested():
    assert SOAP._matrix_view(torch.zeros(7), False) is None
    assert SOAP._matrix_view(torch.zeros(1, 7), False) is None
    assert SOAP._matrix_view(torch.zeros(3, 7), False).shape == (3, 7)
    with pytest.raises(ValueError, match="flatten_nd"):
        SOAP._matrix_view(torch.zeros(2, 3, 4), False)
    assert SOAP._matrix_view(torch.zeros(2, 3, 4), True).shape == (2, 12)
