"""Host-side checks that need no GPU: the C ABI exports what the header declares, argument
validation raises the reference's exception types before anything is launched, layouts match
the reference's allocator, and the ``soap_tp`` import name resolves to this package."""
import ctypes
import subprocess
import sys

import pytest
import torch

import soap_tp_amd
from soap_tp_amd import _native, ops
from soap_tp_amd.binding import NativeBinding
from soap_tp_amd.ops import _utils

GRID = (1, 1)


def test_library_exports_every_declared_symbol():
    declared = _native.declared_functions()
    assert len(declared) >= 30
    assert {"soapmi_gram_ema_f32", "soapmi_rotate_adam_rotate_f32", "soapmi_eigh_f64", "soapmi_qr_f32",
            "soapmi_refresh_f32", "soapmi_initialize_basis_f32"} <= set(declared)
    lib = ctypes.CDLL(str(_native.LIBRARY_PATH))
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/soap_mi355.h but not exported"
    exported = subprocess.run(["nm", "-D", "--defined-only", str(_native.LIBRARY_PATH)],
                              capture_output=True, text=True).stdout
    undeclared = {line.split()[-1] for line in exported.splitlines() if " T soapmi_" in line} - set(declared)
    assert not undeclared, f"exported but not declared: {sorted(undeclared)}"


def test_header_parser_types():
    declared = _native.declared_functions()
    assert declared["soapmi_compiled_gpu_backend"] == ("const char*", [])
    return_type, parameters = declared["soapmi_gram_ema_f32"]
    assert return_type == "int"
    assert parameters == ["const float*", "int64_t", "int64_t", "int64_t", "int", "int", "float*", "int64_t",
                          "float", "int", "void*"]
    assert declared["soapmi_rotate_workspace_bytes"][0] == "size_t"


def test_introspection_needs_no_gpu():
    binding = NativeBinding()
    assert binding.compiled_gpu_backend() == "rocm"
    assert binding.mpi_world_rank_and_size() == (0, 1)
    lib = _native.library()
    assert lib.soapmi_rotate_workspace_bytes(128, 64) >= 128 * 64 * 4
    assert lib.soapmi_qr_workspace_bytes(1024) > 0
    assert lib.soapmi_eigh_workspace_bytes(256, 8) > 2 * 256 * 256 * 8


def test_status_codes_map_to_reference_exception_types():
    with pytest.raises(ValueError, match="beta must be in"):
        _native.call("soapmi_gram_ema_f32", 1, 4, 4, 4, 1, 0, 1, 4, 1.5, 0, None)
    with pytest.raises(ValueError, match="nonzero"):
        _native.call("soapmi_rotate_f32", None, None, None, 4, 4, 4, 4, 4, 1, None, 0, None)
    with pytest.raises(ValueError, match="positive"):
        _native.call("soapmi_qr_f32", 1, 2, 0, 1, 1, None, 0, None)
    with pytest.raises(ValueError, match="step must be positive"):
        _native.call("soapmi_adam_f32", 1, 4, 1, 4, 1, 4, 1, 4, 4, 4, 0, 0.9, 0.9, 1e-8, None)
    with pytest.raises(ValueError, match="workspace holds"):
        _native.call("soapmi_rotate_f32", 8, 16, 24, 4, 4, 4, 4, 4, 1, 32, 8, None)


def test_allocate_layout_matches_reference_allocator():
    buffer = ops.allocate_2d_block_cyclic((5, 7), 2, GRID)
    assert buffer.shape == (5, 7) and buffer.stride() == (1, 5) and buffer.dtype == torch.float32
    assert torch.count_nonzero(buffer) == 0
    assert ops.allocate_2d_block_cyclic((0, 3), 2, GRID).shape == (1, 3)  # dummy row, like the reference
    with pytest.raises(ValueError, match="does not match world_size"):
        ops.allocate_2d_block_cyclic((4, 4), 2, (2, 2))
    with pytest.raises(ValueError, match="positive dimensions"):
        ops.allocate_2d_block_cyclic((4, 4), 2, (0, 1))
    with pytest.raises(ValueError, match="block_size must be positive"):
        ops.allocate_2d_block_cyclic((4, 4), 0, GRID)


def test_block_cyclic_indices_degenerate_and_general():
    assert _utils.block_cyclic_indices(7, 3, 0, 1) == tuple(range(7))
    assert _utils.block_cyclic_indices(10, 2, 1, 2) == (2, 3, 6, 7)
    assert _utils.local_2d_block_cyclic_shape((9, 13), 2, (2, 2), 3) == (4, 6)


def test_buffer_validation_messages():
    good = ops.allocate_2d_block_cyclic((4, 4), 2, GRID)
    assert _utils.validate_2d_block_cyclic_buffer("m", good, (4, 4), 2, GRID, 0) == (4, 4)
    with pytest.raises(ValueError, match="column-major"):
        _utils.validate_2d_block_cyclic_buffer("m", torch.zeros(4, 4), (4, 4), 2, GRID, 0)
    with pytest.raises(ValueError, match="must be 2D"):
        _utils.validate_2d_block_cyclic_buffer("m", torch.zeros(4), (4, 4), 2, GRID, 0)
    with pytest.raises(ValueError, match="storage rows"):
        _utils.validate_2d_block_cyclic_buffer("m", good, (6, 4), 2, GRID, 0)
    with pytest.raises(ValueError, match="storage columns"):
        _utils.validate_2d_block_cyclic_buffer("m", good, (4, 6), 2, GRID, 0)


def test_soap_step_argument_errors_before_any_launch():
    gradient = torch.zeros(4, 4)
    kwargs = dict(global_shape=(4, 4), shard_dim=1, block_size=2, process_grid_shape=GRID)
    with pytest.raises(ValueError, match="basis_refresh_interval must be positive"):
        soap_tp_amd.soap_step(gradient, {}, basis_refresh_interval=0, **kwargs)
    with pytest.raises(ValueError, match="basis_implementation must be 'elpa' or 'eigh'"):
        soap_tp_amd.soap_step(gradient, {}, basis_implementation="jacobi", **kwargs)
    with pytest.raises(ValueError, match="does not match world_size"):
        soap_tp_amd.soap_step(gradient, {}, **{**kwargs, "process_grid_shape": (2, 2)})
    with pytest.raises(ValueError, match="expected"):
        soap_tp_amd.soap_step(gradient, {}, **{**kwargs, "global_shape": (4, 8)})
    with pytest.raises(ValueError, match="requires cuda buffers"):
        soap_tp_amd.soap_step(gradient, {}, **kwargs)  # there is no CPU fallback


def test_ops_reject_cpu_and_bad_arguments():
    matrix = ops.allocate_2d_block_cyclic((4, 6), 2, GRID)
    q_left = ops.allocate_2d_block_cyclic((4, 4), 2, GRID)
    q_right = ops.allocate_2d_block_cyclic((6, 6), 2, GRID)
    with pytest.raises(ValueError, match="direction must be"):
        ops.rotate_2d_block_cyclic_(matrix, q_left, q_right, (4, 6), 2, GRID, direction="up")
    with pytest.raises(ValueError, match="requires cuda buffers"):
        ops.rotate_2d_block_cyclic_(matrix, q_left, q_right, (4, 6), 2, GRID, direction="forward")
    with pytest.raises(ValueError, match="must use float32"):
        ops.rotate_2d_block_cyclic_(matrix.double(), q_left, q_right, (4, 6), 2, GRID, direction="forward")
    with pytest.raises(ValueError, match="must not overlap"):
        ops.rotate_2d_block_cyclic_(q_left, q_left, q_left, (4, 4), 2, GRID, direction="forward")
    with pytest.raises(ValueError, match="step must be positive"):
        ops.adam_update(matrix, matrix.clone(), matrix.clone(), 0)
    with pytest.raises(ValueError, match=r"beta1 must be in \[0, 1\)"):
        ops.adam_update(matrix, matrix.clone(), matrix.clone(), 1, beta1=1.0)
    with pytest.raises(ValueError, match="eps must be positive"):
        ops.adam_update(matrix, matrix.clone(), matrix.clone(), 1, eps=0.0)
    with pytest.raises(ValueError, match="identical shapes"):
        ops.adam_update(matrix, q_left, matrix.clone(), 1)
    with pytest.raises(ValueError, match=r"beta must be in \[0, 1\]"):
        ops.update_left_preconditioner_2d_block_cyclic_(matrix, q_left, 1.5, 2, GRID, shard_dim=1)
    with pytest.raises(ValueError, match="shard_dim must be 0 or 1"):
        ops.update_left_preconditioner_2d_block_cyclic_(matrix, q_left, 0.5, 2, GRID, shard_dim=2)
    with pytest.raises(ValueError, match="implementation must be"):
        ops.initialize_basis_2d_block_cyclic_(q_left, q_left.clone(), q_left.clone(), torch.zeros(4), 4, 2, GRID,
                                              implementation="qr")
    with pytest.raises(ValueError, match="eigenvalues must be float32"):
        ops.initialize_basis_2d_block_cyclic_(q_left, _cm(4), _cm(4), torch.zeros(5), 4, 2, GRID)
    with pytest.raises(ValueError, match="LDAs must match"):
        padded = torch.zeros(4, 6).T[:4]
        ops.estimated_eigenvalue_order_2d_block_cyclic_(q_left, _cm(4), padded, 4, 2, GRID)


def _cm(size):
    return ops.allocate_2d_block_cyclic((size, size), 2, GRID)


def test_binding_argument_checks_mirror_reference_bindings():
    binding = NativeBinding()
    with pytest.raises(ValueError, match="process grid"):
        binding.slate_qr_float(1, 2, 4, 4, 4, 2, 2, 2)
    with pytest.raises(ValueError, match="nonzero"):
        binding.slate_symmetric_multiply_float(0, 1, 2, 4, 4, 2, 1, 1)
    with pytest.raises(ValueError, match="positive"):
        binding.slate_forward_rotation_float(1, 2, 3, 0, 4, 4, 4, 4, 2, 1, 1)
    with pytest.raises(ValueError, match="nonnegative GPU device index"):
        binding.elpa_eigenvectors_2d_block_cyclic_double(1, 2, 3, 4, 4, 4, 2, 1, 1, -1)


def test_soap_tp_import_name_is_an_alias():
    code = ("import soap_tp, soap_tp_amd; from soap_tp import soap_step; from soap_tp.ops import adam_update;"
            "assert soap_step is soap_tp_amd.soap_step and soap_tp.ops is soap_tp_amd.ops; print('ok')")
    result = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True,
                            cwd=str(_native.PACKAGE_DIR.parent))
    assert result.returncode == 0 and "ok" in result.stdout, result.stderr
    assert sorted(ops.__all__) == sorted([
        "adam_update", "allocate_2d_block_cyclic", "estimated_eigenvalue_order_2d_block_cyclic_",
        "initialize_basis_2d_block_cyclic_", "permute_2d_block_cyclic_", "power_iteration_qr_2d_block_cyclic_",
        "qr_2d_block_cyclic_", "redistribute_2d_block_cyclic_to_tp_shard",
        "redistribute_tp_shard_to_2d_block_cyclic", "refresh_bases_and_transport_optimizer_state_",
        "rotate_2d_block_cyclic_", "update_left_preconditioner_2d_block_cyclic_",
        "update_right_preconditioner_2d_block_cyclic_",
    ])


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setattr(_native, "_library", None)
    monkeypatch.setattr(_native, "LIBRARY_PATH", tmp_path / "libsoap_mi355.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _native.library()


def test_reference_import_paths_resolve_to_this_package():
    """Every module path the reference's tests and scripts import (tests/unit/*.py,
    scripts/run_soap_tp_timing_gpu.py:76 of the reference) resolves under the ``soap_tp`` alias to
    the same objects as in ``soap_tp_amd``."""
    import importlib

    import soap_tp
    import soap_tp_amd
    from soap_tp import elpa_bindings, slate_bindings, soap_step
    from soap_tp.ops._utils import allocate_2d_block_cyclic, validate_2d_block_cyclic_buffer
    from soap_tp.ops.factorizations import (initialize_basis_2d_block_cyclic_, power_iteration_qr_2d_block_cyclic_,
                                            refresh_bases_and_transport_optimizer_state_)
    from soap_tp.ops.optimizer import adam_update
    from soap_tp.ops.preconditioners import (update_left_preconditioner_2d_block_cyclic_,
                                             update_right_preconditioner_2d_block_cyclic_)
    from soap_tp.soap import soap_step as soap_step_again

    assert soap_step is soap_tp_amd.soap_step is soap_step_again
    assert soap_tp.ops is soap_tp_amd.ops
    for path in ("ops", "ops._utils", "ops.factorizations", "ops.optimizer", "ops.preconditioners", "soap"):
        assert importlib.import_module(f"soap_tp.{path}") is importlib.import_module(f"soap_tp_amd.{path}")
    assert adam_update is soap_tp_amd.ops.adam_update
    assert allocate_2d_block_cyclic is soap_tp_amd.ops.allocate_2d_block_cyclic
    assert initialize_basis_2d_block_cyclic_ is soap_tp_amd.ops.initialize_basis_2d_block_cyclic_
    assert power_iteration_qr_2d_block_cyclic_ is soap_tp_amd.ops.power_iteration_qr_2d_block_cyclic_
    assert refresh_bases_and_transport_optimizer_state_ is soap_tp_amd.ops.refresh_bases_and_transport_optimizer_state_
    assert update_left_preconditioner_2d_block_cyclic_ is soap_tp_amd.ops.update_left_preconditioner_2d_block_cyclic_
    assert update_right_preconditioner_2d_block_cyclic_ is soap_tp_amd.ops.update_right_preconditioner_2d_block_cyclic_
    assert callable(validate_2d_block_cyclic_buffer)
    # the binding modules expose the reference's function names
    for name in ("compiled_gpu_backend", "mpi_world_rank_and_size", "slate_symmetric_multiply_float", "slate_qr_float",
                 "slate_forward_rotation_float", "slate_backward_rotation_float"):
        assert callable(getattr(slate_bindings, name))
    for name in ("compiled_gpu_backend", "mpi_world_rank_and_size", "initialize_basis_2d_block_cyclic_",
                 "elpa_eigenvectors_2d_block_cyclic_double"):
        assert callable(getattr(elpa_bindings, name))
    assert slate_bindings.compiled_gpu_backend() == "rocm" and elpa_bindings.mpi_world_rank_and_size() == (0, 1)
