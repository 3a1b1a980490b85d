"""The entry point that allocates nothing (``soapmi_rotate_adam_rotate_static_f32``, whose two
temporaries live in a static device array of the library) against the entry point it is a variant
of (``soapmi_rotate_adam_rotate_f32`` with a caller workspace): same kernels, so update, momentum
and variance must be equal bit for bit.  Two calls in a row, the second on a smaller input, so that
what the first call left in the shared array is there when the second one runs.  Collected last, so
that a failure here hides no other test."""
import pytest
import torch

from soap_tp_amd import _native
from tests.helpers import SEED, column_major, make_matrix, make_orthogonal

pytestmark = pytest.mark.gpu
LIMIT = 4194304


def _inputs(rows, columns, seed, device):
    gradient = make_matrix(rows, columns, seed=seed).to(device)
    q_left = column_major(make_orthogonal(rows, seed + 1), device)
    q_right = column_major(make_orthogonal(columns, seed + 2), device)
    momentum = column_major(make_matrix(rows, columns, seed=seed + 3), device)
    variance = column_major(make_matrix(rows, columns, seed=seed + 4).square(), device)
    return gradient, q_left, q_right, momentum, variance


def _call(static, gradient, q_left, q_right, momentum, variance, step, stream):
    rows, columns = gradient.shape
    update = torch.empty_like(gradient)
    arguments = [gradient.data_ptr(), gradient.stride(0), update.data_ptr(), update.stride(0),
                 q_left.data_ptr(), q_left.stride(1), q_right.data_ptr(), q_right.stride(1),
                 momentum.data_ptr(), momentum.stride(1), variance.data_ptr(), variance.stride(1),
                 rows, columns, step, 0.9, 0.95, 1e-8]
    if static:
        _native.call("soapmi_rotate_adam_rotate_static_f32", *arguments, stream)
    else:
        nbytes = _native.library().soapmi_rotate_adam_rotate_workspace_bytes(rows, columns)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=gradient.device)
        _native.call("soapmi_rotate_adam_rotate_f32", *arguments, workspace.data_ptr(), nbytes, stream)
    return update


def test_static_scratch_entry_point_equals_workspace_entry_point(device):
    stream = torch.cuda.current_stream(device).cuda_stream
    for shape, seed in (((1024, 1536), SEED + 900), ((200, 136), SEED + 910)):  # the second is smaller
        gradient, q_left, q_right, momentum, variance = _inputs(*shape, seed, device)
        results = []
        for static in (False, True):
            m, v = momentum.clone(), variance.clone()
            update = _call(static, gradient, q_left, q_right, m, v, 3, stream)
            results.append((update, m, v))
        torch.cuda.synchronize(device)
        for expected, actual in zip(*results):
            assert torch.isfinite(expected).all()
            assert torch.equal(expected, actual), shape


def test_static_scratch_entry_point_allocates_no_device_memory(device):
    """What the entry point exists for: with inputs and outputs in place, the free device memory the
    driver reports is the same before and after its calls (sizes this process has not run before, so
    nothing is served from a cache; the library's own grow-only scratch is not involved either)."""
    stream = torch.cuda.current_stream(device).cuda_stream
    prepared = []
    for shape, seed in (((768, 1280), SEED + 920), ((96, 72), SEED + 930)):
        gradient, q_left, q_right, momentum, variance = _inputs(*shape, seed, device)
        prepared.append((gradient, q_left, q_right, momentum, variance, torch.empty_like(gradient)))
    torch.cuda.synchronize(device)
    free_before, _ = torch.cuda.mem_get_info(device)
    for gradient, q_left, q_right, momentum, variance, update in prepared:
        rows, columns = gradient.shape
        _native.call("soapmi_rotate_adam_rotate_static_f32", gradient.data_ptr(), gradient.stride(0),
                     update.data_ptr(), update.stride(0), q_left.data_ptr(), q_left.stride(1), q_right.data_ptr(),
                     q_right.stride(1), momentum.data_ptr(), momentum.stride(1), variance.data_ptr(),
                     variance.stride(1), rows, columns, 2, 0.9, 0.95, 1e-8, stream)
    torch.cuda.synchronize(device)
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before
    assert all(torch.isfinite(item[5]).all() for item in prepared)


def test_static_scratch_entry_point_rejects_what_does_not_fit(device):
    stream = torch.cuda.current_stream(device).cuda_stream
    rows, columns = 2048, 2049  # one column more than the array holds
    assert rows * columns > LIMIT
    gradient = torch.zeros(rows, columns, device=device)
    square_left = torch.zeros(rows, rows, device=device).T
    square_right = torch.zeros(columns, columns, device=device).T
    moments = torch.zeros(columns, rows, device=device).T
    with pytest.raises(ValueError, match="exceeds the 4194304 elements"):
        _call(True, gradient, square_left, square_right, moments, moments.clone(), 1, stream)
