"""Eigenbasis initialisation on the GPU (sytrd + divide and conquer + back-transformation)
against the CPU oracle (LAPACK), restating tests/unit/test_elpa_bindings.py:460-515 of the
reference for one rank: eigenvalues, orthonormality, P Q = Q diag(w), per-vector agreement for
simple eigenvalues, and equality of the zero-eigenspace projectors for rank-deficient Gram
matrices.  Tolerance 2e-4 absolute/relative as there; the eigenvalue bar of this build is a
relative error <= 1e-5 with respect to the largest eigenvalue."""
import math

import pytest
import torch

from oracle import soap_oracle as oracle
from soap_tp_amd import _native, ops
from tests.helpers import MATRIX_SHAPES, SEED, column_major, eigen_clusters, make_matrix, subspace_distance

pytestmark = pytest.mark.gpu
GRID = (1, 1)
BLOCK = 2


@pytest.fixture(autouse=True, params=[1, 2], ids=["one-stage", "two-stage"])
def eigh_algorithm(request):
    """Every test of this module runs with both tridiagonalisations behind the eigensolver entry
    points: the one-stage reduction (the default) and the two-stage one (dense -> band ->
    tridiagonal, option "eigh_algorithm" = 2)."""
    _native.call("soapmi_set_option", b"eigh_algorithm", request.param)
    yield request.param
    _native.call("soapmi_set_option", b"eigh_algorithm", 1)


def _initialize(preconditioner, implementation, device, poison_upper=False):
    size = preconditioner.shape[0]
    packed = column_major(preconditioner, device)
    if poison_upper:
        packed.copy_(torch.tril(packed) + torch.triu(torch.full_like(packed, 5.0), 1))
    basis = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    work = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    values = torch.empty(size, dtype=torch.float32, device=device)
    result = ops.initialize_basis_2d_block_cyclic_(packed, basis, work, values, size, BLOCK, GRID,
                                                   implementation=implementation)
    assert result is basis
    return values.cpu(), basis.cpu(), work.cpu()


def _check_against_oracle(preconditioner, values, basis, implementation, tol=2e-4):
    size = preconditioner.shape[0]
    expected_values, expected_basis = oracle.eigh_descending(preconditioner, implementation)
    scale = max(expected_values.abs().max().item(), 1e-30)
    assert torch.all(values[:-1] >= values[1:] - 1e-6 * scale)  # descending
    assert (values - expected_values).abs().max().item() <= 1e-5 * scale
    torch.testing.assert_close(basis.T @ basis, torch.eye(size), rtol=tol, atol=tol)
    residual = preconditioner.double() @ basis.double() - basis.double() * values.double()
    assert residual.abs().max().item() <= tol * scale
    # vectors of simple eigenvalues agree up to sign; clusters agree as subspaces
    for start, stop in eigen_clusters(expected_values, 1e-3):
        mine, theirs = basis[:, start:stop], expected_basis[:, start:stop]
        if stop - start == 1:
            assert abs(abs(torch.dot(mine[:, 0].double(), theirs[:, 0].double()).item()) - 1) <= 1e-3
        else:
            assert subspace_distance(mine, theirs) <= 1e-2
    return expected_values, expected_basis


@pytest.mark.parametrize("shape", MATRIX_SHAPES)
@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("implementation", ["elpa", "eigh"])
def test_initialize_basis_gram_matrices(shape, side, implementation, device):
    gradient = make_matrix(*shape)
    gram = gradient @ gradient.T if side == "left" else gradient.T @ gradient
    values, basis, work = _initialize(gram, implementation, device, poison_upper=True)
    expected_values, expected_basis = _check_against_oracle(gram, values, basis, implementation)
    if implementation == "elpa":
        assert torch.equal(work, -(torch.tril(gram) + torch.tril(gram, -1).T))  # work <- -P (reference :500)
    # zero eigenspace of a rank-deficient Gram matrix (test_elpa_bindings.py:341-457)
    rank = min(shape)
    size = gram.shape[0]
    if size > rank:
        assert torch.all(values[rank:].abs() <= 2e-4 * values[0])
        mine = basis[:, rank:] @ basis[:, rank:].T
        theirs = expected_basis[:, rank:] @ expected_basis[:, rank:].T
        torch.testing.assert_close(mine, theirs, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("size", [1, 2, 3, 5, 31, 32, 33, 34, 64, 66, 100, 257, 600, 1000])
@pytest.mark.parametrize("implementation", ["elpa", "eigh"])
def test_initialize_basis_sizes(size, implementation, device):
    g = make_matrix(size, size + 5, seed=SEED + size)
    _check_against_oracle(g @ g.T / size, *_initialize(g @ g.T / size, implementation, device)[:2], implementation)


@pytest.mark.parametrize("implementation", ["elpa", "eigh"])
def test_initialize_basis_special_matrices(implementation, device):
    size = 96
    diagonal = torch.diag(torch.linspace(1.0, 3.0, size)[torch.randperm(size, generator=torch.Generator().manual_seed(1))])
    values, basis, _ = _initialize(diagonal, implementation, device)
    assert torch.allclose(values, torch.linspace(3.0, 1.0, size), atol=1e-6)
    assert torch.allclose(basis.abs().sum(0), torch.ones(size)) and torch.allclose(basis.abs().max(0).values, torch.ones(size))
    values, basis, _ = _initialize(torch.zeros(size, size), implementation, device)
    assert values.abs().max().item() <= 1.1e-30  # "eigh" adds the reference's 1e-30 diagonal shift
    torch.testing.assert_close(basis.T @ basis, torch.eye(size))
    toeplitz = 2 * torch.eye(size) - torch.diag(torch.ones(size - 1), 1) - torch.diag(torch.ones(size - 1), -1)
    values, basis, _ = _initialize(toeplitz, implementation, device)
    expected = torch.tensor([2 - 2 * math.cos(k * math.pi / (size + 1)) for k in range(size, 0, -1)])
    assert torch.allclose(values, expected.float(), atol=2e-6)
    wilkinson = torch.diag((torch.arange(size) - size // 2).abs().float()) + torch.diag(torch.ones(size - 1), 1) \
        + torch.diag(torch.ones(size - 1), -1)
    _check_against_oracle(wilkinson, *_initialize(wilkinson, implementation, device)[:2], implementation)
    tiny = 1e-12 * (make_matrix(40, 60) @ make_matrix(40, 60).T)
    _check_against_oracle(tiny, *_initialize(tiny, implementation, device)[:2], implementation)


def test_low_rank_plus_noise_gram_signal_and_bulk(device):
    # the benchmark's regime: 16 signal directions over a noise bulk of nearly equal eigenvalues
    gradient = oracle.low_rank_plus_noise(300, 420, 16, seed=SEED)
    gram = 0.05 * gradient @ gradient.T
    for implementation in ("elpa", "eigh"):
        values, basis, _ = _initialize(gram, implementation, device)
        expected_values, expected_basis = oracle.eigh_descending(gram, implementation)
        scale = expected_values[0].item()
        assert (values - expected_values).abs().max().item() <= 1e-5 * scale
        assert subspace_distance(basis[:, :8], expected_basis[:, :8]) <= 1e-3
        residual = gram.double() @ basis.double() - basis.double() * values.double()
        assert torch.linalg.matrix_norm(residual).item() <= 1e-5 * torch.linalg.matrix_norm(gram.double()).item() * 10
        torch.testing.assert_close(basis.T @ basis, torch.eye(300), rtol=1e-4, atol=1e-4)


def test_eigh_f64_c_abi_directly(device):
    """soapmi_eigh_f64 is the replacement for elpa_eigenvectors_2d_block_cyclic_double: ascending,
    float64, input destroyed, lower triangle referenced."""
    size = 200
    g = make_matrix(size, size, dtype=torch.float64)
    matrix = (g + g.T) / 2
    a = column_major(torch.tril(matrix) + torch.triu(torch.full_like(matrix, 9.0), 1), device)
    q = torch.zeros(size, size, dtype=torch.float64, device=device).T
    w = torch.zeros(size, dtype=torch.float64, device=device)
    _native.call("soapmi_eigh_f64", a.data_ptr(), w.data_ptr(), q.data_ptr(), size, size, size, None, 0,
                 torch.cuda.current_stream().cuda_stream)
    expected = torch.linalg.eigvalsh(matrix)
    assert torch.allclose(w.cpu(), expected, rtol=0, atol=1e-12 * expected.abs().max().item() * size)
    qc = q.cpu()
    assert (qc.T @ qc - torch.eye(size, dtype=torch.float64)).abs().max().item() < 1e-12
    assert (matrix @ qc - qc * w.cpu()).abs().max().item() < 1e-11
    with pytest.raises(ValueError, match="leading dimensions"):
        _native.call("soapmi_eigh_f64", a.data_ptr(), w.data_ptr(), q.data_ptr(), size, size - 1, size, None, 0, None)


@pytest.mark.parametrize("size", [1, 2, 33, 200, 700])
def test_eigh_f32_c_abi_directly(size, device):
    """soapmi_eigh_f32 is the solver behind the `eigh` variant (torch.linalg.eigh on the float32
    Gram matrix in the reference, src/soap_tp/ops/factorizations.py:446-469): ascending, input
    destroyed, lower triangle referenced.  Against LAPACK in fp64 on the same float32 matrix."""
    g = make_matrix(size, size + 5)
    matrix = g @ g.T
    a = column_major(torch.tril(matrix) + torch.triu(torch.full_like(matrix, 9.0), 1), device, pad=3)
    q = column_major(torch.zeros(size, size), device, pad=1)
    w = torch.zeros(size, dtype=torch.float32, device=device)
    nbytes = _native.library().soapmi_eigh_workspace_bytes(size, 4)
    work = torch.empty(max(1, nbytes), dtype=torch.uint8, device=device)
    _native.call("soapmi_eigh_f32", a.data_ptr(), w.data_ptr(), q.data_ptr(), size, a.stride(1), q.stride(1),
                 work.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
    exact = torch.tril(matrix).double()
    exact = exact + torch.tril(exact, -1).T
    expected = torch.linalg.eigvalsh(exact)
    scale = expected.abs().max().item()
    values, vectors = w.cpu().double(), q.cpu().double()
    assert torch.all(values[1:] >= values[:-1])
    assert (values - expected).abs().max().item() <= 1e-5 * scale
    assert (vectors.T @ vectors - torch.eye(size, dtype=torch.float64)).abs().max().item() <= 1e-4
    assert torch.linalg.matrix_norm(exact @ vectors - vectors * values).item() <= 5e-5 * torch.linalg.matrix_norm(exact).item()


@pytest.mark.parametrize("kind", ["clusters", "glued_wilkinson", "block_diagonal"])
def test_eigh_f64_with_heavy_deflation(kind, device):
    """Spectra that make the divide and conquer deflate: eigenvalues repeated in groups (rotations
    between columns of the two children of a merge), glued Wilkinson blocks (pairs that agree to
    working precision) and an exactly decoupled block-diagonal matrix (whole merges with nothing to
    solve).  Checked through invariants: spectrum against LAPACK, orthogonality, residual."""
    size = 520
    generator = torch.Generator().manual_seed(SEED + 91)
    if kind == "clusters":
        basis, _ = torch.linalg.qr(torch.randn(size, size, generator=generator, dtype=torch.float64))
        spectrum = torch.tensor([0.0, 1e-9, 0.5, 1.0, 1.0 + 1e-13, 2.0, 7.0, 7.5], dtype=torch.float64)
        matrix = (basis * spectrum[torch.randint(0, len(spectrum), (size,), generator=generator)]) @ basis.T
        matrix = (matrix + matrix.T) / 2
    elif kind == "glued_wilkinson":
        block = 21
        w21 = torch.diag((torch.arange(block) - block // 2).abs().double()) + torch.diag(torch.ones(block - 1), 1).double() \
            + torch.diag(torch.ones(block - 1), -1).double()
        copies = size // block + 1
        matrix = torch.block_diag(*[w21] * copies)[:size, :size].clone()
        for c in range(1, copies):  # weak glue between neighbouring blocks
            if c * block < size:
                matrix[c * block, c * block - 1] = matrix[c * block - 1, c * block] = 1e-8
    else:
        g = torch.randn(size // 2, size // 2, generator=generator, dtype=torch.float64)
        matrix = torch.block_diag(g + g.T, 3.0 * torch.eye(size - size // 2, dtype=torch.float64))
    a = column_major(torch.tril(matrix), device)
    q = torch.zeros(size, size, dtype=torch.float64, device=device).T
    w = torch.zeros(size, dtype=torch.float64, device=device)
    _native.call("soapmi_eigh_f64", a.data_ptr(), w.data_ptr(), q.data_ptr(), size, size, size, None, 0,
                 torch.cuda.current_stream().cuda_stream)
    expected = torch.linalg.eigvalsh(matrix)
    scale = max(expected.abs().max().item(), 1.0)
    assert torch.allclose(w.cpu(), expected, rtol=0, atol=1e-12 * scale * size)
    qc = q.cpu()
    assert (qc.T @ qc - torch.eye(size, dtype=torch.float64)).abs().max().item() < 1e-12
    assert (matrix @ qc - qc * w.cpu()).abs().max().item() < 1e-11 * scale


def test_injected_elpa_binding_follows_reference_staging(device):
    from soap_tp_amd.binding import NativeBinding

    class Counting(NativeBinding):
        calls = 0

        def elpa_eigenvectors_2d_block_cyclic_double(self, *args):
            type(self).calls += 1
            assert len(args) == 10 and args[3:6] == (13, 13, 13) and args[7:9] == (1, 1)
            return super().elpa_eigenvectors_2d_block_cyclic_double(*args)

    gram = make_matrix(13, 9) @ make_matrix(13, 9).T
    packed = column_major(gram, device)
    basis = ops.allocate_2d_block_cyclic((13, 13), BLOCK, GRID, device=device)
    work = ops.allocate_2d_block_cyclic((13, 13), BLOCK, GRID, device=device)
    values = torch.empty(13, device=device)
    ops.initialize_basis_2d_block_cyclic_(packed, basis, work, values, 13, BLOCK, GRID, elpa_binding=Counting())
    assert Counting.calls == 1
    _check_against_oracle(gram, values.cpu(), basis.cpu(), "elpa")
    padded = torch.zeros(13, 16, device=device).T[:13]
    with pytest.raises(ValueError, match="exact ELPA leading dimension"):
        ops.initialize_basis_2d_block_cyclic_(packed, basis, padded, values, 13, BLOCK, GRID)


def test_two_stage_and_one_stage_agree_at_2048(device):
    """The two tridiagonalisations on one float64 matrix of size 2048 (64 stage-1 panels, 2046 sweeps of
    the bulge chase): same spectrum to rounding, both with small residual and orthonormal vectors."""
    size = 2048
    gradient = oracle.low_rank_plus_noise(size, size + 512, 32, seed=SEED + 5).double()
    matrix = 0.05 * gradient @ gradient.T
    results = []
    try:
        for algorithm in (1, 2):
            _native.call("soapmi_set_option", b"eigh_algorithm", algorithm)
            a = column_major(torch.tril(matrix), device)
            q = torch.zeros(size, size, dtype=torch.float64, device=device).T
            w = torch.zeros(size, dtype=torch.float64, device=device)
            nbytes = _native.library().soapmi_eigh_workspace_bytes(size, 8)
            work = torch.empty(nbytes, dtype=torch.uint8, device=device)
            _native.call("soapmi_eigh_f64", a.data_ptr(), w.data_ptr(), q.data_ptr(), size, size, size, work.data_ptr(),
                         nbytes, torch.cuda.current_stream().cuda_stream)
            results.append((w.clone(), q.clone()))
    finally:
        _native.call("soapmi_set_option", b"eigh_algorithm", 1)
    scale = results[0][0].abs().max().item()
    assert (results[0][0] - results[1][0]).abs().max().item() <= 1e-12 * scale
    device_matrix = matrix.to(device)
    for w, q in results:
        assert torch.all(w[1:] >= w[:-1])
        assert ((device_matrix @ q - q * w).norm() / device_matrix.norm()).item() <= 1e-13
        assert (q.T @ q - torch.eye(size, dtype=torch.float64, device=device)).abs().max().item() <= 1e-12
