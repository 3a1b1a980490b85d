"""Shared test utilities: seeded inputs in the style of the reference's unit tests
(seed 42, ``torch.normal(0, 2)``; tests/unit/test_factorizations.py:116-125 of the reference),
error measures, and sign/subspace-invariant basis comparisons."""
import math

import torch

SEED = 42
# the five op-level shapes of the reference's unit tests (tests/unit/test_optimizer.py:11-17)
MATRIX_SHAPES = ((8, 8), (8, 12), (12, 8), (9, 13), (13, 9))


def make_matrix(rows, columns, seed=SEED, dtype=torch.float32):
    generator = torch.Generator().manual_seed(seed)
    return torch.normal(mean=0, std=2, size=(rows, columns), generator=generator, dtype=dtype)


def make_orthogonal(size, seed):
    q, r = torch.linalg.qr(make_matrix(size, size, seed=seed, dtype=torch.float64))
    return (q * torch.sign(torch.diagonal(r))).to(torch.float32)


def make_preconditioner(size, seed):
    g = make_matrix(size, size + 3, seed=seed)
    return g @ g.T


def relative_l2(actual, reference):
    difference = torch.linalg.vector_norm(actual.double().cpu() - reference.double().cpu()).item()
    norm = torch.linalg.vector_norm(reference.double().cpu()).item()
    if norm == 0.0:
        return 0.0 if difference == 0.0 else math.inf
    return difference / norm


def column_major(tensor, device=None, pad=0):
    """Copy of ``tensor`` in packed column-major storage (stride (1, rows + pad))."""
    rows, columns = tensor.shape
    storage = torch.zeros((max(1, columns), max(1, rows) + pad), dtype=tensor.dtype, device=device or tensor.device)
    view = storage.T[:rows] if pad else storage.T
    view[:rows, :columns].copy_(tensor)
    return view


def align_signs(actual, reference):
    """Per-column signs that map ``actual`` onto ``reference``
    (tests/unit/test_factorizations.py:582-585 of the reference)."""
    signs = torch.sign(torch.sum(reference.double() * actual.double(), dim=0))
    signs[signs == 0] = 1
    return signs.to(actual.dtype)


def eigen_clusters(values, rel_gap):
    """Index ranges of eigenvalues (sorted descending) closer than rel_gap * max|value|."""
    values = values.double()
    scale = values.abs().max().item() or 1.0
    clusters, start = [], 0
    for i in range(1, len(values) + 1):
        if i == len(values) or abs(values[i - 1].item() - values[i].item()) > rel_gap * scale:
            clusters.append((start, i))
            start = i
    return clusters


def subspace_distance(basis_a, basis_b):
    """Spectral norm of the difference of the orthogonal projectors onto two column spaces."""
    a, b = basis_a.double().cpu(), basis_b.double().cpu()
    return torch.linalg.matrix_norm(a @ a.T - b @ b.T, ord=2).item()
