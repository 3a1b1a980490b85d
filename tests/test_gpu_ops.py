"""Op-level parity of the HIP path against the CPU oracle, on the inputs of the reference's own
unit tests (seed 42, N(0, 2), block size 2, shapes (8,8) (8,12) (12,8) (9,13) (13,9)) restated
for one rank, plus larger and ragged sizes.  Every call goes Python -> ctypes -> C ABI.

Tolerances (float32 path): relative L2 <= 1e-5 on products, Adam and Gram matrices -- the
reference's own bar (tests/unit/test_preconditioners.py:405-417, test_factorizations.py:345-373);
data movement (permute, layout copies, argsort) is exact."""
import math

import pytest
import torch

from oracle import soap_oracle as oracle
from soap_tp_amd import ops
from tests.helpers import (MATRIX_SHAPES, SEED, align_signs, column_major, make_matrix, make_orthogonal,
                           make_preconditioner, relative_l2)

pytestmark = pytest.mark.gpu
GRID = (1, 1)
BLOCK = 2
RTOL = 1e-5
EXTRA_SHAPES = ((1, 1), (1, 7), (130, 70), (256, 384), (300, 129))


# ---- Gram EMA (tests/unit/test_preconditioners.py of the reference) ------------------------------
@pytest.mark.parametrize("shape", MATRIX_SHAPES + EXTRA_SHAPES)
@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("shard_dim", [0, 1])
def test_preconditioner_update_from_zero(shape, side, shard_dim, device):
    gradient = make_matrix(*shape)
    size = shape[0] if side == "left" else shape[1]
    packed = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    update = (ops.update_left_preconditioner_2d_block_cyclic_ if side == "left"
              else ops.update_right_preconditioner_2d_block_cyclic_)
    result = update(gradient.to(device), packed, 0.0, BLOCK, GRID, shard_dim=shard_dim)
    assert result is packed
    expected = oracle.gram_ema(torch.zeros(size, size), gradient, 0.0, side)
    assert relative_l2(packed, expected) <= RTOL
    torch.testing.assert_close(packed.cpu(), expected, rtol=RTOL, atol=RTOL * expected.abs().max().item())
    assert torch.equal(packed, packed.T)  # both triangles, bit-identical mirror


@pytest.mark.parametrize("beta", [0.25, 0.95, 1.0])
def test_preconditioner_update_nonzero_beta(beta, device):
    gradient = make_matrix(9, 13, seed=SEED + 100)  # tests/unit/test_preconditioners.py:591-608
    packed = column_major(torch.full((9, 9), 2.0), device)
    ops.update_left_preconditioner_2d_block_cyclic_(gradient.to(device), packed, beta, BLOCK, GRID, shard_dim=0)
    expected = oracle.gram_ema(torch.full((9, 9), 2.0), gradient, beta, "left")
    assert relative_l2(packed, expected) <= RTOL


def test_preconditioner_lower_only_and_layouts(device):
    gradient = make_matrix(70, 130)
    start = make_preconditioner(130, SEED + 1)
    expected = oracle.gram_ema(start.clone(), gradient, 0.9, "right")
    lower = column_major(start, device, pad=3)
    upper_before = torch.triu(lower, 1).clone()
    ops.update_right_preconditioner_2d_block_cyclic_(gradient.to(device), lower, 0.9, BLOCK, GRID, shard_dim=1,
                                                     mirror=False)
    assert relative_l2(torch.tril(lower), torch.tril(expected)) <= RTOL
    assert torch.equal(torch.triu(lower, 1), upper_before)  # upper triangle untouched
    # a column-major (transposed-view) gradient takes the other operand layout
    full = column_major(start, device)
    ops.update_right_preconditioner_2d_block_cyclic_(gradient.to(device).T.contiguous().T, full, 0.9, BLOCK, GRID,
                                                     shard_dim=1)
    assert relative_l2(full, expected) <= RTOL
    half = column_major(start, device)
    ops.update_right_preconditioner_2d_block_cyclic_(gradient.to(device).half(), half, 0.9, BLOCK, GRID, shard_dim=1)
    assert relative_l2(half, oracle.gram_ema(start.clone(), gradient.half().float(), 0.9, "right")) <= RTOL


# ---- Adam (tests/unit/test_optimizer.py) ---------------------------------------------------------
@pytest.mark.parametrize("shape", MATRIX_SHAPES + ((257, 130),))
@pytest.mark.parametrize("layout", ["column_major", "row_major"])
def test_adam_update(shape, layout, device):
    step, beta1, beta2, eps = 3, 0.8, 0.9, 1e-6
    host = [make_matrix(*shape, seed=SEED), make_matrix(*shape, seed=SEED + 1),
            make_matrix(*shape, seed=SEED + 2).square()]
    expected_update = oracle.adam_update(host[0].clone(), m_ref := host[1].clone(), v_ref := host[2].clone(),
                                         step, beta1, beta2, eps)
    place = (lambda t: column_major(t, device)) if layout == "column_major" else (lambda t: t.to(device))
    gradient, momentum, variance = (place(t) for t in host)
    update = ops.adam_update(gradient, momentum, variance, step=step, beta1=beta1, beta2=beta2, eps=eps)
    assert update.shape == gradient.shape and update.stride() == variance.stride()
    assert relative_l2(update, expected_update) <= RTOL
    torch.testing.assert_close(momentum.cpu(), m_ref)
    torch.testing.assert_close(variance.cpu(), v_ref)
    torch.testing.assert_close(update.cpu(), expected_update)


# ---- permutation and layout copies ---------------------------------------------------------------
@pytest.mark.parametrize("shape", MATRIX_SHAPES + ((300, 129),))
def test_permute_and_redistribute_are_exact(shape, device):
    rows, columns = shape
    matrix = make_matrix(rows, columns)
    generator = torch.Generator().manual_seed(SEED)
    row_order, column_order = torch.randperm(rows, generator=generator), torch.randperm(columns, generator=generator)
    packed = ops.redistribute_tp_shard_to_2d_block_cyclic(matrix.to(device), shape, BLOCK, GRID, shard_dim=1)
    assert packed.stride(0) == 1 and torch.equal(packed.cpu(), matrix)
    result = ops.permute_2d_block_cyclic_(packed, shape, row_order.tolist(), column_order.to(device), BLOCK, GRID)
    assert result is packed
    assert torch.equal(packed.cpu(), oracle.permute(matrix, row_order, column_order))
    shard = ops.redistribute_2d_block_cyclic_to_tp_shard(packed, shape, BLOCK, GRID, shard_dim=0)
    assert shard.is_contiguous() and torch.equal(shard.cpu(), oracle.permute(matrix, row_order, column_order))
    with pytest.raises(ValueError, match="row_order must be a permutation"):
        ops.permute_2d_block_cyclic_(packed, shape, [0] * rows, column_order, BLOCK, GRID)
    with pytest.raises(ValueError, match="column_order must be a permutation"):
        ops.permute_2d_block_cyclic_(packed, shape, row_order, column_order[:-1], BLOCK, GRID)


@pytest.mark.parametrize("shape", [(1, 1), (9, 13), (64, 96), (300, 129), (1000, 257), (4100, 36)])
@pytest.mark.parametrize("orders", ["both", "rows", "columns", "neither"])
def test_gather_entry_point_is_exact(shape, orders, device):
    """soapmi_gather_f32, the out-of-place form of the permutation (out[i, j] = in[row_order[i],
    col_order[j]], src/soap_tp/ops/optimizer.py:408); a NULL order is the identity.  Padded leading
    dimensions on both sides; nothing may be written between the columns of the output."""
    from soap_tp_amd import _native

    rows, columns = shape
    matrix = make_matrix(rows, columns, seed=SEED + rows)
    generator = torch.Generator().manual_seed(SEED + columns)
    row_order = torch.randperm(rows, generator=generator) if orders in ("both", "rows") else None
    column_order = torch.randperm(columns, generator=generator) if orders in ("both", "columns") else None
    source = column_major(matrix, device, pad=2)
    target = column_major(torch.zeros(rows, columns), device, pad=5)
    device_rows = row_order.to(device) if row_order is not None else None
    device_columns = column_order.to(device) if column_order is not None else None
    _native.call("soapmi_gather_f32", source.data_ptr(), source.stride(1), target.data_ptr(), target.stride(1), rows,
                 columns, device_rows.data_ptr() if device_rows is not None else None,
                 device_columns.data_ptr() if device_columns is not None else None,
                 torch.cuda.current_stream().cuda_stream)
    expected = oracle.permute(matrix, row_order if row_order is not None else torch.arange(rows),
                              column_order if column_order is not None else torch.arange(columns))
    assert torch.equal(target.cpu(), expected)
    between = torch.as_strided(target, (5, columns), (1, rows + 5), target.storage_offset() + rows)
    assert torch.count_nonzero(between).item() == 0
    assert torch.equal(source.cpu(), matrix)  # the input is read only


@pytest.mark.parametrize("shape", [(8, 12), (13, 9), (96, 160), (256, 384), (1024, 1024), (700, 1300), (2048, 512)])
@pytest.mark.parametrize("row_major", [True, False])
@pytest.mark.parametrize("mirror", [True, False])
def test_gram_pair_equals_the_two_single_updates(shape, row_major, mirror, device):
    """soapmi_gram_ema_pair_f32 (both Gram updates of a step in one launch) against two calls of
    soapmi_gram_ema_f32: the same products element by element, so the results are equal bit for bit
    whichever tile either path picks."""
    from soap_tp_amd import _native
    rows, columns = shape
    gradient = make_matrix(rows, columns, seed=SEED + rows + columns)
    stored = gradient.to(device) if row_major else column_major(gradient, device)
    ldg = stored.stride(0) if row_major else stored.stride(1)
    stream = torch.cuda.current_stream().cuda_stream
    start_left = column_major(make_preconditioner(rows, SEED + 11), device)
    start_right = column_major(make_preconditioner(columns, SEED + 12), device)
    single = [start_left.clone(), start_right.clone()]
    for side in (0, 1):
        _native.call("soapmi_gram_ema_f32", stored.data_ptr(), rows, columns, ldg, 1 if row_major else 0, side,
                     single[side].data_ptr(), single[side].stride(1), 0.9, 1 if mirror else 0, stream)
    paired = [start_left.clone(), start_right.clone()]
    _native.call("soapmi_gram_ema_pair_f32", stored.data_ptr(), rows, columns, ldg, 1 if row_major else 0,
                 paired[0].data_ptr(), paired[0].stride(1), paired[1].data_ptr(), paired[1].stride(1), 0.9,
                 1 if mirror else 0, stream)
    for expected, actual in zip(single, paired):
        assert torch.equal(expected, actual)
    expected_left = oracle.gram_ema(make_preconditioner(rows, SEED + 11), gradient, 0.9, "left")
    assert relative_l2(torch.tril(paired[0]), torch.tril(expected_left)) <= RTOL


# ---- rotations (tests/unit/test_factorizations.py:376-399) ---------------------------------------
@pytest.mark.parametrize("shape", MATRIX_SHAPES + ((130, 70), (256, 384)))
@pytest.mark.parametrize("direction", ["forward", "backward"])
def test_rotate(shape, direction, device):
    rows, columns = shape
    matrix = make_matrix(rows, columns, seed=SEED + rows * 100 + columns)
    q_left, q_right = make_orthogonal(rows, SEED + 1000 + rows), make_orthogonal(columns, SEED + 2000 + columns)
    packed = column_major(matrix, device, pad=1)
    result = ops.rotate_2d_block_cyclic_(packed, column_major(q_left, device), column_major(q_right, device, pad=2),
                                         shape, BLOCK, GRID, direction=direction)
    assert result is packed
    expected = oracle.rotate(matrix, q_left, q_right, direction)
    assert relative_l2(packed, expected) <= RTOL
    torch.testing.assert_close(packed.cpu(), expected, rtol=2e-4, atol=2e-4)
    assert abs(packed.norm().item() / matrix.norm().item() - 1) < 1e-5  # orthogonal invariance


# ---- the product every MFMA stage runs on, through its own entry point ---------------------------
# Closed form: C = alpha op(A) op(B) + beta C in fp64 on the CPU (what SLATE's gemm computes for the
# reference's rotations, src/soap_tp/csrc/slate_bindings.cpp:257-273).  Shapes pick every path of the
# kernel: the general path (odd sizes, padded leading dimensions), the 128 x 128 fast path, and the
# 64 x 64 tile's fast path with K = 1 .. 9 slabs of 32 (its loop is peeled into a part that keeps two
# slabs in flight and a tail; K = 32, 64, 96 have no steady part, 128 and 160 one pass of it, ...).
PRODUCT_SHAPES = ((1, 1, 1), (3, 5, 7), (65, 33, 17), (130, 70, 200), (128, 128, 16), (256, 384, 64),
                  (2048, 2048, 48), (2048, 2048, 256)) + tuple((64, 128, 32 * slabs) for slabs in range(1, 10)) + (
                  (192, 64, 1024), (300, 129, 96))


@pytest.mark.parametrize("shape", PRODUCT_SHAPES)
@pytest.mark.parametrize("transposes", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_product_entry_point(shape, transposes, dtype, device):
    from soap_tp_amd import _native

    m, n, k = shape
    trans_a, trans_b = transposes
    if dtype == torch.float64 and m * n * k > 2048 * 2048 * 48:
        pytest.skip("the fp64 product takes the same code path at the smaller size")
    a = make_matrix(k if trans_a else m, m if trans_a else k, seed=SEED + m + 3 * k, dtype=dtype)
    b = make_matrix(n if trans_b else k, k if trans_b else n, seed=SEED + n + 5 * k, dtype=dtype)
    c = make_matrix(m, n, seed=SEED + m * n, dtype=dtype)
    name = "soapmi_gemm_f32" if dtype == torch.float32 else "soapmi_gemm_f64"
    tolerance = RTOL if dtype == torch.float32 else 1e-13
    for alpha, beta, pad in ((1.0, 0.0, 0), (-0.5, 1.0, 0), (2.0, -0.25, 3)):
        stored_a, stored_b = column_major(a, device, pad=pad), column_major(b, device, pad=2 * pad)
        stored_c = column_major(c, device, pad=pad)
        _native.call(name, trans_a, trans_b, m, n, k, alpha, stored_a.data_ptr(), stored_a.stride(1),
                     stored_b.data_ptr(), stored_b.stride(1), beta, stored_c.data_ptr(), stored_c.stride(1),
                     torch.cuda.current_stream().cuda_stream)
        op_a = a.double().T if trans_a else a.double()
        op_b = b.double().T if trans_b else b.double()
        expected = alpha * (op_a @ op_b) + beta * c.double()
        assert relative_l2(stored_c, expected) <= tolerance, (alpha, beta, pad)
        if pad:  # nothing was written between the columns
            between = torch.as_strided(stored_c, (pad, n), (1, m + pad), stored_c.storage_offset() + m)
            assert torch.count_nonzero(between).item() == 0


# ---- order, QR, power iteration (tests/unit/test_slate_bindings.py) ------------------------------
@pytest.mark.parametrize("size", [8, 12, 9, 13, 100, 257])
def test_estimated_order_qr_and_power_iteration(size, device):
    preconditioner, basis = make_preconditioner(size, SEED + 5000), make_orthogonal(size, SEED + 7000)
    expected_order, expected_estimates, expected_work = oracle.estimated_order(preconditioner, basis)
    p_dev, q_dev = column_major(preconditioner, device), column_major(basis, device)
    work = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    order = ops.estimated_eigenvalue_order_2d_block_cyclic_(p_dev, q_dev, work, size, BLOCK, GRID)
    assert order.dtype == torch.int64 and order.tolist() == expected_order.tolist()
    assert relative_l2(work, expected_work) <= RTOL

    matrix = make_matrix(size, size, seed=SEED + size)
    factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    assert ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID) is factor
    expected_q = oracle.householder_qr(matrix)
    assert relative_l2(factor, expected_q) <= 5e-5  # same sign convention: no alignment needed
    torch.testing.assert_close(factor.T @ factor, torch.eye(size, device=device), rtol=1e-4, atol=1e-4)
    r = factor.double().T.cpu() @ matrix.double()
    assert torch.tril(r, -1).abs().max().item() <= 1e-4 * matrix.abs().max().item() * math.sqrt(size)

    returned = ops.power_iteration_qr_2d_block_cyclic_(p_dev, q_dev, work, size, BLOCK, GRID)
    expected_order2, expected_basis = oracle.power_iteration_qr(preconditioner, basis)
    assert returned.tolist() == expected_order2.tolist()
    signs = align_signs(q_dev.cpu(), expected_basis)
    assert relative_l2(q_dev.cpu() * signs, expected_basis) <= 1e-4
    torch.testing.assert_close(q_dev.T @ q_dev, torch.eye(size, device=device), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("size", [40, 300, 700])
def test_qr_launch_per_column_panel_path(size, device):
    """The panel factorisation used beyond 128 workgroups (n > 32768), forced at small sizes."""
    from soap_tp_amd import _native
    matrix = make_matrix(size, size, seed=SEED + 31 * size)
    results = []
    try:
        for limit in (0, 128):
            _native.call("soapmi_set_option", b"qr_persistent_max_workgroups", limit)
            factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
            results.append(factor.cpu())
    finally:
        _native.call("soapmi_set_option", b"qr_persistent_max_workgroups", 128)
    expected_q = oracle.householder_qr(matrix)
    for factor in results:
        assert relative_l2(factor, expected_q) <= 5e-5
        torch.testing.assert_close(factor.T @ factor, torch.eye(size), rtol=1e-4, atol=1e-4)
    assert relative_l2(results[0], results[1]) <= 1e-5
    with pytest.raises(ValueError):
        _native.call("soapmi_set_option", b"qr_persistent_max_workgroups", 129)


@pytest.mark.parametrize("size", [96, 300, 545, 1000, 1312])
def test_qr_update_riding_along_with_the_next_panel(size, device):
    """A panel's update of the rest of its 256-column block either rides along in the next panel's
    launch (the default) or is a launch of its own: the same sums in the same order, so the same bits.
    Sizes with a last panel narrower than 32 columns take the separate launch for that panel."""
    from soap_tp_amd import _native
    matrix = make_matrix(size, size, seed=SEED + 7 * size)
    results = []
    try:
        for carried in (0, 1):
            _native.call("soapmi_set_option", b"qr_carry_update", carried)
            factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
            results.append(factor.cpu())
    finally:
        _native.call("soapmi_set_option", b"qr_carry_update", 1)
    assert relative_l2(results[1], oracle.householder_qr(matrix)) <= 5e-5
    assert torch.equal(results[0], results[1])
    with pytest.raises(ValueError):
        _native.call("soapmi_set_option", b"qr_carry_update", 2)


@pytest.mark.parametrize("size", [200, 600, 1300])
def test_qr_with_padded_leading_dimensions(size, device):
    """soapmi_qr_f32 called directly with leading dimensions larger than n, for the matrix and for Q:
    the factorisation then cannot use the matrix's own columns as the reflector block of the Q formation."""
    from soap_tp_amd import _native
    matrix = make_matrix(size, size, seed=SEED + 3 * size)
    lda, ldq = size + 24, size + 8
    a_store = torch.full((size, lda), float("nan"), device=device)
    q_store = torch.full((size, ldq), float("nan"), device=device)
    a_store[:, :size] = matrix.T.to(device)  # column j of the matrix in row j of the store: column-major with ld = lda
    need = _native.library().soapmi_qr_workspace_bytes(size)
    work = torch.empty(need, dtype=torch.uint8, device=device)
    _native.call("soapmi_qr_f32", a_store.data_ptr(), q_store.data_ptr(), size, lda, ldq, work.data_ptr(), need,
                 torch.cuda.current_stream().cuda_stream)
    factor = q_store[:, :size].T.cpu()
    assert bool(torch.isnan(q_store[:, size:]).all())  # the padding is not written
    assert relative_l2(factor, oracle.householder_qr(matrix)) <= 5e-5
    torch.testing.assert_close(factor.T @ factor, torch.eye(size), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("size", [289, 545, 1000])
def test_qr_block_reflector_widths(size, device):
    """Sizes whose last 256-column block reflector has a width that is no multiple of 32, 64 or 128:
    the factor T of such a block is assembled from unequal spans (33 = 32 + 1, 232 = 128 + 64 + 32 + 8)."""
    matrix = make_matrix(size, size, seed=SEED + 17 * size)
    factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
    ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
    expected_q = oracle.householder_qr(matrix)
    assert relative_l2(factor, expected_q) <= 5e-5
    torch.testing.assert_close(factor.T @ factor, torch.eye(size, device=device), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("size", [300, 1000, 1057, 1312, 2304, 2500])
def test_qr_super_blocks(size, device):
    """Three blocking levels (256-column blocks applied inside 1024-column super-blocks, the matrix beyond
    updated once per super-block with K = 1024) against two: both against LAPACK's Householder QR, and
    against each other.  Sizes with one, two and three super-blocks, the last one a full 1024 columns,
    33, 288, 256 and 452 wide (its T factor is then assembled from unequal spans)."""
    from soap_tp_amd import _native
    matrix = make_matrix(size, size, seed=SEED + 11 * size)
    results = {}
    try:
        for width in (256, 1024, 0):
            _native.call("soapmi_set_option", b"qr_super_block", width)
            factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
            results[width] = factor.cpu()
    finally:
        _native.call("soapmi_set_option", b"qr_super_block", 0)
    expected_q = oracle.householder_qr(matrix)
    for width, factor in results.items():
        assert relative_l2(factor, expected_q) <= 5e-5, width
        torch.testing.assert_close(factor.T @ factor, torch.eye(size), rtol=1e-4, atol=1e-4)
        r = factor.double().T @ matrix.double()
        assert torch.tril(r, -1).abs().max().item() <= 1e-4 * matrix.abs().max().item() * math.sqrt(size)
    assert torch.equal(results[0], results[1024])  # sizes up to 4096 take three levels when left to the library
    with pytest.raises(ValueError):
        _native.call("soapmi_set_option", b"qr_super_block", 512)


@pytest.mark.parametrize("kind", ["paired_columns", "graded", "rank_deficient", "repeated_column"])
def test_qr_super_blocks_on_hard_matrices(kind, device):
    """The hard matrices of the test below at a size with two super-blocks, three blocking levels forced."""
    from soap_tp_amd import _native
    size = 1400
    generator = torch.Generator().manual_seed(SEED + 321)
    matrix = torch.randn(size, size, generator=generator)
    if kind == "paired_columns":
        matrix[:, 1::2] = matrix[:, 0::2] + 1e-4 * torch.randn(size, size // 2, generator=generator)
    elif kind == "graded":
        matrix = matrix * torch.logspace(0, -12, size)[None, :]
    elif kind == "rank_deficient":
        matrix = matrix[:, :40] @ torch.randn(40, size, generator=generator)
    else:
        matrix[:, 1:64] = matrix[:, :1]
    try:
        _native.call("soapmi_set_option", b"qr_super_block", 1024)
        factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
        ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
    finally:
        _native.call("soapmi_set_option", b"qr_super_block", 0)
    q = factor.cpu().double()
    a = matrix.double()
    assert torch.isfinite(q).all()
    assert (q.T @ q - torch.eye(size, dtype=torch.float64)).abs().max().item() <= 2e-5
    r = torch.triu(q.T @ a)
    column_norms = a.norm(dim=0).clamp_min(1e-300)
    assert ((a - q @ r).norm(dim=0) / column_norms).max().item() <= 2e-5  # column-wise backward error


@pytest.mark.parametrize("kind", ["paired_columns", "graded", "rank_deficient", "repeated_column"])
@pytest.mark.parametrize("columns_per_round", [1, 2, 3, 4, 32])
def test_qr_is_backward_stable_on_hard_matrices(kind, columns_per_round, device):
    """Orthogonality of Q and the backward error of A = Q R on matrices built to hurt a panel that
    derives a column's norm from dot products: neighbouring columns that are nearly parallel,
    columns graded over twelve orders of magnitude, exact rank deficiency, exact repeats."""
    from soap_tp_amd import _native
    size = 600
    generator = torch.Generator().manual_seed(SEED + 123)
    matrix = torch.randn(size, size, generator=generator)
    if kind == "paired_columns":
        matrix[:, 1::2] = matrix[:, 0::2] + 1e-4 * torch.randn(size, size // 2, generator=generator)
    elif kind == "graded":
        matrix = matrix * torch.logspace(0, -12, size)[None, :]
    elif kind == "rank_deficient":
        matrix = matrix[:, :40] @ torch.randn(40, size, generator=generator)
    else:
        matrix[:, 1:64] = matrix[:, :1]
    try:
        _native.call("soapmi_set_option", b"qr_columns_per_round", columns_per_round)
        factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
        ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
    finally:
        _native.call("soapmi_set_option", b"qr_columns_per_round", 32)
    q = factor.cpu().double()
    a = matrix.double()
    assert torch.isfinite(q).all()
    assert (q.T @ q - torch.eye(size, dtype=torch.float64)).abs().max().item() <= 2e-5
    r = torch.triu(q.T @ a)
    column_norms = a.norm(dim=0).clamp_min(1e-300)
    assert ((a - q @ r).norm(dim=0) / column_norms).max().item() <= 2e-5  # column-wise backward error


def test_lost_messages_poison_the_result_instead_of_hanging(device):
    """With no patience for another workgroup's message (spin limit 0) the persistent kernels leave
    early; the outputs must then be NaN-poisoned or, if every message happened to be there at the
    first poll, correct - never silently wrong - and the next call with the default limit is clean."""
    from soap_tp_amd import _native
    size = 700  # three workgroups of 256 rows
    matrix = make_matrix(size, size, seed=SEED + 77)
    symmetric = make_preconditioner(size, SEED + 78).double()
    expected_q = oracle.householder_qr(matrix)
    expected_values = torch.linalg.eigvalsh(symmetric)

    def run():
        factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
        ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
        a = column_major(symmetric, device)
        values = torch.empty(size, dtype=torch.float64, device=device)
        vectors = torch.empty(size, size, dtype=torch.float64, device=device).T
        _native.call("soapmi_eigh_f64", a.data_ptr(), values.data_ptr(), vectors.data_ptr(), size, a.stride(1),
                     vectors.stride(1), 0, 0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return factor.cpu(), values.cpu()

    assert not _native.device_error_flag(clear=True)
    try:
        _native.call("soapmi_set_option", b"message_spin_limit", 0)
        factor, values = run()
    finally:
        _native.call("soapmi_set_option", b"message_spin_limit", 1 << 22)
        reported = _native.device_error_flag(clear=True)  # cleared: later tests start clean
    assert torch.isnan(factor).any() or relative_l2(factor, expected_q) <= 5e-5
    assert torch.isnan(values).all() or relative_l2(values, expected_values) <= 1e-12
    # the host learns of a failure without looking at the data: the report word is up exactly when
    # something was poisoned
    assert reported == bool(torch.isnan(factor).any() or torch.isnan(values).any())
    factor, values = run()
    assert relative_l2(factor, expected_q) <= 5e-5
    assert relative_l2(values, expected_values) <= 1e-12
    assert not _native.device_error_flag(clear=True)


def test_soap_step_raises_after_a_factorisation_failed_on_the_device(device):
    """A refresh whose QR gives up (spin limit 0, several workgroups) leaves NaN-poisoned bases; the
    next call of soap_step on that state must raise instead of computing with them, and so must
    every call after it.  If every message happened to be there at the first poll nothing failed
    and nothing may be raised.  The failure is the state's own: the device-wide flag stays down."""
    import soap_tp_amd
    from soap_tp_amd import _native, state_io
    shape = (700, 520)
    generator = torch.Generator().manual_seed(SEED + 79)
    state = {}
    kwargs = dict(global_shape=shape, shard_dim=1, block_size=128, process_grid_shape=GRID, basis_refresh_interval=2)
    assert not _native.device_error_flag(clear=True)
    for _ in range(2):
        soap_tp_amd.soap_step(torch.randn(*shape, generator=generator).to(device), state, **kwargs)
    try:
        _native.call("soapmi_set_option", b"message_spin_limit", 0)
        soap_tp_amd.soap_step(torch.randn(*shape, generator=generator).to(device), state, **kwargs)  # refreshes
        torch.cuda.synchronize()
    finally:
        _native.call("soapmi_set_option", b"message_spin_limit", 1 << 22)
    poisoned = bool(torch.isnan(state["left_basis"]).any() or torch.isnan(state["right_basis"]).any())
    assert bool(state["status"][0] != 0) == poisoned
    gradient = torch.randn(*shape, generator=generator).to(device)
    if poisoned:
        for _ in range(2):
            with pytest.raises(RuntimeError, match="gave up waiting"):
                soap_tp_amd.soap_step(gradient, state, **kwargs)
        with pytest.raises(ValueError, match="failed on the device"):
            state_io.pack_state(state)
    else:
        soap_tp_amd.soap_step(gradient, state, **kwargs)
    assert not _native.device_error_flag(clear=True)


def test_a_failed_factorisation_is_attributed_to_its_state(device):
    """Two parameters on one device.  One parameter's refresh runs with no patience for messages (spin
    limit 0 during that call only; every kernel still exits normally).  Only that parameter's state
    may raise afterwards; the other one keeps stepping, through its own refreshes too, and its
    results equal those of a run in which nothing failed."""
    import soap_tp_amd
    from soap_tp_amd import _native
    shapes = {"a": (700, 520), "b": (520, 700)}
    kwargs = {name: dict(global_shape=shape, shard_dim=1, block_size=128, process_grid_shape=GRID,
                         basis_refresh_interval=2) for name, shape in shapes.items()}
    generator = torch.Generator().manual_seed(SEED + 81)
    gradients = {name: [torch.randn(*shape, generator=generator).to(device) for _ in range(7)]
                 for name, shape in shapes.items()}

    def run(fail):
        states = {"a": {}, "b": {}}
        updates = []
        raised = False
        for t in range(7):
            for name in ("a", "b"):
                failing = fail and name == "a" and t == 2  # the first refresh of parameter a
                try:
                    if failing:
                        _native.call("soapmi_set_option", b"message_spin_limit", 0)
                    try:
                        update = soap_tp_amd.soap_step(gradients[name][t], states[name], **kwargs[name])
                    except RuntimeError as error:
                        assert name == "a" and t > 2 and "gave up waiting" in str(error)
                        raised = True
                        continue
                    if failing:
                        torch.cuda.synchronize()
                finally:
                    if failing:
                        _native.call("soapmi_set_option", b"message_spin_limit", 1 << 22)
                if name == "b":
                    updates.append(update.cpu())
        return states, updates, raised

    assert not _native.device_error_flag(clear=True)
    clean_states, clean_updates, clean_raised = run(fail=False)
    assert not clean_raised
    states, updates, raised = run(fail=True)
    poisoned = bool(torch.isnan(states["a"]["left_basis"]).any() or torch.isnan(states["a"]["right_basis"]).any())
    assert raised == poisoned  # (all messages there at the first poll: nothing failed, nothing raised)
    assert int(states["b"]["status"][0]) == 0 and int(states["b"]["step"]) == 6
    assert len(updates) == len(clean_updates) == 7
    for update, clean in zip(updates, clean_updates):
        assert torch.equal(update, clean)
    assert not _native.device_error_flag(clear=True)  # the device-wide word was never involved


def test_status_word_through_the_c_abi(device):
    """soapmi_set_status_word called directly: while a caller-owned word (pinned host memory) is set for this
    thread, a factorisation that gives up raises that word and leaves the device-wide one alone; after
    NULL the device-wide word is back in charge.  (Spin limit 0 makes the kernels give up without
    waiting; every kernel exits normally.)"""
    from soap_tp_amd import _native
    size = 700
    matrix = make_matrix(size, size, seed=SEED + 83)
    word = torch.zeros(1, dtype=torch.int32, pin_memory=True)
    stream = torch.cuda.current_stream().cuda_stream
    need = _native.library().soapmi_qr_workspace_bytes(size)
    work = torch.empty(need, dtype=torch.uint8, device=device)

    def qr():
        a, q = column_major(matrix, device), torch.empty(size, size, device=device).T
        _native.call("soapmi_qr_f32", a.data_ptr(), q.data_ptr(), size, a.stride(1), q.stride(1), work.data_ptr(), need,
                     stream)
        torch.cuda.synchronize()
        return q

    assert not _native.device_error_flag(clear=True)
    try:
        _native.call("soapmi_set_option", b"message_spin_limit", 0)
        _native.call("soapmi_set_status_word", word.data_ptr())
        with_word = qr()
        _native.call("soapmi_set_status_word", 0)
        assert not _native.device_error_flag(clear=True)  # whatever happened went to the caller's word
        assert bool(word[0] != 0) == bool(torch.isnan(with_word).any())
        without_word = qr()
        assert _native.device_error_flag(clear=True) == bool(torch.isnan(without_word).any())
    finally:
        _native.call("soapmi_set_status_word", 0)
        _native.call("soapmi_set_option", b"message_spin_limit", 1 << 22)
        _native.device_error_flag(clear=True)
    word.zero_()
    _native.call("soapmi_set_status_word", word.data_ptr())
    try:
        clean = qr()
    finally:
        _native.call("soapmi_set_status_word", 0)
    assert int(word[0]) == 0 and relative_l2(clean.cpu(), oracle.householder_qr(matrix)) <= 5e-5


@pytest.mark.parametrize("budget", [256, 20])
def test_factorisations_on_several_streams_share_the_chip_safely(budget, device):
    """Four QR factorisations of 4096 x 4096 matrices (16 workgroups each in their panel kernels) and
    two eigensolves enqueued back to back on separate streams.  With the default budget of resident
    persistent workgroups all of them fit side by side; with a budget of 20 each has to wait, on the
    device, for the one before.  Either way every result must equal the one computed alone, bit for
    bit, and nothing may be reported as failed."""
    from soap_tp_amd import _native
    size = 4096
    matrices = [make_matrix(size, size, seed=SEED + 300 + i) for i in range(4)]
    symmetric = [make_preconditioner(2048, SEED + 400 + i).double() for i in range(2)]

    def qr_on(stream, matrix):
        with torch.cuda.stream(stream):
            factor = ops.allocate_2d_block_cyclic((size, size), BLOCK, GRID, device=device)
            ops.qr_2d_block_cyclic_(column_major(matrix, device), factor, size, BLOCK, GRID)
        return factor

    def eigh_on(stream, matrix):
        n = matrix.shape[0]
        with torch.cuda.stream(stream):
            a = column_major(matrix, device)
            values = torch.empty(n, dtype=torch.float64, device=device)
            vectors = torch.empty(n, n, dtype=torch.float64, device=device).T
            nbytes = _native.library().soapmi_eigh_workspace_bytes(n, 8)
            work = torch.empty(nbytes, dtype=torch.uint8, device=device)
            _native.call("soapmi_eigh_f64", a.data_ptr(), values.data_ptr(), vectors.data_ptr(), n, a.stride(1),
                         vectors.stride(1), work.data_ptr(), nbytes, stream.cuda_stream)
        return values, vectors, work, a

    main = torch.cuda.current_stream(device)
    alone = [qr_on(main, matrix) for matrix in matrices]
    alone_eigh = [eigh_on(main, matrix)[:2] for matrix in symmetric]
    torch.cuda.synchronize()
    assert not _native.device_error_flag(clear=True)
    streams = [torch.cuda.Stream(device=device) for _ in range(6)]
    try:
        _native.call("soapmi_set_option", b"persistent_workgroup_budget", budget)
        together = [qr_on(stream, matrix) for stream, matrix in zip(streams, matrices)]
        together_eigh = [eigh_on(stream, matrix) for stream, matrix in zip(streams[4:], symmetric)]
        torch.cuda.synchronize()
    finally:
        _native.call("soapmi_set_option", b"persistent_workgroup_budget", 256)
    assert not _native.device_error_flag(clear=True)
    for expected, actual in zip(alone, together):
        assert torch.isfinite(actual).all()
        assert torch.equal(expected, actual)
    for (values, vectors), result in zip(alone_eigh, together_eigh):
        assert torch.equal(values, result[0]) and torch.equal(vectors, result[1])
    # and one of them against the oracle
    q = together[0].double()
    a = matrices[0].double().to(device)
    identity_error = q.T @ q
    identity_error.diagonal().sub_(1.0)
    assert identity_error.abs().max().item() <= 1e-4
    r = torch.triu(q.T @ a)
    assert ((a - q @ r).norm(dim=0) / a.norm(dim=0)).max().item() <= 2e-5


def test_argsort_ties_and_large(device):
    from soap_tp_amd import _native
    for count in (1, 2, 33, 4096, 16384, 20000):
        keys = torch.randn(count, generator=torch.Generator().manual_seed(count))
        if count > 10:
            keys[3] = keys[7] = keys[9]
        order = torch.empty(count, dtype=torch.int64, device=device)
        keys_dev = keys.to(device)
        nbytes = _native.library().soapmi_argsort_workspace_bytes(count)
        work = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _native.call("soapmi_argsort_desc_f32", keys_dev.data_ptr(), count, order.data_ptr(), work.data_ptr(),
                     work.numel(), torch.cuda.current_stream().cuda_stream)
        assert order.tolist() == torch.argsort(keys, descending=True, stable=True).tolist()
    # NaNs go first in index order (as torch.argsort(descending=True) places them), signed zeros tie,
    # infinities order like numbers
    special = torch.tensor([0.0, float("nan"), -0.0, float("inf"), -1.0, float("-inf"), 0.0, float("nan"), 2.5, -0.0])
    order = torch.empty(special.numel(), dtype=torch.int64, device=device)
    special_dev = special.to(device)
    _native.call("soapmi_argsort_desc_f32", special_dev.data_ptr(), special.numel(), order.data_ptr(), None, 0,
                 torch.cuda.current_stream().cuda_stream)
    assert order.tolist() == [1, 7, 3, 8, 0, 2, 6, 9, 4, 5]
    assert order.tolist() == torch.argsort(special, descending=True, stable=True).tolist()


# ---- refresh (tests/unit/test_factorizations.py:501-613) -----------------------------------------
@pytest.mark.parametrize("shape", MATRIX_SHAPES + ((130, 70),))
@pytest.mark.parametrize("storage", ["full", "lower"])
def test_refresh_bases_and_transport_optimizer_state(shape, storage, device):
    rows, columns = shape
    state = {
        "momentum": make_matrix(rows, columns, seed=SEED + 3000),
        "variance": make_matrix(rows, columns, seed=SEED + 4000).square(),
        "left_preconditioner": make_preconditioner(rows, SEED + 5000),
        "right_preconditioner": make_preconditioner(columns, SEED + 6000),
        "left_basis": make_orthogonal(rows, SEED + 7000),
        "right_basis": make_orthogonal(columns, SEED + 8000),
    }
    dev = {name: column_major(t, device) for name, t in state.items()}
    if storage == "lower":  # the upper triangles hold stale values until the refresh rebuilds them
        for side in ("left", "right"):
            p = dev[f"{side}_preconditioner"]
            p.copy_(torch.tril(p) + torch.triu(torch.full_like(p, 3.0), 1))
    left_work = ops.allocate_2d_block_cyclic((rows, rows), BLOCK, GRID, device=device)
    right_work = ops.allocate_2d_block_cyclic((columns, columns), BLOCK, GRID, device=device)
    left_order, right_order = ops.refresh_bases_and_transport_optimizer_state_(
        dev["momentum"], dev["variance"], dev["left_preconditioner"], dev["right_preconditioner"],
        dev["left_basis"], dev["right_basis"], left_work, right_work, shape, BLOCK, GRID,
        symmetrize=(storage == "lower"))
    expected_left, expected_right = oracle.refresh(state)
    assert left_order.tolist() == expected_left.tolist() and right_order.tolist() == expected_right.tolist()
    left_signs = align_signs(dev["left_basis"].cpu(), state["left_basis"])
    right_signs = align_signs(dev["right_basis"].cpu(), state["right_basis"])
    assert relative_l2(dev["left_basis"].cpu() * left_signs, state["left_basis"]) <= 1e-4
    assert relative_l2(dev["right_basis"].cpu() * right_signs, state["right_basis"]) <= 1e-4
    assert relative_l2(dev["momentum"].cpu() * left_signs[:, None] * right_signs[None, :], state["momentum"]) <= 1e-4
    assert torch.equal(dev["variance"].cpu(), state["variance"])
    for side, size in (("left", rows), ("right", columns)):
        q = dev[f"{side}_basis"]
        torch.testing.assert_close(q.T @ q, torch.eye(size, device=device), rtol=1e-4, atol=1e-4)
        if storage == "lower":  # the refresh rebuilt the upper triangle from the lower one
            p = dev[f"{side}_preconditioner"]
            assert torch.equal(p, p.T)


def test_refresh_on_one_stream_gives_the_same_bits(device):
    """`refresh_streams` only changes where the two factorisation chains are enqueued."""
    from soap_tp_amd import _native
    rows, columns = 300, 520
    results = []
    try:
        for streams in (2, 1):
            _native.call("soapmi_set_option", b"refresh_streams", streams)
            dev = {
                "momentum": column_major(make_matrix(rows, columns, seed=SEED + 3000), device),
                "variance": column_major(make_matrix(rows, columns, seed=SEED + 4000).square(), device),
                "left_preconditioner": column_major(make_preconditioner(rows, SEED + 5000), device),
                "right_preconditioner": column_major(make_preconditioner(columns, SEED + 6000), device),
                "left_basis": column_major(make_orthogonal(rows, SEED + 7000), device),
                "right_basis": column_major(make_orthogonal(columns, SEED + 8000), device),
            }
            left_work = ops.allocate_2d_block_cyclic((rows, rows), BLOCK, GRID, device=device)
            right_work = ops.allocate_2d_block_cyclic((columns, columns), BLOCK, GRID, device=device)
            orders = ops.refresh_bases_and_transport_optimizer_state_(
                dev["momentum"], dev["variance"], dev["left_preconditioner"], dev["right_preconditioner"],
                dev["left_basis"], dev["right_basis"], left_work, right_work, (rows, columns), BLOCK, GRID)
            results.append(([o.tolist() for o in orders], {name: t.cpu() for name, t in dev.items()}))
    finally:
        _native.call("soapmi_set_option", b"refresh_streams", 2)
    assert results[0][0] == results[1][0]
    for name in results[0][1]:
        assert torch.equal(results[0][1][name], results[1][1][name]), name
    with pytest.raises(ValueError):
        _native.call("soapmi_set_option", b"refresh_streams", 3)
