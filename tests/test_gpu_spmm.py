"""GPU parity of the sum-of-products SpMM (mamtorch_kernel_sparsev1::cusparsemm) through the C ABI and
through the operator.  The reference checks it by printing the max-abs error against the dense
``a @ b`` (test/test_sparse.py:33-44); here every cell must be within rtol 1e-5 of the fp64 oracle plus
the rounding floor of an fp32 sum in any order, 2^-22 x the sum of |terms| of that cell."""
import numpy as np
import ctypes

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _random_sparse(rows, k, sparse_rate, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(rows, k, generator=g)
    return a * torch.bernoulli(torch.full((rows, k), 1 - sparse_rate), generator=g)


def _check(got, want, floor, what):
    err = np.abs(got.cpu().numpy().astype(np.float64) - want)
    bound = 1e-5 * np.abs(want) + 2.0 ** -22 * floor + 1e-30
    assert (err <= bound).all(), "%s: worst excess %g at %s" % (what, (err - bound).max(),
                                                                 np.unravel_index((err - bound).argmax(), err.shape))


SHAPES = [(37, 53, 29, 0.9), (200, 310, 64, 0.7), (5, 1, 3, 0.0), (64, 64, 100, 0.99), (1, 40, 256, 0.5),
          (300, 1000, 260, 0.9), (129, 17, 4, 0.2), (33, 90, 1, 0.5), (0, 5, 7, 0.5), (6, 5, 0, 0.5)]


@pytest.mark.parametrize("rows,k,cols,rate", SHAPES)
def test_csr_and_coo_against_oracle(rows, k, cols, rate):
    from mamtorch_amd import capi

    a = _random_sparse(rows, k, rate, seed=rows + cols)
    b = torch.randn(k, cols, generator=torch.Generator().manual_seed(k))
    csr = a.to_sparse_csr()
    crow, col, val = csr.crow_indices(), csr.col_indices(), csr.values()
    want, floor = oracle.csr_spmm(crow.numpy(), col.numpy(), val.numpy(), b.numpy())
    c = capi.csr_spmm(crow.to(DEV), col.to(DEV), val.to(DEV), b.to(DEV), rows)
    torch.cuda.synchronize()
    _check(c, want, floor, "csr")
    coo = a.to_sparse_coo().coalesce()
    idx = coo.indices()
    c2 = capi.coo_spmm(idx[0].contiguous().to(DEV), idx[1].contiguous().to(DEV), coo.values().to(DEV), b.to(DEV), rows)
    torch.cuda.synchronize()
    _check(c2, want, floor, "coo")


def test_coo_unsorted_with_duplicates_and_strided_b():
    from mamtorch_amd import capi

    rows, k, cols = 70, 90, 48
    g = torch.Generator().manual_seed(3)
    nnz = 2000
    row = torch.randint(0, rows, (nnz,), generator=g)
    col = torch.randint(0, k, (nnz,), generator=g)
    val = torch.randn(nnz, generator=g)
    wide = torch.randn(k, cols + 16, generator=g)
    b = wide[:, 8:8 + cols]                      # a view: row stride cols + 16, 32-byte offset
    want, floor = oracle.coo_spmm(row.numpy(), col.numpy(), val.numpy(), b.contiguous().numpy(), rows)
    bd = wide.to(DEV)[:, 8:8 + cols]
    c = capi.coo_spmm(row.to(DEV), col.to(DEV), val.to(DEV), bd, rows)
    torch.cuda.synchronize()
    _check(c, want, floor, "coo unsorted")
    # the same matrix through CSR with unsorted columns inside the rows
    order = torch.argsort(row, stable=True)
    crow = torch.zeros(rows + 1, dtype=torch.int64)
    crow[1:] = torch.cumsum(torch.bincount(row, minlength=rows), 0)
    c2 = capi.csr_spmm(crow.to(DEV), col[order].to(DEV), val[order].to(DEV), bd, rows)
    torch.cuda.synchronize()
    _check(c2, want, floor, "csr unsorted columns")


@pytest.mark.parametrize("layout", [torch.sparse_csr, torch.sparse_coo])
def test_operator_name_keys_and_reference_style_check(layout):
    """The reference's own check (test/test_sparse.py:21-44) with seeds: random sizes in [10, 1000], 90 %
    zeros, result against the dense product."""
    import mamtorch_amd as mt

    rng = np.random.default_rng(7)
    n, l, m = (int(v) for v in rng.integers(10, 1000, 3))
    a = _random_sparse(n, l, 0.9, seed=n).to(DEV)
    b = torch.randn(l, m, generator=torch.Generator().manual_seed(m)).to(DEV)
    asparse = a.to_sparse(layout=layout)
    res = torch.ops.mamtorch_kernel_sparsev1.cusparsemm(asparse, b)
    assert res.shape == (n, m) and res.dtype == torch.float32 and res.device == b.device
    res2 = mt.sparse.kernel.v1.cusparsemm(asparse, b)
    want = a.double() @ b.double()
    floor = a.abs().double() @ b.abs().double()
    for r in (res, res2):
        assert bool(((r.double() - want).abs() <= 1e-5 * want.abs() + 2.0 ** -22 * floor).all())
    with pytest.raises(RuntimeError):
        torch.ops.mamtorch_kernel_sparsev1.cusparsemm(asparse, b[:-1])


def test_full_size_against_dense_matmul():
    from mamtorch_amd import capi

    n = 4096
    a = _random_sparse(n, n, 0.9, seed=1).to(DEV)
    b = torch.randn(n, n, generator=torch.Generator().manual_seed(2)).to(DEV)
    csr = a.to_sparse_csr()
    c = capi.csr_spmm(csr.crow_indices(), csr.col_indices(), csr.values(), b, n)
    want = a.double() @ b.double()
    floor = a.abs().double() @ b.abs().double()
    assert bool(((c.double() - want).abs() <= 1e-5 * want.abs() + 2.0 ** -22 * floor).all())
    # linearity, a size-independent property: (2A) @ b == 2 (A @ b) bit for bit (scaling by 2 is exact)
    c2 = capi.csr_spmm(csr.crow_indices(), csr.col_indices(), csr.values() * 2, b, n)
    assert torch.equal(c2, c * 2)


@pytest.mark.parametrize("rows,k,rate", [(37, 53, 0.5), (200, 310, 0.7), (5, 1, 0.0), (64, 1000, 0.3), (0, 5, 0.5), (300, 7, 0.99)])
def test_sparse_operand_written_out_dense(rows, k, rate):
    """mam_csr_to_dense / mam_coo_to_dense: exact (every cell is one stored value, or the sum of a repeated
    coordinate's values)."""
    from mamtorch_amd import capi

    a = _random_sparse(rows, k, rate, seed=rows + k)
    csr = a.to_sparse_csr()
    d = capi.csr_to_dense(csr.crow_indices().to(DEV), csr.col_indices().to(DEV), csr.values().to(DEV), rows, k)
    assert torch.equal(d.cpu(), a + 0.0)           # a + 0.0: the cleared cells are +0
    coo = a.to_sparse_coo().coalesce()
    idx = coo.indices()
    # every coordinate twice, halved values, shuffled: repeated coordinates add up
    perm = torch.randperm(2 * idx.shape[1], generator=torch.Generator().manual_seed(1))
    row2, col2 = torch.cat([idx[0], idx[0]])[perm], torch.cat([idx[1], idx[1]])[perm]
    val2 = torch.cat([coo.values() * 0.5, coo.values() * 0.5])[perm]
    d2 = capi.coo_to_dense(row2.contiguous().to(DEV), col2.contiguous().to(DEV), val2.contiguous().to(DEV), rows, k)
    assert torch.equal(d2.cpu(), a + 0.0)


@pytest.mark.parametrize("layout", [torch.sparse_csr, torch.sparse_coo])
@pytest.mark.parametrize("n,l,m,rate", [(300, 500, 260, 0.6), (1024, 2048, 512, 0.7), (129, 64, 64, 0.0), (64, 100, 63, 0.5)])
def test_operator_at_high_density(layout, n, l, m, rate):
    """From one stored entry in eight on (and 64 columns of b) the operator writes the operand out dense and
    calls the library GEMM; (64, 100, 63) stays on the sparse kernels.  Same bar as everywhere: the fp64 product
    within rtol 1e-5 plus the rounding floor of an fp32 sum."""
    a = _random_sparse(n, l, rate, seed=n + m).to(DEV)
    b = torch.randn(l, m, generator=torch.Generator().manual_seed(m)).to(DEV)
    asparse = a.to_sparse(layout=layout)
    res = torch.ops.mamtorch_kernel_sparsev1.cusparsemm(asparse, b)
    assert res.shape == (n, m) and res.dtype == torch.float32
    want = a.double() @ b.double()
    floor = a.abs().double() @ b.abs().double()
    assert bool(((res.double() - want).abs() <= 1e-5 * want.abs() + 2.0 ** -22 * floor).all())


@pytest.mark.parametrize("layout", [torch.sparse_csr, torch.sparse_coo])
@pytest.mark.parametrize("above", [False, True])
def test_operator_either_side_of_the_density_threshold(layout, above):
    """The operator changes route at one stored entry in eight (CSR; one in sixteen for COO): sparse kernel below,
    dense copy + library GEMM from there on, and with it the order of summation: one entry below and exactly at
    the threshold, both against the fp64 defining sum within rtol 1e-5 plus the rounding floor of an fp32 sum."""
    R, K, C = 96, 256, 128
    nnz = R * K // (8 if layout == torch.sparse_csr else 16) + (0 if above else -1)
    g = torch.Generator().manual_seed(17 + int(above))
    where = torch.randperm(R * K, generator=g)[:nnz]
    a = torch.zeros(R * K)
    a[where] = torch.randn(nnz, generator=g)
    a = a.view(R, K).to(DEV)
    assert int((a != 0).sum()) == nnz
    b = torch.randn(K, C, generator=g).to(DEV)
    res = torch.ops.mamtorch_kernel_sparsev1.cusparsemm(a.to_sparse(layout=layout), b)
    want = a.double() @ b.double()
    floor = a.abs().double() @ b.abs().double()
    assert bool(((res.double() - want).abs() <= 1e-5 * want.abs() + 2.0 ** -22 * floor).all())


def test_to_dense_skips_coordinates_outside_the_matrix():
    """mam_csr_to_dense / mam_coo_to_dense write at the coordinates they are given: an entry outside the
    matrix (a malformed tensor) is dropped instead of written out of range."""
    R, K = 4, 8
    crow = torch.tensor([0, 2, 3, 3, 5], dtype=torch.int64, device=DEV)
    col = torch.tensor([1, 8, -1, 7, 1 << 40], dtype=torch.int64, device=DEV)
    val = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0], device=DEV)
    guard = torch.full((R + 2, K), 9.0, device=DEV)          # rows before and after the matrix must stay
    from mamtorch_amd import capi

    l = capi.lib()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert l.mam_csr_to_dense(P(crow), P(col), P(val), P(guard[1]), K, R, K, st) == 0
    torch.cuda.synchronize()
    want = torch.full((R + 2, K), 9.0)
    want[1:R + 1] = 0.0
    want[1, 1] = 1.0
    want[4, 7] = 4.0
    assert torch.equal(guard.cpu(), want)
    row = torch.tensor([0, 4, -1, 3, 2], dtype=torch.int64, device=DEV)
    col2 = torch.tensor([1, 0, 0, 7, 8], dtype=torch.int64, device=DEV)
    guard.fill_(9.0)
    assert l.mam_coo_to_dense(P(row), P(col2), P(val), 5, P(guard[1]), K, R, K, st) == 0
    torch.cuda.synchronize()
    want = torch.full((R + 2, K), 9.0)
    want[1:R + 1] = 0.0
    want[1, 1] = 1.0
    want[4, 7] = 4.0
    assert torch.equal(guard.cpu(), want)
