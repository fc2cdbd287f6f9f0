"""GPU parity of the CSR-sparse MAM forward / backward through the C ABI.  The forward must equal
the dense MAM forward on the densified weight, bit for bit, including rows with no stored entry
and rows whose stored products are all negative (an implicit zero wins)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal, pruned_csr

pytestmark = pytest.mark.gpu


def _forward_backward(x, dense, crow, col, val, what, bias=None):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K = x.shape
    M = dense.shape[0]
    want = oracle.forward(x.numpy(), dense.numpy(), oracle.W_MK, None if bias is None else bias.numpy())
    xd = x.to(dev)
    parts = [t.to(dev) for t in (crow, col, val)]
    w_sel = torch.full((2, N, M), 7.0, dtype=torch.float32, device=dev)
    pos_sel = torch.full((2, N, M), -7, dtype=torch.int32, device=dev)
    x_sel = torch.full((2, N, M), 7.0, dtype=torch.float32, device=dev)
    c, amax, amin = capi.csr_fc_forward(xd, *parts, M, None if bias is None else bias.to(dev), w_sel, pos_sel, x_sel)
    c2, amax2, amin2 = capi.csr_fc_forward(xd, *parts, M, None if bias is None else bias.to(dev))
    torch.cuda.synchronize()
    assert_bits_equal(c.cpu().numpy(), want[0], what + " c")
    assert_index_equal(amax.cpu().numpy(), want[1], what + " argmax")
    assert_index_equal(amin.cpu().numpy(), want[2], what + " argmin")
    assert torch.equal(c.view(torch.int32), c2.view(torch.int32)) and torch.equal(amax, amax2) and torch.equal(amin, amin2)
    # hand-over arrays: position of the selected entry in col/val (-1: an implicit zero) and its value
    pos = pos_sel.cpu().numpy().astype(np.int64)
    sel = np.stack([want[1], want[2]]).astype(np.int64)
    rows_of = np.broadcast_to(np.arange(M), (2, N, M))
    stored = pos >= 0
    assert (pos[stored] >= crow.numpy()[rows_of[stored]]).all() and (pos[stored] < crow.numpy()[rows_of[stored] + 1]).all()
    assert (col.numpy()[pos[stored]] == sel[stored]).all(), what + " pos_sel points at another column"
    assert (dense.numpy()[rows_of[~stored], sel[~stored]] == 0).all()
    is_stored = np.zeros((M, K), dtype=bool)
    is_stored[np.repeat(np.arange(M), np.diff(crow.numpy())), col.numpy()] = True
    assert (is_stored[rows_of, sel] == stored).all(), what + " pos_sel misses a stored column"
    ws = w_sel.cpu().numpy()
    assert_bits_equal(ws[stored], val.numpy()[pos[stored]], what + " w_sel")
    assert (ws[~stored] == 0).all()
    # ... and the selected inputs x[n, selected column] (0 where an implicit zero was selected)
    xs = x_sel.cpu().numpy()
    n_of = np.broadcast_to(np.arange(N)[None, :, None], (2, N, M))
    assert_bits_equal(xs[stored], x.numpy()[n_of[stored], sel[stored]], what + " x_sel")
    assert (xs[~stored] == 0).all()
    grad = torch.randn(N, M, generator=torch.Generator().manual_seed(1))
    xo, vo = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(), want[1], want[2])
    # rtol 1e-5 plus the rounding floor of an fp32 sum in any order: 2^-22 x the sum of |terms| of the
    # cell, measured by the oracle's backward over absolute values
    xa, va = oracle.csr_backward(np.abs(x.numpy()), crow.numpy(), col.numpy(), np.abs(val.numpy()),
                                 np.abs(grad.numpy()), want[1], want[2])
    for handed in (0, 1, 2):
        xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin,
                                      w_sel if handed else None, pos_sel if handed else None,
                                      x_sel if handed == 2 else None)
        torch.cuda.synchronize()
        tag = what + (" (search)", " (hand-over)", " (hand-over with inputs)")[handed]
        for got, wanted, floor, name in ((xg, xo, xa, "x_grad"), (vg, vo, va, "val_grad")):
            err = np.abs(got.cpu().numpy().astype(np.float64) - wanted)
            bound = 1e-5 * np.abs(wanted) + 2.0 ** -22 * floor + 1e-30
            assert (err <= bound).all(), "%s %s: worst excess %g" % (tag, name, (err - bound).max())
    # stored positions agree with the dense backward; pruned positions get nothing
    xdense, wdense = oracle.backward(x.numpy(), dense.numpy(), grad.numpy(), want[1], want[2], oracle.W_MK)
    np.testing.assert_allclose(xo, xdense, rtol=1e-6, atol=1e-7)
    rows = np.repeat(np.arange(M), np.diff(crow.numpy()))
    np.testing.assert_allclose(vo, wdense[rows, col.numpy()], rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("density", [0.0, 0.01, 0.03, 0.1, 0.5, 1.0])
def test_densities(density):
    M, K, N = 300, 1000, 37
    dense, crow, col, val = pruned_csr(M, K, density, seed=int(density * 100))
    x = torch.randn(N, K, generator=torch.Generator().manual_seed(2))
    _forward_backward(x, dense, crow, col, val, "density %g" % density)


@pytest.mark.parametrize("N,M,K", [(301, 130, 257), (64, 7, 33), (65, 9, 4), (1, 5, 300), (517, 66, 100)])
def test_batch_tiles_and_ragged_shapes(N, M, K):
    # more than one batch tile, batch sizes that are no multiple of 4, neuron counts that are no
    # multiple of the 4 rows of a workgroup, unaligned row lengths
    dense, crow, col, val = pruned_csr(M, K, 0.2, seed=N + M)
    x = torch.randn(N, K, generator=torch.Generator().manual_seed(N))
    _forward_backward(x, dense, crow, col, val, "N%d M%d K%d" % (N, M, K))


def test_implicit_zero_rules():
    g = torch.Generator().manual_seed(3)
    M, K, N = 64, 96, 20
    dense, crow, col, val = pruned_csr(M, K, 0.25, seed=3, scale=1.0)
    val = val.clone()
    # row 0: all stored weights negative, row 1: all positive, row 2: stored explicit zeros
    val[crow[0]:crow[1]] = -val[crow[0]:crow[1]].abs()
    val[crow[1]:crow[2]] = val[crow[1]:crow[2]].abs()
    val[crow[2]:crow[3]] = 0.0
    dense = torch.zeros(M, K)
    for m in range(M):
        dense[m, col[crow[m]:crow[m + 1]]] = val[crow[m]:crow[m + 1]]
    x = torch.randn(N, K, generator=g)
    x[0] = x[0].abs()           # positive inputs: in row 0 every stored product is negative
    x[1] = -x[1].abs()
    x[2] = 0.0                  # all products are +-0
    x[3, :8] = 0.0
    _forward_backward(x, dense, crow, col, val, "implicit zero rules",
                      bias=torch.randn(M, generator=g))


@pytest.mark.parametrize("K", [7, 8, 19])
def test_signed_zeros_and_ties_inside_stored_pairs(K):
    """Fully stored rows (no implicit zero to fall back on), so every extreme is a stored entry.  The kernel
    records the pair of consecutive entries in which an extreme last improved and settles afterwards which
    of the two it was: zero extremes whose first occurrence is the SECOND entry of a pair (the value must
    carry that product's sign), ties within a pair and across pairs (lowest column wins), odd row lengths
    (the last entry is paired with itself)."""
    M, N = 6, 12
    g = torch.Generator().manual_seed(K)
    crow = torch.arange(0, (M + 1) * K, K, dtype=torch.int64)
    col = torch.arange(K, dtype=torch.int64).repeat(M)
    w = -torch.rand(M, K, generator=g) - 0.5            # all weights negative
    x = torch.rand(N, K, generator=g) + 0.5              # all inputs positive: every product negative ...
    x[0, 1] = 0.0                                        # ... except zeros: -0.0 at the second entry of pair 0
    x[1, 1] = 0.0
    x[1, 4] = -0.0                                       # a +0.0 product later: the max stays the first zero
    x[2, 3] = 0.0                                        # second entry of pair 1
    x[3, 2] = 0.0                                        # first entry of pair 1
    x[4, K - 1] = 0.0                                    # the last entry (paired with itself when K is odd)
    x[5, 0] = -0.0                                       # +0.0 at the very first entry
    x[5, 1] = 0.0
    x[6] = -x[6]                                         # all products positive: the min side gets the zeros
    x[6, 1] = 0.0
    x[7] = -x[7]
    x[7, K - 1] = -0.0
    w[1] = w[0]                                          # equal rows of w: ties between neurons are no issue
    x[8] = 1.0
    w[2, :] = -1.0                                       # every product equal: both extremes at column 0
    x[9] = 1.0
    w[3, :] = -2.0
    w[3, 1] = -1.0                                       # max at the second entry of pair 0, min tied at 0
    x[10] = 1.0
    w[4, :] = -1.0
    w[4, 5] = -3.0                                       # min at the second entry of pair 2
    w[4, 2] = -0.5                                       # max at the first entry of pair 1
    val = w.reshape(-1).clone()
    _forward_backward(x, w.clone(), crow, col, val, "signed zeros and ties in pairs, K=%d" % K)


def test_first_columns_stored_and_last_missing():
    # the lowest missing column is K-1 / is 0 / lies between stored runs
    K, N = 40, 6
    rows = [list(range(K - 1)), list(range(1, K)), [0, 1, 2, 5, 6], [], list(range(K))]
    M = len(rows)
    crow = torch.tensor([0] + list(np.cumsum([len(r) for r in rows])), dtype=torch.int64)
    col = torch.tensor([c for r in rows for c in r], dtype=torch.int64)
    g = torch.Generator().manual_seed(4)
    val = -torch.rand(col.numel(), generator=g) - 0.1
    dense = torch.zeros(M, K)
    for m in range(M):
        dense[m, col[crow[m]:crow[m + 1]]] = val[crow[m]:crow[m + 1]]
    x = torch.rand(N, K, generator=g) + 0.1
    x[1] = -x[1]
    _forward_backward(x, dense, crow, col, val, "missing column position")


@pytest.mark.parametrize("density", [0.1, 0.03, 0.01])
def test_config5_full_size_equals_dense_kernel(density):
    """W 4096x4096 pruned per row, N256: against the GPU dense forward on the densified weight
    (itself checked against the oracle), and against the C oracle on sampled batch rows."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    M = K = 4096
    N = 256
    dense, crow, col, val = pruned_csr(M, K, density, seed=11)
    assert col.numel() == int(round(density * K)) * M
    x = torch.randn(N, K, generator=torch.Generator().manual_seed(5))
    xd = x.to(dev)
    parts = [t.to(dev) for t in (crow, col, val)]
    c, amax, amin = capi.csr_fc_forward(xd, *parts, M)
    cd, dmax, dmin = capi.fc_forward(xd, dense.to(dev), capi.W_MK)
    torch.cuda.synchronize()
    assert torch.equal(c.view(torch.int32), cd.view(torch.int32))
    assert torch.equal(amax, dmax) and torch.equal(amin, dmin)
    rows = torch.arange(0, N, 16)
    want = oracle.csr_forward(x[rows].numpy(), crow.numpy(), col.numpy(), val.numpy(), K)
    assert_bits_equal(c[rows.to(dev)].cpu().numpy(), want[0], "config 5 c")
    assert_index_equal(amax[rows.to(dev)].cpu().numpy(), want[1], "config 5 argmax")
    grad = torch.randn(N, M, generator=torch.Generator().manual_seed(6))
    w_sel = torch.empty((2, N, M), dtype=torch.float32, device=dev)
    pos_sel = torch.empty((2, N, M), dtype=torch.int32, device=dev)
    x_sel = torch.empty((2, N, M), dtype=torch.float32, device=dev)
    c3, amax3, amin3 = capi.csr_fc_forward(xd, *parts, M, None, w_sel, pos_sel, x_sel)
    assert torch.equal(c3.view(torch.int32), cd.view(torch.int32)) and torch.equal(amax3, dmax)
    xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin)
    xg2, vg2 = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin, w_sel, pos_sel)
    xg3, vg3 = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin, w_sel, pos_sel, x_sel)
    xdg, wdg = capi.fc_backward(xd, dense.to(dev), grad.to(dev), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    # two fp32 summation orders of the same terms: each may be off by the rounding floor of the
    # sum of absolute terms (measured by a backward pass over absolute values)
    xabs, wabs = capi.fc_backward(xd.abs(), dense.to(dev).abs(), grad.to(dev).abs(), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    rws = torch.repeat_interleave(torch.arange(M), crow[1:] - crow[:-1]).to(dev)
    want_v, abs_v = wdg[rws, col.to(dev)], wabs[rws, col.to(dev)]
    for got_x, got_v in ((xg, vg), (xg2, vg2), (xg3, vg3)):
        assert bool(((got_x - xdg).abs() <= 1e-5 * xdg.abs() + 2.0 ** -21 * xabs).all())
        assert bool(((got_v - want_v).abs() <= 1e-5 * want_v.abs() + 2.0 ** -21 * abs_v).all())
    # and against the C oracle's CSR backward (fp64 accumulation) over the whole batch, every route
    amax_c, amin_c = amax.cpu().numpy(), amin.cpu().numpy()
    want_xg, want_vg = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(),
                                           amax_c, amin_c)
    floor_xg, floor_vg = oracle.csr_backward(x.abs().numpy(), crow.numpy(), col.numpy(), val.abs().numpy(),
                                             grad.abs().numpy(), amax_c, amin_c)
    for route, (got_x, got_v) in (("gather", (xg, vg)), ("w_sel", (xg2, vg2)), ("w_sel + x_sel", (xg3, vg3))):
        for name, got, want, floor in (("x_grad", got_x, want_xg, floor_xg), ("val_grad", got_v, want_vg, floor_vg)):
            err = np.abs(got.cpu().numpy().astype(np.float64) - want)
            bound = 1e-5 * np.abs(want) + 2.0 ** -22 * floor
            assert (err <= bound).all(), "config 5 %s (%s): worst %.3g over the bound" % (name, route, (err - bound).max())


def test_nan_in_stored_values_is_ignored():
    """A NaN product never wins and never sticks (the dense rule, ordered compares): NaN in a row's first
    stored value, in mid-row, and a row whose stored values are all NaN (an implicit zero is then both
    extremes).  x stays finite: the implicit-zero candidate is read at the lowest missing column only."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    M, K, N = 48, 200, 70
    dense, crow, col, val = pruned_csr(M, K, 0.2, seed=9, scale=1.0)
    val = val.clone()
    val[crow[0]] = float("nan")
    val[(crow[1] + crow[2]) // 2] = float("nan")
    val[crow[2]:crow[3]] = float("nan")
    val[crow[5] + 1] = float("nan")
    val[crow[5] + 2] = float("nan")
    x = torch.randn(N, K, generator=torch.Generator().manual_seed(10))
    want = oracle.csr_forward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), K)
    for n_rows in (N, 33):            # both batch-tile shapes of the kernel
        c, amax, amin = capi.csr_fc_forward(x[:n_rows].to(dev), crow.to(dev), col.to(dev), val.to(dev), M)
        torch.cuda.synchronize()
        assert_bits_equal(c.cpu().numpy(), want[0][:n_rows], "nan values c")
        assert_index_equal(amax.cpu().numpy(), want[1][:n_rows], "nan values argmax")
        assert_index_equal(amin.cpu().numpy(), want[2][:n_rows], "nan values argmin")


def test_validate_csr_names_what_is_malformed():
    """The operators trust the index arrays; sparse.validate_csr is the explicit check."""
    import mamtorch_amd as mt

    dev = torch.device("cuda:0")
    dense, crow, col, val = pruned_csr(37, 50, 0.2, seed=3)
    good = torch.sparse_csr_tensor(crow.to(dev), col.to(dev), val.to(dev), size=(37, 50))
    mt.sparse.validate_csr(good)
    mt.sparse.validate_csr(dense.to(dev).to_sparse_csr())
    mt.sparse.validate_csr(torch.zeros(5, 7, device=dev).to_sparse_csr())
    col_bad = col.clone()
    col_bad[3] = 50
    with pytest.raises(ValueError, match="out of range"):
        mt.sparse.validate_csr(torch.sparse_csr_tensor(crow.to(dev), col_bad.to(dev), val.to(dev), size=(37, 50)))
    col_swapped = col.clone()
    col_swapped[[0, 1]] = col[[1, 0]]
    with pytest.raises(ValueError, match="ascending"):
        mt.sparse.validate_csr(torch.sparse_csr_tensor(crow.to(dev), col_swapped.to(dev), val.to(dev), size=(37, 50)))
    crow_bad = crow.clone()
    crow_bad[5], crow_bad[6] = crow[6], crow[5]
    with pytest.raises(ValueError, match="decrease"):
        mt.sparse.validate_csr(torch.sparse_csr_tensor(crow_bad.to(dev), col.to(dev), val.to(dev), size=(37, 50)))
    crow_short = crow.clone()
    crow_short[-1] -= 1
    with pytest.raises(ValueError, match="0 to nnz"):
        mt.sparse.validate_csr(torch.sparse_csr_tensor(crow_short.to(dev), col.to(dev), val.to(dev), size=(37, 50)))
