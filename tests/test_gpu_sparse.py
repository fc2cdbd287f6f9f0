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
    c, amax, amin = capi.csr_fc_forward(xd, *parts, M, None if bias is None else bias.to(dev), w_sel, pos_sel)
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
    grad = torch.randn(N, M, generator=torch.Generator().manual_seed(1))
    xo, vo = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(), want[1], want[2])
    # rtol 1e-5 plus the rounding floor of an fp32 sum in any order: 2^-22 x the sum of |terms| of the
    # cell, measured by the oracle's backward over absolute values
    xa, va = oracle.csr_backward(np.abs(x.numpy()), crow.numpy(), col.numpy(), np.abs(val.numpy()),
                                 np.abs(grad.numpy()), want[1], want[2])
    for handed in (False, True):
        xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin,
                                      w_sel if handed else None, pos_sel if handed else None)
        torch.cuda.synchronize()
        tag = what + (" (hand-over)" if handed else " (search)")
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
    c3, amax3, amin3 = capi.csr_fc_forward(xd, *parts, M, None, w_sel, pos_sel)
    assert torch.equal(c3.view(torch.int32), cd.view(torch.int32)) and torch.equal(amax3, dmax)
    xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin)
    xg2, vg2 = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin, w_sel, pos_sel)
    xdg, wdg = capi.fc_backward(xd, dense.to(dev), grad.to(dev), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    # two fp32 summation orders of the same terms: each may be off by the rounding floor of the
    # sum of absolute terms (measured by a backward pass over absolute values)
    xabs, wabs = capi.fc_backward(xd.abs(), dense.to(dev).abs(), grad.to(dev).abs(), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    rws = torch.repeat_interleave(torch.arange(M), crow[1:] - crow[:-1]).to(dev)
    want_v, abs_v = wdg[rws, col.to(dev)], wabs[rws, col.to(dev)]
    for got_x, got_v in ((xg, vg), (xg2, vg2)):
        assert bool(((got_x - xdg).abs() <= 1e-5 * xdg.abs() + 2.0 ** -21 * xabs).all())
        assert bool(((got_v - want_v).abs() <= 1e-5 * want_v.abs() + 2.0 ** -21 * abs_v).all())
