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
    c, amax, amin = capi.csr_fc_forward(xd, *parts, M, None if bias is None else bias.to(dev))
    torch.cuda.synchronize()
    assert_bits_equal(c.cpu().numpy(), want[0], what + " c")
    assert_index_equal(amax.cpu().numpy(), want[1], what + " argmax")
    assert_index_equal(amin.cpu().numpy(), want[2], what + " argmin")
    grad = torch.randn(N, M, generator=torch.Generator().manual_seed(1))
    xo, vo = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(), want[1], want[2])
    xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin)
    torch.cuda.synchronize()
    np.testing.assert_allclose(xg.cpu().numpy(), xo, rtol=1e-5, atol=1e-6, err_msg=what + " x_grad")
    np.testing.assert_allclose(vg.cpu().numpy(), vo, rtol=1e-5, atol=1e-6, err_msg=what + " val_grad")
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
    xg, vg = capi.csr_fc_backward(xd, *parts, grad.to(dev), amax, amin)
    xdg, wdg = capi.fc_backward(xd, dense.to(dev), grad.to(dev), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    # two fp32 summation orders of the same terms: each may be off by the rounding floor of the
    # sum of absolute terms (measured by a backward pass over absolute values)
    xabs, wabs = capi.fc_backward(xd.abs(), dense.to(dev).abs(), grad.to(dev).abs(), amax, amin, capi.W_MK)
    torch.cuda.synchronize()
    rws = torch.repeat_interleave(torch.arange(M), crow[1:] - crow[:-1]).to(dev)
    want_v, abs_v = wdg[rws, col.to(dev)], wabs[rws, col.to(dev)]
    assert bool(((xg - xdg).abs() <= 1e-5 * xdg.abs() + 2.0 ** -21 * xabs).all())
    assert bool(((vg - want_v).abs() <= 1e-5 * want_v.abs() + 2.0 ** -21 * abs_v).all())
