"""The module's `splits` as one call each way (mam_fc_forward_ranges / mam_fc_backward_ranges) through the C ABI:
every K range is a MAM neuron of its own, the output is the sum over the ranges in ascending order and then the
bias.  Oracle: the C oracle on each slice, added in fp32 in that order (the reference runs one operator per slice
and adds with `+=`, mamtorch/nn/v4/fullyconnected.py:163-176, bias at :197-198)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal, random_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _oracle_ranges(x, w_mk, bias, range_len):
    N, K = x.shape
    total = None
    amax, amin = [], []
    for k0 in range(0, K, range_len):
        k1 = min(K, k0 + range_len)
        c, i1, i2 = oracle.forward(np.ascontiguousarray(x[:, k0:k1]), np.ascontiguousarray(w_mk[:, k0:k1]), oracle.W_MK)
        total = c if total is None else (total + c).astype(np.float32)
        amax.append(i1 + k0)
        amin.append(i2 + k0)
    if bias is not None:
        total = (total + bias[None, :]).astype(np.float32)
    return total, np.stack(amax), np.stack(amin)


@pytest.mark.parametrize("N,K,M,range_len", [(256, 4096, 512, 1024), (96, 2048, 200, 512), (70, 123, 45, 41),
                                             (33, 100, 20, 34), (64, 784, 256, 262), (40, 300, 70, 300),
                                             (17, 64, 33, 16), (300, 1536, 640, 768), (64, 784, 256, 256),
                                             (50, 1072, 130, 512)])
def test_forward_and_backward_over_ranges(N, K, M, range_len):
    from mamtorch_amd import capi

    x, w, grad = random_case(N, K, M, seed=N + K)
    bias = torch.randn(M, generator=torch.Generator().manual_seed(1))
    want_c, want_max, want_min = _oracle_ranges(x.numpy(), w.numpy(), bias.numpy(), range_len)
    xd, gd, bd = x.to(DEV), grad.to(DEV), bias.to(DEV)
    # backward oracle: every range routes grad to its own two positions -> one backward per slice
    xg_want = np.zeros((N, K), np.float32)
    wg_want = np.zeros((M, K), np.float32)
    xg_floor, wg_floor = np.zeros((N, K)), np.zeros((M, K))
    for r, k0 in enumerate(range(0, K, range_len)):
        k1 = min(K, k0 + range_len)
        xs, ws = np.ascontiguousarray(x.numpy()[:, k0:k1]), np.ascontiguousarray(w.numpy()[:, k0:k1])
        a, b = oracle.backward(xs, ws, grad.numpy(), want_max[r] - k0, want_min[r] - k0, oracle.W_MK)
        xg_want[:, k0:k1], wg_want[:, k0:k1] = a, b
        a, b = oracle.backward(np.abs(xs), np.abs(ws), np.abs(grad.numpy()), want_max[r] - k0, want_min[r] - k0, oracle.W_MK)
        xg_floor[:, k0:k1], wg_floor[:, k0:k1] = a, b
    for layout in (capi.W_MK, capi.W_KM):
        wd = (w if layout == capi.W_MK else w.T).contiguous().to(DEV)
        tag = "N%d K%d M%d range %d layout %d" % (N, K, M, range_len, layout)
        c, amax, amin = capi.fc_forward_ranges(xd, wd, range_len, layout, bd)
        cv, _, _ = capi.fc_forward_ranges(xd, wd, range_len, layout, bd, with_indices=False)
        torch.cuda.synchronize()
        assert_bits_equal(c.cpu().numpy(), want_c, tag + " c")
        assert_bits_equal(cv.cpu().numpy(), want_c, tag + " values-only c")
        assert_index_equal(amax.cpu().numpy(), want_max, tag + " argmax")
        assert_index_equal(amin.cpu().numpy(), want_min, tag + " argmin")
        xg, wg = capi.fc_backward_ranges(xd, wd, gd, amax, amin, range_len, layout)
        torch.cuda.synchronize()
        wg = wg.cpu().numpy() if layout == capi.W_MK else wg.cpu().numpy().T
        for got, wanted, floor, name in ((xg.cpu().numpy(), xg_want, xg_floor, "x_grad"), (wg, wg_want, wg_floor, "w_grad")):
            err = np.abs(got.astype(np.float64) - wanted)
            assert (err <= 1e-5 * np.abs(wanted) + 2.0 ** -22 * floor + 1e-30).all(), tag + " " + name
        xg_only, none = capi.fc_backward_ranges(xd, wd, gd, amax, amin, range_len, layout, want_w=False)
        assert none is None and torch.equal(xg_only, xg)     # exact sums: no dependence on the order of arrival


def test_headline_shape_with_the_modules_splits():
    """Config 2 (batch 256, 4096 -> 4096) with splits = 4: the oracle on a sample of batch rows, and on all rows
    the property that the output is the sum over the ranges of (max + min) of the selected products."""
    from mamtorch_amd import capi

    N, K, M, range_len = 256, 4096, 4096, 1024
    g = torch.Generator().manual_seed(2)
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / 64.0
    grad = torch.randn(N, M, generator=g)
    xd, wd, gd = x.to(DEV), w.to(DEV), grad.to(DEV)
    c, amax, amin = capi.fc_forward_ranges(xd, wd, range_len, capi.W_MK, None)
    torch.cuda.synchronize()
    rows = torch.arange(0, N, 16)
    want_c, want_max, want_min = _oracle_ranges(x[rows].numpy(), w.numpy(), None, range_len)
    assert_bits_equal(c[rows.to(DEV)].cpu().numpy(), want_c, "headline splits c")
    assert_index_equal(amax[:, rows.to(DEV)].cpu().numpy(), want_max, "headline splits argmax")
    assert_index_equal(amin[:, rows.to(DEV)].cpu().numpy(), want_min, "headline splits argmin")
    # all rows: c = sum over ranges, in ascending order, of x[n, argmax] * w[m, argmax] + x[n, argmin] * w[m, argmin]
    total = None
    cols = torch.arange(M, device=DEV)[None, :]
    nrows = torch.arange(N, device=DEV)[:, None]
    for r in range(K // range_len):
        i1, i2 = amax[r].long(), amin[r].long()
        assert int(i1.min()) >= r * range_len and int(i1.max()) < (r + 1) * range_len
        part = xd[nrows, i1] * wd[cols, i1] + xd[nrows, i2] * wd[cols, i2]
        total = part if total is None else total + part
    assert torch.equal(total.view(torch.int32), c.view(torch.int32))
    # backward: each range routes grad to its own two positions; sums of the gradients match the closed form
    xg, wg = capi.fc_backward_ranges(xd, wd, gd, amax, amin, range_len, capi.W_MK)
    torch.cuda.synchronize()
    want_x = torch.zeros(N, K, dtype=torch.float64, device=DEV)
    want_w = torch.zeros(M, K, dtype=torch.float64, device=DEV)
    for r in range(K // range_len):
        for idx in (amax[r].long(), amin[r].long()):
            want_x.scatter_add_(1, idx, (gd * wd[cols, idx]).double())
            want_w.scatter_add_(1, idx.T.contiguous(), (gd * xd[nrows, idx]).double().T.contiguous())
    bad = (xg != want_x.float())
    assert not bool(bad.any()), "x_grad: %d cells differ from the exact sum rounded once, worst %g" % (
        int(bad.sum()), float((xg.double() - want_x).abs().max()))
    assert torch.allclose(wg.double(), want_w, rtol=1e-5, atol=1e-5)


def test_zero_extremes_inside_ranges_keep_their_sign():
    """All products of a range non-positive with zeros among them: the range's max is the FIRST zero product of
    that range, sign included, in the indexed and in the values-only form."""
    from mamtorch_amd import capi

    N, K, M, range_len = 8, 96, 16, 32
    g = torch.Generator().manual_seed(9)
    x = torch.rand(N, K, generator=g) + 0.5
    w = -torch.rand(M, K, generator=g) - 0.5
    x[0, 40] = 0.0          # -0.0 product in range 1
    x[1, 70] = -0.0         # +0.0 product in range 2
    x[2, 33] = 0.0
    x[2, 35] = -0.0         # first zero of range 1 is -0.0, a +0.0 follows
    want_c, want_max, want_min = _oracle_ranges(x.numpy(), w.numpy(), None, range_len)
    for layout in (capi.W_MK, capi.W_KM):
        wd = (w if layout == capi.W_MK else w.T).contiguous().to(DEV)
        c, amax, amin = capi.fc_forward_ranges(x.to(DEV), wd, range_len, layout)
        cv, _, _ = capi.fc_forward_ranges(x.to(DEV), wd, range_len, layout, with_indices=False)
        assert_bits_equal(c.cpu().numpy(), want_c, "zero extremes c")
        assert_bits_equal(cv.cpu().numpy(), want_c, "zero extremes values-only c")
        assert_index_equal(amax.cpu().numpy(), want_max, "zero extremes argmax")


def test_module_splits_run_as_one_operator_and_train():
    import mamtorch_amd as mt

    g = torch.Generator().manual_seed(4)
    N, K, M, splits = 50, 200, 24, 3
    x = torch.randn(N, K, generator=g)
    layer = mt.nn.FullyConnected(K, M, bias=True, splits=splits)
    w, b = layer.weight.detach().clone(), layer.bias.detach().clone()
    want_c, want_max, want_min = _oracle_ranges(x.numpy(), w.numpy(), b.numpy(), layer.in_subfeatures)
    layer = layer.to(DEV).train()
    xd = x.to(DEV).requires_grad_(True)
    y = layer(xd)
    assert_bits_equal(y.detach().cpu().numpy(), want_c, "module splits (training)")
    grad = torch.randn(N, M, generator=g)
    y.backward(grad.to(DEV))
    xg_want = np.zeros((N, K), np.float32)
    for r, k0 in enumerate(range(0, K, layer.in_subfeatures)):
        k1 = min(K, k0 + layer.in_subfeatures)
        a, _ = oracle.backward(np.ascontiguousarray(x.numpy()[:, k0:k1]), np.ascontiguousarray(w.numpy()[:, k0:k1]),
                               grad.numpy(), want_max[r] - k0, want_min[r] - k0, oracle.W_MK)
        xg_want[:, k0:k1] = a
    np.testing.assert_allclose(xd.grad.cpu().numpy(), xg_want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(layer.bias.grad.cpu().numpy(), grad.sum(0).numpy(), rtol=1e-5, atol=1e-5)
    assert layer.weight.grad is not None and layer.weight.grad.shape == (M, K)
    with torch.no_grad():
        assert_bits_equal(layer.eval()(x.to(DEV)).cpu().numpy(), want_c, "module splits (eval)")
    a = torch.randn(9, 40, generator=g).to(DEV).requires_grad_(True)
    wt = torch.randn(7, 40, generator=g).to(DEV).requires_grad_(True)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_ranges, (a, wt, None, 16, True),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
