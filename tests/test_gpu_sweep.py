"""Seeded sweep of random small shapes through the C ABI against the C oracle: dense forward on both tilings
and both weight layouts (values, indices, values-only, hand-over arrays), dense backward with and without the
hand-over, and the CSR path with its hand-over arrays.  The shapes are the ones the launch heuristics treat
case by case: few tiles (K split into 2 to 16 ranges, a last range of a single 16-k group), ragged K and M,
unaligned rows, batches on either side of the per-row / per-slab backward kernels.

Bars: forward values and indices bit-exact; gradients |got - want| <= 1e-5 |want| + floor * S, S = the sum of
the absolute values of the cell's terms (the rounding floor of any fp32 summation order; 2^-22 for N(0,1)
gradients, 2^-18 where the gradient spans many binades, which the fixed-point cells window)."""
import random

import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _close(got, want, abs_sum, what, floor):
    err = np.abs(got.astype(np.float64) - want)
    tol = RTOL * np.abs(want) + floor * abs_sum + 1e-30
    bad = np.argwhere((err > tol) & np.isfinite(want))
    assert bad.size == 0, "%s: %d cells out of tolerance, first %s got %r want %r (sum|terms| %r)" % (
        what, len(bad), bad[0].tolist(), got[tuple(bad[0])], want[tuple(bad[0])], abs_sum[tuple(bad[0])])


def _shape(rnd, kind):
    if kind == "small":
        return rnd.randint(1, 300), rnd.randint(1, 700), rnd.randint(1, 300)
    if kind == "k16":
        return rnd.randint(1, 300), 16 * rnd.randint(1, 70), 4 * rnd.randint(1, 80)
    if kind == "aligned":
        return rnd.randint(1, 300), 64 * rnd.randint(1, 40), 4 * rnd.randint(1, 80)
    if kind == "bigN":
        return rnd.randint(2048, 3000), rnd.randint(1, 200), 4 * rnd.randint(1, 40)
    if kind == "bigN_aligned":
        return rnd.randint(2048, 3000), 16 * rnd.randint(1, 24), 4 * rnd.randint(1, 48)
    return rnd.randint(1, 400), rnd.randint(1, 900), rnd.choice([rnd.randint(1, 300), 4 * rnd.randint(1, 80)])


def _inputs(rnd, seed, N, K, M):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, K, generator=g) * rnd.choice([1.0, 1e-3, 1e3])
    if rnd.random() < 0.3:
        x = torch.round(x * 2) / 2          # ties and zeros
    w = torch.randn(M, K, generator=g)
    if rnd.random() < 0.3:
        w = torch.round(w)
    grad = torch.randn(N, M, generator=g)
    gk = rnd.choice(["plain", "plain", "binades", "head", "few"])
    if gk == "binades":
        grad = grad * torch.exp2(torch.randint(-50, 30, (N, M), generator=g).float())
    elif gk == "head":
        grad[:, max(1, M // 8):] *= 2.0 ** -45
    elif gk == "few":
        grad[torch.rand(N, M, generator=g) < 0.002] *= 2.0 ** 35
    return g, x, w, grad, (2.0 ** -22 if gk == "plain" else 2.0 ** -18)


@pytest.mark.parametrize("seed", [3, 4])
def test_dense_sweep(seed):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    rnd = random.Random(seed)
    try:
        for it in range(28):
            kind = rnd.choice(["small", "k16", "aligned", "aligned", "bigN", "bigN_aligned"])
            N, K, M = _shape(rnd, kind)
            _, x, w, grad, floor = _inputs(rnd, seed * 100003 + it * 7919, N, K, M)
            xd, gd = x.to(dev), grad.to(dev)
            want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
            xo, wo = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), want[1], want[2], oracle.W_MK)
            xa, wa = oracle.backward(x.abs().numpy(), w.abs().numpy(), grad.abs().numpy(), want[1], want[2],
                                     oracle.W_MK)
            cols, rows = np.arange(M)[None, :], np.arange(N)[:, None]
            for layout, wl, tiling in ((capi.W_MK, w.contiguous(), capi.FORWARD_TILING_AUTO),
                                       (capi.W_MK, w.contiguous(), capi.FORWARD_TILING_WIDE),
                                       (capi.W_KM, w.T.contiguous(), capi.FORWARD_TILING_AUTO)):
                capi.set_option(capi.OPT_FORWARD_TILING, tiling)
                wd = wl.to(dev)
                wsel = torch.full((2, N, M), float("nan"), device=dev)
                xsel = torch.full((2, N, M), float("nan"), device=dev)
                c, amax, amin = capi.fc_forward(xd, wd, layout, w_sel=wsel, x_sel=xsel)
                cv = capi.fc_forward_values(xd, wd, layout)
                torch.cuda.synchronize()
                tag = "case %d %s %s layout %d tiling %d: %s" % (it, kind, (N, K, M), layout, tiling,
                                                                 capi.fc_forward_describe(xd, wd, layout, True))
                assert_bits_equal(c.cpu().numpy(), want[0], tag + " c")
                assert_bits_equal(cv.cpu().numpy(), want[0], tag + " values only")
                assert_index_equal(amax.cpu().numpy(), want[1], tag + " argmax")
                assert_index_equal(amin.cpu().numpy(), want[2], tag + " argmin")
                assert_bits_equal(wsel[0].cpu().numpy(), w.numpy()[cols, want[1]], tag + " w_sel of the max")
                assert_bits_equal(wsel[1].cpu().numpy(), w.numpy()[cols, want[2]], tag + " w_sel of the min")
                assert_bits_equal(xsel[0].cpu().numpy(), x.numpy()[rows, want[1]], tag + " x_sel of the max")
                assert_bits_equal(xsel[1].cpu().numpy(), x.numpy()[rows, want[2]], tag + " x_sel of the min")
                for sel in (False, True):
                    xg, wg = capi.fc_backward(xd, wd, gd, amax, amin, layout, w_sel=wsel if sel else None,
                                              x_sel=xsel if sel else None)
                    torch.cuda.synchronize()
                    wg = wg.cpu().numpy() if layout == capi.W_MK else wg.cpu().numpy().T
                    _close(xg.cpu().numpy(), xo, xa, tag + " x_grad hand-over %s" % sel, floor)
                    _close(wg, wo, wa, tag + " w_grad hand-over %s" % sel, max(floor, 2.0 ** -20))
    finally:
        capi.set_option(capi.OPT_FORWARD_TILING, capi.FORWARD_TILING_AUTO)


@pytest.mark.parametrize("seed", [5])
def test_sparse_sweep(seed):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    rnd = random.Random(seed)
    for it in range(24):
        N, K, M = _shape(rnd, "sparse")
        g, x, w, grad, floor = _inputs(rnd, seed * 100003 + it * 7919, N, K, M)
        dens = rnd.choice([0.0, 0.02, 0.1, 0.5, 1.0])
        csr = torch.where(torch.rand(M, K, generator=g) < dens, w, torch.zeros(())).to_sparse_csr()
        dense = csr.to_dense()       # what the CSR tensor holds (to_sparse_csr drops the zeros of w, signed or not)
        crow, col, val = csr.crow_indices(), csr.col_indices(), csr.values()
        want = oracle.forward(x.numpy(), dense.numpy(), oracle.W_MK)
        parts = [t.to(dev) for t in (crow, col, val)]
        xd, gd = x.to(dev), grad.to(dev)
        wsel = torch.full((2, N, M), 7.0, device=dev)
        psel = torch.full((2, N, M), -7, dtype=torch.int32, device=dev)
        xsel = torch.full((2, N, M), 7.0, device=dev)
        c, amax, amin = capi.csr_fc_forward(xd, *parts, M, None, wsel, psel, xsel)
        torch.cuda.synchronize()
        tag = "case %d sparse %s density %.2f" % (it, (N, K, M), dens)
        assert_bits_equal(c.cpu().numpy(), want[0], tag + " c")
        assert_index_equal(amax.cpu().numpy(), want[1], tag + " argmax")
        assert_index_equal(amin.cpu().numpy(), want[2], tag + " argmin")
        xo, vo = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(), want[1], want[2])
        xa, va = oracle.csr_backward(np.abs(x.numpy()), crow.numpy(), col.numpy(), np.abs(val.numpy()),
                                     np.abs(grad.numpy()), want[1], want[2])
        for mode in (0, 1, 2):      # no hand-over; weights and positions; weights, positions and inputs
            xg, vg = capi.csr_fc_backward(xd, *parts, gd, amax, amin, wsel if mode else None,
                                          psel if mode else None, xsel if mode == 2 else None)
            torch.cuda.synchronize()
            _close(xg.cpu().numpy(), xo, xa, tag + " x_grad mode %d" % mode, floor)
            _close(vg.cpu().numpy(), vo, va, tag + " val_grad mode %d" % mode, floor)
