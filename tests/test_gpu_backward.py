"""GPU parity of the MAM backward through the C ABI.

Bar: |got - want| <= 1e-5 * |want| + 2^-22 * S, where `want` is the oracle's order-independent
(fp64-accumulated) sum and S is the sum of the absolute values of the fp32 terms that make up
that cell.  The second term is the rounding floor of ANY fp32 summation order (the reference's
atomicAdd order is itself unspecified): where a cell's terms cancel, a relative bound on the
result alone cannot be met by fp32 adds.  For cells with a single term the bar is plain rtol 1e-5."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import config1, random_case

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
RTOL = 1e-5
FLOOR = 2.0 ** -22
STATS = []     # (what, worst plain relative error, cells beyond plain rtol, cells) of every comparison made


def _check(x, w_mk, grad, amax, amin, what, layouts=(0, 1)):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    xo, wo = oracle.backward(x.numpy(), w_mk.numpy(), grad.numpy(), amax, amin, oracle.W_MK)
    xs, ws_ = oracle.backward(x.abs().numpy(), w_mk.abs().numpy(), grad.abs().numpy(), amax, amin, oracle.W_MK)

    def close(got, want, abs_sum, msg):
        err = np.abs(got.astype(np.float64) - want)
        tol = RTOL * np.abs(want) + FLOOR * abs_sum + 1e-30
        # reported, not asserted: how far plain rtol 1e-5 alone would carry
        nz = np.abs(want) > 0
        rel = err[nz] / np.abs(want[nz]) if nz.any() else np.zeros(1)
        beyond = int((err > RTOL * np.abs(want) + 1e-30).sum())
        STATS.append((msg, float(rel.max()), beyond, int(want.size)))
        print("[backward tolerance] %s: worst plain relative error %.3g; %d of %d cells (%.4f %%) beyond plain "
              "rtol 1e-5 and inside the summation floor" % (msg, rel.max(), beyond, want.size,
                                                            100.0 * beyond / want.size))
        bad = np.argwhere(err > tol)
        assert bad.size == 0, "%s: %d cells out of tolerance, first %s got %r want %r (sum|terms| %r)" % (
            msg, len(bad), bad[0].tolist(), got[tuple(bad[0])], want[tuple(bad[0])], abs_sum[tuple(bad[0])])

    xd, gd = x.to(dev), grad.to(dev)
    a1, a2 = torch.tensor(amax).to(dev), torch.tensor(amin).to(dev)
    for layout in layouts:
        wd = (w_mk if layout == capi.W_MK else w_mk.T).contiguous().to(dev)
        xg, wg = capi.fc_backward(xd, wd, gd, a1, a2, layout)
        # the same call with the selected weights handed over instead of gathered
        cols = torch.arange(w_mk.shape[0])[None, :]
        w_sel = torch.stack([w_mk[cols, torch.tensor(amax).long()], w_mk[cols, torch.tensor(amin).long()]]).to(dev)
        rows = torch.arange(x.shape[0])[:, None]
        x_sel = torch.stack([x[rows, torch.tensor(amax).long()], x[rows, torch.tensor(amin).long()]]).to(dev)
        xg2, _ = capi.fc_backward(xd, wd, gd, a1, a2, layout, want_w=False, w_sel=w_sel.contiguous())
        xg3, wg3 = capi.fc_backward(xd, wd, gd, a1, a2, layout, w_sel=w_sel.contiguous(), x_sel=x_sel.contiguous())
        _, wg4 = capi.fc_backward(xd, wd, gd, a1, a2, layout, want_x=False, x_sel=x_sel.contiguous())
        torch.cuda.synchronize()
        close(xg2.cpu().numpy(), xo, xs, "%s x_grad (w_sel) layout %d" % (what, layout))
        close(xg3.cpu().numpy(), xo, xs, "%s x_grad (w_sel, x_sel) layout %d" % (what, layout))
        for got, tag in ((wg3, "w_sel, x_sel"), (wg4, "x_sel")):
            got = got.cpu().numpy() if layout == capi.W_MK else got.cpu().numpy().T
            close(got, wo, ws_, "%s w_grad (%s) layout %d" % (what, tag, layout))
        wg = wg.cpu().numpy() if layout == capi.W_MK else wg.cpu().numpy().T
        close(xg.cpu().numpy(), xo, xs, "%s x_grad layout %d" % (what, layout))
        close(wg, wo, ws_, "%s w_grad layout %d" % (what, layout))
    return xo, wo


def test_known_answers():
    def conv(v):
        return [conv(e) for e in v] if isinstance(v, list) else float(v)
    for kat in json.load(open(os.path.join(GOLDEN, "kat.json"))):
        if "a" not in kat:
            continue
        a = torch.tensor(conv(kat["a"]), dtype=torch.float32)
        b = torch.tensor(conv(kat["b"]), dtype=torch.float32)
        g = torch.tensor(conv(kat["grad"]), dtype=torch.float32)
        xo, wo = _check(a, b.T.contiguous(), g, np.asarray(kat["argmax"], np.int32),
                        np.asarray(kat["argmin"], np.int32), kat["name"])
        np.testing.assert_array_equal(xo, np.asarray(kat["a_grad"], np.float32))
        np.testing.assert_array_equal(wo.T, np.asarray(kat["b_grad"], np.float32))


def test_golden_brute_fixtures():
    data = np.load(os.path.join(GOLDEN, "brute_small.npz"))
    for i in range(5):
        f = lambda n: data["case%d_%s" % (i, n)]
        xo, wo = _check(torch.tensor(f("x")), torch.tensor(f("b")).T.contiguous(), torch.tensor(f("grad")),
                        f("argmax"), f("argmin"), "fixture %d" % i)
        np.testing.assert_allclose(xo, f("x_grad"), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(wo.T, f("b_grad"), rtol=1e-6, atol=1e-7)


def test_config1():
    x, w, bias, grad = config1()
    _, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
    _check(x, w, grad, amax, amin, "config 1")


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (65, 33, 130), (200, 1001, 70), (17, 9, 300), (300, 257, 31)])
def test_ragged_shapes(shape):
    N, K, M = shape
    x, w, grad = random_case(N, K, M, seed=sum(shape))
    _, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
    _check(x, w, grad, amax, amin, "shape %s" % (shape,))


def test_concentrated_and_duplicate_selections():
    g = torch.Generator().manual_seed(5)
    N, K, M = 128, 64, 96
    x, w, grad = random_case(N, K, M, seed=5)
    # every output selects the same k for max and min: 2*M terms collide on one x_grad cell per row
    amax = np.full((N, M), 7, np.int32)
    _check(x, w, grad, amax, amax.copy(), "all on k=7")
    # random picks, unrelated to the true extremes (as in the reference's backward benchmark,
    # test/test.py:316-317)
    amax = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32).numpy()
    amin = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32).numpy()
    _check(x, w, grad, amax, amin, "random picks")


def test_k_larger_than_one_lds_histogram():
    N, K, M = 6, 70000, 40
    x, w, grad = random_case(N, K, M, seed=9)
    g = torch.Generator().manual_seed(9)
    amax = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32).numpy()
    amin = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32).numpy()
    amax[0, :] = K - 1
    amin[0, :] = 0
    _check(x, w, grad, amax, amin, "K=70000")


def test_either_output_can_be_skipped_and_strided_inputs():
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M, off, sub = 40, 64, 50, 3, 29
    x, w, grad = random_case(N, K, M, seed=3)
    xs, ws = x[:, off:off + sub].contiguous(), w[:, off:off + sub].contiguous()
    _, amax, amin = oracle.forward(xs.numpy(), ws.numpy(), oracle.W_MK)
    xo, wo = oracle.backward(xs.numpy(), ws.numpy(), grad.numpy(), amax, amin, oracle.W_MK)
    xd, wd = x.to(dev).narrow(1, off, sub), w.to(dev).narrow(1, off, sub)
    a1, a2 = torch.tensor(amax).to(dev), torch.tensor(amin).to(dev)
    xg, wg = capi.fc_backward(xd, wd, grad.to(dev), a1, a2, capi.W_MK)
    np.testing.assert_allclose(xg.cpu().numpy(), xo, rtol=RTOL, atol=1e-6)
    np.testing.assert_allclose(wg.cpu().numpy(), wo, rtol=RTOL, atol=1e-6)
    xg, none = capi.fc_backward(xd, wd, grad.to(dev), a1, a2, capi.W_MK, want_w=False)
    assert none is None
    np.testing.assert_allclose(xg.cpu().numpy(), xo, rtol=RTOL, atol=1e-6)
    none, wg = capi.fc_backward(xd, wd, grad.to(dev), a1, a2, capi.W_MK, want_x=False)
    assert none is None
    np.testing.assert_allclose(wg.cpu().numpy(), wo, rtol=RTOL, atol=1e-6)


def test_headline_config2_full_size():
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    N, K, M = 256, 4096, 4096
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / 64
    grad = torch.randn(N, M, generator=g)
    _, amax, amin = capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK)
    xo, wo = _check(x, w, grad, amax.cpu().numpy(), amin.cpu().numpy(), "config 2")
    # at most 2*N*M cells of the weight gradient are touched
    assert np.count_nonzero(wo) <= 2 * N * M
    # linearity in grad
    xd, wd = x.to(dev), w.to(dev)
    g2 = torch.randn(N, M, generator=g)
    xa, wa = capi.fc_backward(xd, wd, grad.to(dev), amax, amin, capi.W_MK)
    xb, wb = capi.fc_backward(xd, wd, g2.to(dev), amax, amin, capi.W_MK)
    xc, wc = capi.fc_backward(xd, wd, (grad + g2).to(dev), amax, amin, capi.W_MK)
    assert torch.allclose(xa + xb, xc, rtol=1e-4, atol=1e-5)
    assert torch.allclose(wa + wb, wc, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dims", [(768, 3072), (3072, 768)])
def test_vit_mlp_config3_shapes(dims):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    K, M = dims
    N = 12608
    g = torch.Generator().manual_seed(K)
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / K ** 0.5
    grad = torch.randn(N, M, generator=g)
    _, amax, amin = capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK)
    _check(x, w, grad, amax.cpu().numpy(), amin.cpu().numpy(), "config 3", layouts=(1,))


@pytest.mark.parametrize("shape", [(2100, 100, 36), (2048, 64, 4), (4099, 517, 132), (2500, 16, 20)])
def test_large_batch_shares_of_the_batch_add_up(shape):
    """From 2048 batch rows on, slabs of the (out, in) weight gradient may be wider than 4 neurons and the
    batch is split over several workgroups per slab that add their shares: ragged last slab, ragged
    last share, and selections piled up on a few k."""
    N, K, M = shape
    g = torch.Generator().manual_seed(N + K)
    x = torch.randn(N, K, generator=g)
    w = torch.randn(M, K, generator=g)
    grad = torch.randn(N, M, generator=g)
    amax = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32)
    amin = torch.randint(0, min(K, 3), (N, M), generator=g, dtype=torch.int32)
    _check(x, w, grad, amax.numpy(), amin.numpy(), "large batch %s" % (shape,))


@pytest.mark.parametrize("fork", ["0", "1"])
def test_x_grad_on_the_second_stream_or_not(fork):
    """With both gradients asked for, x_grad may run on a second stream of the library between two events
    (taken by itself for large problems and under graph capture); option MAM_OPT_BACKWARD_FORK forces
    either way.
    The caller's stream must see both results, call after call."""
    from mamtorch_amd import capi

    capi.set_option(capi.OPT_BACKWARD_FORK, int(fork))
    try:
        dev = torch.device("cuda:0")
        g = torch.Generator().manual_seed(5)
        N, K, M = 96, 200, 64
        x = torch.randn(N, K, generator=g)
        w = torch.randn(M, K, generator=g)
        for rep in range(3):
            grad = torch.randn(N, M, generator=g)
            amax = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32)
            amin = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32)
            _check(x, w, grad, amax.numpy(), amin.numpy(), "fork=%s call %d" % (fork, rep))
            # consumers on the caller's stream right after the call, no synchronisation in between
            xg, wg = capi.fc_backward(x.to(dev), w.to(dev), grad.to(dev), amax.to(dev), amin.to(dev), capi.W_MK)
            sums = (xg.double().sum() + wg.double().sum()).item()
            xo, wo = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), amax.numpy(), amin.numpy(), oracle.W_MK)
            assert abs(sums - (xo.astype(np.float64).sum() + wo.astype(np.float64).sum())) < 1e-2
    finally:
        capi.set_option(capi.OPT_BACKWARD_FORK, capi.BACKWARD_FORK_AUTO)


@pytest.mark.parametrize("shape", [(64, 784, 256), (96, 200, 64), (256, 1024, 512), (130, 4096, 72), (40, 36, 8)])
def test_both_gradients_in_one_launch_or_two(shape):
    """(M,K) weights, aligned operands, a batch below twice the CU count, K <= 4096: one launch can hold the
    workgroups of both gradient kernels (option MAM_OPT_BACKWARD_ONE_LAUNCH: by default for small calls, 2 =
    wherever the shape allows it, 0 = never).  Either way the
    results meet the oracle; x_grad from handed-over weights is the exact sum, so the two ways agree bit for bit."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = shape
    x, w, grad = random_case(N, K, M, seed=N + M)
    _, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
    got = {}
    try:
        for mode in (0, 2):
            capi.set_option(capi.OPT_BACKWARD_ONE_LAUNCH, mode)
            _check(x, w, grad, amax, amin, "one launch=%d shape %s" % (mode, shape), layouts=(capi.W_MK,))
            w_sel = torch.empty(2, N, M, device=dev)
            x_sel = torch.empty(2, N, M, device=dev)
            c, a1, a2 = capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK, w_sel=w_sel, x_sel=x_sel)
            got[mode] = capi.fc_backward(x.to(dev), w.to(dev), grad.to(dev), a1, a2, capi.W_MK, w_sel=w_sel, x_sel=x_sel)
            torch.cuda.synchronize()
    finally:
        capi.set_option(capi.OPT_BACKWARD_ONE_LAUNCH, 1)
    assert torch.equal(got[0][0].view(torch.int32), got[2][0].view(torch.int32)), "x_grad differs between the two ways"
    # w_grad: two orders of fp32 additions, each held to the oracle's bar by _check above


def _dynamic_range_grad(N, M, pattern, seed):
    """grad whose terms span far more binades than a 64-bit fixed-point window holds."""
    g = torch.Generator().manual_seed(seed)
    grad = torch.randn(N, M, generator=g)
    if pattern == "few tiny":            # a handful of terms 2^-70 below the rest: parked and added afterwards
        idx = torch.randint(0, M, (N, 3), generator=g)
        grad.scatter_(1, idx, torch.full((N, 3), 2.0 ** -70))
    elif pattern == "few huge":          # a few terms 2^40 above the first ones
        idx = torch.randint(M // 2, M, (N, 2), generator=g)
        grad.scatter_(1, idx, torch.full((N, 2), 2.0 ** 40))
    elif pattern == "head huge":         # the first neurons decide the window, everything after them is below it
        grad[:, 4:] *= 2.0 ** -60
    elif pattern == "head tiny":         # ... or far above it
        grad[:, :M // 2] *= 2.0 ** -60
    elif pattern == "every binade":      # exponents spread over 100 binades
        grad *= torch.exp2(torch.randint(-60, 40, (N, M), generator=g).float())
    elif pattern == "denormal":
        grad *= 2.0 ** -140
    return grad


@pytest.mark.parametrize("pattern", ["few tiny", "few huge", "head huge", "head tiny", "every binade", "denormal"])
@pytest.mark.parametrize("shape", [(40, 256, 4100), (2048, 128, 520)])
def test_x_grad_over_a_wide_dynamic_range(shape, pattern):
    """x_grad accumulates in 64-bit fixed point inside a window of exponents; terms outside the window take
    the fp32 path, and a window that fits almost nothing makes the workgroup start over with fp32 atomics.
    Every one of those routes has to meet the same bar, for the one-row-per-workgroup kernel (first shape)
    and the rows-per-workgroup kernel of large batches (second shape)."""
    N, K, M = shape
    x, w, _ = random_case(N, K, M, seed=N + M)
    grad = _dynamic_range_grad(N, M, pattern, seed=K)
    _, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
    _check(x, w, grad, amax, amin, "%s %s" % (pattern, shape,), layouts=(1,))


@pytest.mark.parametrize("shape", [(40, 256, 4100), (2048, 128, 520)])
def test_x_grad_with_non_finite_terms(shape):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = shape
    x, w, grad = random_case(N, K, M, seed=N)
    grad[1, 5], grad[2, 7], grad[3, 9] = float("inf"), float("nan"), float("-inf")
    c, amax, amin = capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK)
    a1, a2 = amax.cpu().numpy(), amin.cpu().numpy()
    cols = torch.arange(M)[None, :]
    w_sel = torch.stack([w[cols, amax.cpu().long()], w[cols, amin.cpu().long()]]).contiguous().to(dev)
    xg, _ = capi.fc_backward(x.to(dev), w.to(dev), grad.to(dev), amax, amin, capi.W_MK, want_w=False, w_sel=w_sel)
    torch.cuda.synchronize()
    xo, _ = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), a1, a2, oracle.W_MK)
    got = xg.cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(xo))
    assert np.array_equal(np.isinf(got), np.isinf(xo)) and np.array_equal(got[np.isinf(xo)], xo[np.isinf(xo)])
    fin = np.isfinite(xo)
    np.testing.assert_allclose(got[fin], xo[fin], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [(256, 512, 1024), (4096, 256, 512)])
def test_x_grad_is_reproducible_bit_for_bit(shape):
    """Inside the window the sum of a cell is exact, so neither the order in which lanes arrive nor the
    launch changes a bit of x_grad."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = shape
    x, w, grad = random_case(N, K, M, seed=3)
    xd, wd, gd = x.to(dev), w.to(dev), grad.to(dev)
    ws = torch.empty(2, N, M, device=dev)
    xs = torch.empty(2, N, M, device=dev)
    c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK, w_sel=ws, x_sel=xs)
    first, _ = capi.fc_backward(xd, wd, gd, amax, amin, capi.W_MK, want_w=False, w_sel=ws)
    for _ in range(3):
        again, _ = capi.fc_backward(xd, wd, gd, amax, amin, capi.W_MK, want_w=False, w_sel=ws)
        assert torch.equal(first, again)
    # and it is the correctly rounded exact sum: fp64 accumulation of the fp32 terms, rounded once
    xo, _ = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), amax.cpu().numpy(), amin.cpu().numpy(), oracle.W_MK)
    np.testing.assert_array_equal(first.cpu().numpy(), xo.astype(np.float32))
    # the same without the hand-over (weights gathered by index), in both weight layouts
    gathered, _ = capi.fc_backward(xd, wd, gd, amax, amin, capi.W_MK, want_w=False)
    assert torch.equal(first, gathered)
    gathered, _ = capi.fc_backward(xd, wd.T.contiguous(), gd, amax, amin, capi.W_KM, want_w=False)
    assert torch.equal(first, gathered)


# ---- strict gradient parity: option MAM_OPT_BACKWARD_EXACT ----

def _exact_gradients(x, w, grad, with_x_sel=True):
    """Forward with the hand-over, then the backward with w_grad in fixed-point cells: (x_grad, w_grad,
    oracle x_grad, oracle w_grad) as numpy arrays."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, M = x.shape[0], w.shape[0]
    xd, wd, gd = x.to(dev), w.to(dev), grad.to(dev)
    ws = torch.empty(2, N, M, device=dev)
    xs = torch.empty(2, N, M, device=dev)
    _, amax, amin = capi.fc_forward(xd, wd, capi.W_MK, w_sel=ws, x_sel=xs)
    capi.set_option(capi.OPT_BACKWARD_EXACT, 1)
    try:
        xg, wg = capi.fc_backward(xd, wd, gd, amax, amin, capi.W_MK, w_sel=ws, x_sel=xs if with_x_sel else None)
        torch.cuda.synchronize()
    finally:
        capi.set_option(capi.OPT_BACKWARD_EXACT, 0)
    xo, wo = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), amax.cpu().numpy(), amin.cpu().numpy(), oracle.W_MK)
    return xg.cpu().numpy(), wg.cpu().numpy(), xo, wo


@pytest.mark.parametrize("config", ["config 1", "config 2"])
@pytest.mark.parametrize("with_x_sel", [True, False])
def test_exact_option_gradients_equal_the_oracle_bit_for_bit(config, with_x_sel):
    """With MAM_OPT_BACKWARD_EXACT both gradients are exact sums of their fp32 terms rounded once: bit-equal
    to the oracle's fp64-accumulated values at the two configurations the CPU oracle runs whole, no
    tolerance, no summation floor."""
    if config == "config 1":
        x, w, _, grad = config1()
    else:
        g = torch.Generator().manual_seed(0)
        x = torch.randn(256, 4096, generator=g)
        w = (torch.rand(4096, 4096, generator=g) * 2 - 1) / 64
        grad = torch.randn(256, 4096, generator=g)
    xg, wg, xo, wo = _exact_gradients(x, w, grad, with_x_sel)
    assert np.array_equal(xg.view(np.int32), xo.view(np.int32)), config + ": x_grad is not the rounded exact sum"
    assert np.array_equal(wg.view(np.int32), wo.view(np.int32)), config + ": w_grad is not the rounded exact sum"


@pytest.mark.parametrize("dims", [(768, 3072), (3072, 768)])
def test_exact_option_meets_plain_rtol_at_config3(dims):
    """Config 3 (12608 rows) with MAM_OPT_BACKWARD_EXACT: plain rtol 1e-5 on every cell of both gradients,
    no floor term (cells whose terms cancel included)."""
    K, M = dims
    g = torch.Generator().manual_seed(K)
    x = torch.randn(12608, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / K ** 0.5
    grad = torch.randn(12608, M, generator=g)
    xg, wg, xo, wo = _exact_gradients(x, w, grad)
    for name, got, want in (("x_grad", xg, xo), ("w_grad", wg, wo)):
        err = np.abs(got.astype(np.float64) - want)
        assert (err <= RTOL * np.abs(want)).all(), "config 3 %s: worst %.3g relative" % (
            name, (err[want != 0] / np.abs(want[want != 0])).max())


def test_exact_option_on_ragged_and_small_shapes():
    """Shapes the fixed-point w_grad kernel serves (M and K multiples of 4) with a partial last k chunk, and
    shapes it does not serve, which fall through to the fp32 route: all within the documented bar."""
    from mamtorch_amd import capi

    capi.set_option(capi.OPT_BACKWARD_EXACT, 1)
    try:
        for shape in ((33, 2052, 8), (5, 4, 4), (300, 4100, 12), (17, 9, 300), (64, 784, 256)):
            x, w, grad = random_case(*shape, seed=sum(shape))
            _, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
            _check(x, w, grad, amax, amin, "exact option, shape %s" % (shape,))
    finally:
        capi.set_option(capi.OPT_BACKWARD_EXACT, 0)


# ---- backward and selection count in one call ----

@pytest.mark.parametrize("shape", [(256, 4096, 4096), (64, 784, 256), (300, 1028, 36), (33, 100, 18), (2100, 64, 8)])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_backward_count_equals_the_two_calls(shape, mode):
    """mam_fc_backward_count = mam_fc_backward followed by mam_selection_count: counts exactly equal, x_grad
    bit-equal (the same kernel), w_grad equal within the documented bar (the fused kernel adds in another
    order).  Shapes on and off the fused route, every count mode, counters that are not zero at the start."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = shape
    x, w, grad = random_case(N, K, M, seed=N + mode)
    xd, wd, gd = x.to(dev), w.to(dev), grad.to(dev)
    ws = torch.empty(2, N, M, device=dev)
    xs = torch.empty(2, N, M, device=dev)
    _, amax, amin = capi.fc_forward(xd, wd, capi.W_MK, w_sel=ws, x_sel=xs)
    start = torch.randint(0, 5, (M, K), dtype=torch.int32, generator=torch.Generator().manual_seed(1)).to(dev)
    mc1, nc1, mc2, nc2 = start.clone(), start.clone(), start.clone(), start.clone()
    xg1, wg1 = capi.fc_backward(xd, wd, gd, amax, amin, capi.W_MK, w_sel=ws, x_sel=xs)
    capi.selection_count(amax, amin, mc1, nc1, mode)
    xg2, wg2 = capi.fc_backward_count(xd, wd, gd, amax, amin, mc2, nc2, mode, capi.W_MK, w_sel=ws, x_sel=xs)
    torch.cuda.synchronize()
    assert torch.equal(mc1, mc2) and torch.equal(nc1, nc2)
    assert torch.equal(xg1, xg2)
    _, wabs = capi.fc_backward(xd.abs(), wd.abs(), gd.abs(), amax, amin, capi.W_MK, want_x=False)
    torch.cuda.synchronize()
    assert bool(((wg1 - wg2).abs() <= 2 * (RTOL * wg1.abs() + FLOOR * wabs)).all())
    # and the counts against the oracle
    before = start.cpu().numpy()
    if mode == 2:     # flags, max and min apart: +1 where at least one batch row picked the cell
        want_m, want_n = before.copy(), before.copy()
        cols = np.broadcast_to(np.arange(M), (N, M))
        want_m[cols, amax.cpu().numpy()] += 1
        want_n[cols, amin.cpu().numpy()] += 1
    else:
        want_m, want_n = oracle.selection_count(amax.cpu().numpy(), amin.cpu().numpy(), before, before, mode=mode)
    assert np.array_equal(mc2.cpu().numpy(), want_m) and np.array_equal(nc2.cpu().numpy(), want_n)
