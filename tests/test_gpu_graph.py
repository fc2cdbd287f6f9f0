"""The C ABI under HIP graph capture: forward (both tilings, with and without split K), backward with
the hand-over, selection count and the CSR path are recorded once and replayed on changing inputs; every
replay is checked against the oracle, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal, pruned_csr, random_case

pytestmark = pytest.mark.gpu
RTOL = 1e-5
FLOOR = 2.0 ** -22


def _close(got, want, abs_sum, what):
    err = np.abs(got.astype(np.float64) - want)
    bad = np.argwhere(err > RTOL * np.abs(want) + FLOOR * abs_sum + 1e-30)
    assert bad.size == 0, "%s: %d cells out of tolerance, first %s" % (what, len(bad), bad[0].tolist())


@pytest.mark.parametrize("shape,layout_mk", [((64, 784, 256), True), ((256, 4096, 512), True), ((70, 123, 45), False)])
def test_dense_step_replays(shape, layout_mk):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = shape
    layout = capi.W_MK if layout_mk else capi.W_KM
    cases = [random_case(N, K, M, seed=s) for s in range(3)]
    # static buffers of the recorded step
    xs = torch.empty(N, K, device=dev)
    ws = torch.empty((M, K) if layout_mk else (K, M), device=dev)
    gs = torch.empty(N, M, device=dev)
    w_sel = torch.empty(2, N, M, device=dev)
    x_sel = torch.empty(2, N, M, device=dev)
    max_count = torch.zeros(M, K, dtype=torch.int32, device=dev)
    min_count = torch.zeros(M, K, dtype=torch.int32, device=dev)

    def load(case):
        x, w, g = case
        xs.copy_(x)
        ws.copy_(w if layout_mk else w.T.contiguous())
        gs.copy_(g)

    def step():
        c, amax, amin = capi.fc_forward(xs, ws, layout, w_sel=w_sel, x_sel=x_sel)
        cv = capi.fc_forward_values(xs, ws, layout)
        xg, wg = capi.fc_backward(xs, ws, gs, amax, amin, layout, w_sel=w_sel, x_sel=x_sel)
        capi.selection_count(amax, amin, max_count, min_count, capi.COUNT_HITS)
        return c, amax, amin, cv, xg, wg

    load(cases[0])
    step()                       # first call outside the capture: one-time kernel attributes are set here
    torch.cuda.synchronize()
    max_count.zero_()
    min_count.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    want_max = np.zeros((M, K), np.int64)
    want_min = np.zeros((M, K), np.int64)
    for r, case in enumerate(cases + cases[:1]):
        load(case)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c, amax, amin, cv, xg, wg = (t.cpu().numpy() for t in outs)
        x, w, g = case
        want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
        tag = "replay %d shape %s" % (r, shape)
        assert_bits_equal(c, want[0], tag + " c")
        assert_bits_equal(cv, want[0], tag + " values-only c")
        assert_index_equal(amax, want[1], tag + " argmax")
        assert_index_equal(amin, want[2], tag + " argmin")
        xo, wo = oracle.backward(x.numpy(), w.numpy(), g.numpy(), want[1], want[2], oracle.W_MK)
        xa, wa = oracle.backward(x.abs().numpy(), w.abs().numpy(), g.abs().numpy(), want[1], want[2], oracle.W_MK)
        _close(xg, xo, xa, tag + " x_grad")
        _close(wg if layout_mk else wg.T, wo, wa, tag + " w_grad")
        np.add.at(want_max, (np.arange(M)[None, :].repeat(N, 0), want[1]), 1)
        np.add.at(want_min, (np.arange(M)[None, :].repeat(N, 0), want[2]), 1)
        assert np.array_equal(max_count.cpu().numpy(), want_max), tag + " max_count"
        assert np.array_equal(min_count.cpu().numpy(), want_min), tag + " min_count"
        # eager work between replays, on the same buffers' device
        torch.randn(256, 256, device=dev).sum().item()


def test_sparse_step_replays():
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = 96, 300, 130
    dense, crow, col, val = pruned_csr(M, K, 0.1, seed=5)
    parts = [t.to(dev) for t in (crow, col, val)]
    xs = torch.empty(N, K, device=dev)
    gs = torch.empty(N, M, device=dev)
    w_sel = torch.empty(2, N, M, device=dev)
    pos_sel = torch.empty(2, N, M, dtype=torch.int32, device=dev)
    x_sel = torch.empty(2, N, M, device=dev)

    def step():
        c, amax, amin = capi.csr_fc_forward(xs, *parts, M, None, w_sel, pos_sel, x_sel)
        xg, vg = capi.csr_fc_backward(xs, *parts, gs, amax, amin, w_sel, pos_sel, x_sel)
        return c, amax, amin, xg, vg

    cases = [random_case(N, K, M, seed=20 + s) for s in range(3)]
    xs.copy_(cases[0][0])
    gs.copy_(cases[0][2])
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for r, (x, _, g) in enumerate(cases):
        xs.copy_(x)
        gs.copy_(g)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c, amax, amin, xg, vg = (t.cpu().numpy() for t in outs)
        want = oracle.forward(x.numpy(), dense.numpy(), oracle.W_MK)
        tag = "sparse replay %d" % r
        assert_bits_equal(c, want[0], tag + " c")
        assert_index_equal(amax, want[1], tag + " argmax")
        assert_index_equal(amin, want[2], tag + " argmin")
        xo, wo = oracle.backward(x.numpy(), dense.numpy(), g.numpy(), want[1], want[2], oracle.W_MK)
        xa, wa = oracle.backward(x.abs().numpy(), dense.abs().numpy(), g.abs().numpy(), want[1], want[2], oracle.W_MK)
        _close(xg, xo, xa, tag + " x_grad")
        mask = (dense != 0).numpy()
        _close(vg, wo[mask], wa[mask], tag + " val_grad")
        torch.randn(128, 128, device=dev).sum().item()


def test_backward_count_exact_option_and_select_replay():
    """The one-call backward + selection count (fused kernel), the backward with MAM_OPT_BACKWARD_EXACT and the
    radix select of a threshold, recorded once and replayed on changing inputs: counts exact, the exact option's
    gradients bit-equal to the fp64-accumulated oracle, the selected element equal to the sorted one."""
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = 128, 2048, 256
    cases = [random_case(N, K, M, seed=40 + s) for s in range(3)]
    xs = torch.empty(N, K, device=dev)
    ws = torch.empty(M, K, device=dev)
    gs = torch.empty(N, M, device=dev)
    w_sel = torch.empty(2, N, M, device=dev)
    x_sel = torch.empty(2, N, M, device=dev)
    max_count = torch.zeros(M, K, dtype=torch.int32, device=dev)
    min_count = torch.zeros(M, K, dtype=torch.int32, device=dev)
    rank = (M * K * 9) // 10

    def step():
        c, amax, amin = capi.fc_forward(xs, ws, capi.W_MK, w_sel=w_sel, x_sel=x_sel)
        xg, wg = capi.fc_backward_count(xs, ws, gs, amax, amin, max_count, min_count, capi.COUNT_HITS, capi.W_MK,
                                        w_sel=w_sel, x_sel=x_sel)
        capi.set_option(capi.OPT_BACKWARD_EXACT, 1)
        try:
            xe, we = capi.fc_backward(xs, ws, gs, amax, amin, capi.W_MK, w_sel=w_sel, x_sel=x_sel)
        finally:
            capi.set_option(capi.OPT_BACKWARD_EXACT, 0)
        found = capi.select_abs_ranks([(ws, capi.PRUNE_MAGNITUDE, None, None)], [rank])
        return amax, amin, xg, wg, xe, we, found

    def load(case):
        x, w, g = case
        xs.copy_(x)
        ws.copy_(w)
        gs.copy_(g)

    load(cases[0])
    step()
    torch.cuda.synchronize()
    max_count.zero_()
    min_count.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    want_max = np.zeros((M, K), np.int64)
    want_min = np.zeros((M, K), np.int64)
    for r, case in enumerate(cases + cases[:1]):
        load(case)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        amax, amin, xg, wg, xe, we, found = (t.cpu().numpy() for t in outs)
        x, w, g = case
        want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
        tag = "replay %d" % r
        assert_index_equal(amax, want[1], tag + " argmax")
        assert_index_equal(amin, want[2], tag + " argmin")
        xo, wo = oracle.backward(x.numpy(), w.numpy(), g.numpy(), want[1], want[2], oracle.W_MK)
        xa, wa = oracle.backward(x.abs().numpy(), w.abs().numpy(), g.abs().numpy(), want[1], want[2], oracle.W_MK)
        _close(xg, xo, xa, tag + " x_grad (one call with the count)")
        _close(wg, wo, wa, tag + " w_grad (one call with the count)")
        assert_bits_equal(xe, xo.astype(np.float32), tag + " x_grad (exact option)")
        assert_bits_equal(we, wo.astype(np.float32), tag + " w_grad (exact option)")
        np.add.at(want_max, (np.arange(M)[None, :].repeat(N, 0), want[1]), 1)
        np.add.at(want_min, (np.arange(M)[None, :].repeat(N, 0), want[2]), 1)
        assert np.array_equal(max_count.cpu().numpy(), want_max), tag + " max_count"
        assert np.array_equal(min_count.cpu().numpy(), want_min), tag + " min_count"
        assert found[0] == np.sort(np.abs(w.numpy()).ravel())[rank], tag + " selected element"
        torch.randn(256, 256, device=dev).sum().item()
