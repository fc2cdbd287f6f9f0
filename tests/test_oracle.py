"""Pins the CPU oracle (oracle/mam_oracle.c, oracle/torch_port.py) without the reference:
hand-derived known answers, an independent pure-Python brute force, closed-form special cases,
autograd of a gather formulation and fp64 finite differences.  CPU only."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import brute, torch_port
from helpers import assert_bits_equal, assert_index_equal, config1, pruned_csr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _arr(v, dtype=np.float32):
    def conv(e):
        if isinstance(e, list):
            return [conv(i) for i in e]
        return float(e) if isinstance(e, str) else e
    return np.asarray(conv(v), dtype=dtype)


def _kats():
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("kat", [k for k in _kats() if "a" in k], ids=lambda k: k["name"])
def test_known_answers_forward_backward(kat):
    a, b, g = _arr(kat["a"]), _arr(kat["b"]), _arr(kat["grad"])
    for fwd in (lambda: oracle.forward(a, b),
                lambda: oracle.forward(a, np.ascontiguousarray(b.T), oracle.W_MK),
                lambda: brute.forward(a, b),
                lambda: tuple(t.numpy() for t in torch_port.forward(torch.tensor(a), torch.tensor(b)))):
        c, amax, amin = fwd()
        assert_bits_equal(c, _arr(kat["c"]), kat["name"] + " c")
        assert_index_equal(amax, _arr(kat["argmax"], np.int32), kat["name"] + " argmax")
        assert_index_equal(amin, _arr(kat["argmin"], np.int32), kat["name"] + " argmin")
    amax, amin = _arr(kat["argmax"], np.int32), _arr(kat["argmin"], np.int32)
    xg, bg = oracle.backward(a, b, g, amax, amin)
    np.testing.assert_array_equal(xg, _arr(kat["a_grad"]))
    np.testing.assert_array_equal(bg, _arr(kat["b_grad"]))
    xg, wg = oracle.backward(a, np.ascontiguousarray(b.T), g, amax, amin, oracle.W_MK)
    np.testing.assert_array_equal(xg, _arr(kat["a_grad"]))
    np.testing.assert_array_equal(wg, _arr(kat["b_grad"]).T)
    xt, bt = torch_port.backward(torch.tensor(a), torch.tensor(b), torch.tensor(g), torch.tensor(amax),
                                 torch.tensor(amin))
    np.testing.assert_array_equal(xt.numpy(), _arr(kat["a_grad"]))
    np.testing.assert_array_equal(bt.numpy(), _arr(kat["b_grad"]))


def test_known_answer_selection_count():
    kat = [k for k in _kats() if k["name"] == "selection_count"][0]
    amax, amin = _arr(kat["sel_argmax"], np.int32), _arr(kat["sel_argmin"], np.int32)
    zeros = np.zeros((kat["M"], kat["K"]), np.int32)
    for impl in (oracle, brute):
        mc, nc = impl.selection_count(amax, amin, zeros, zeros, mode=0)
        np.testing.assert_array_equal(mc, _arr(kat["ref_max_count"], np.int32))
        np.testing.assert_array_equal(nc, zeros)
        mc, nc = impl.selection_count(amax, amin, zeros, zeros, mode=1)
        np.testing.assert_array_equal(mc, _arr(kat["hits_max_count"], np.int32))
        np.testing.assert_array_equal(nc, _arr(kat["hits_min_count"], np.int32))
    # the literal advanced-index "+= 1" of the module (duplicates do not accumulate)
    lit = torch_port.selection_count_reference(torch.tensor(amax), torch.tensor(amin),
                                               torch.zeros((kat["M"], kat["K"]), dtype=torch.int32))
    np.testing.assert_array_equal(lit.numpy(), _arr(kat["ref_max_count"], np.int32))
    # three hits on one cell add 1, not 3
    z = torch.zeros(3, 4, dtype=torch.int32)
    z[torch.tensor([0, 0, 0, 1]), torch.tensor([2, 2, 2, 3])] += 1
    assert z.tolist() == [[0, 0, 1, 0], [0, 0, 0, 1], [0, 0, 0, 0]]


def test_golden_brute_fixtures():
    data = np.load(os.path.join(GOLDEN, "brute_small.npz"))
    n_cases = len({k.split("_")[0] for k in data.files})
    assert n_cases == 5
    for i in range(n_cases):
        f = lambda name: data["case%d_%s" % (i, name)]
        c, amax, amin = oracle.forward(f("x"), f("b"), oracle.W_KM, f("bias"))
        assert_bits_equal(c, f("c"), "case%d c" % i)
        assert_index_equal(amax, f("argmax"), "case%d argmax" % i)
        assert_index_equal(amin, f("argmin"), "case%d argmin" % i)
        ct, tmax, tmin = torch_port.forward(torch.tensor(f("x")), torch.tensor(f("b")), torch.tensor(f("bias")))
        assert_bits_equal(ct.numpy(), f("c"), "case%d torch c" % i)
        assert_index_equal(tmax.numpy(), f("argmax"), "case%d torch argmax" % i)
        assert_index_equal(tmin.numpy(), f("argmin"), "case%d torch argmin" % i)
        xg, bg = oracle.backward(f("x"), f("b"), f("grad"), f("argmax"), f("argmin"))
        np.testing.assert_allclose(xg, f("x_grad"), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(bg, f("b_grad"), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("seed", range(6))
def test_three_statements_agree_on_random_inputs(seed):
    rng = np.random.default_rng(seed)
    N, K, M = rng.integers(1, 7), rng.integers(1, 24), rng.integers(1, 9)
    x = rng.standard_normal((N, K)).astype(np.float32)
    b = rng.standard_normal((K, M)).astype(np.float32)
    if seed % 2:   # coarse values: many ties and zeros
        x, b = np.round(x), np.round(b)
    bias = rng.standard_normal(M).astype(np.float32)
    cb, b1, b2 = brute.forward(x, b, bias)
    for c, a1, a2 in (oracle.forward(x, b, oracle.W_KM, bias),
                      oracle.forward(x, np.ascontiguousarray(b.T), oracle.W_MK, bias),
                      tuple(t.numpy() for t in torch_port.forward(torch.tensor(x), torch.tensor(b), torch.tensor(bias)))):
        assert_bits_equal(c, cb, "c")
        assert_index_equal(a1, b1, "argmax")
        assert_index_equal(a2, b2, "argmin")
    g = rng.standard_normal((N, M)).astype(np.float32)
    xb, bb = brute.backward(x, b, g, b1, b2)
    xo, bo = oracle.backward(x, b, g, b1, b2)
    np.testing.assert_allclose(xo, xb, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(bo, bb, rtol=1e-6, atol=1e-7)
    zeros = np.zeros((M, K), np.int32)
    for mode in (0, 1):
        for got, want in zip(oracle.selection_count(b1, b2, zeros + 3, zeros + 1, mode),
                             brute.selection_count(b1, b2, zeros + 3, zeros + 1, mode)):
            np.testing.assert_array_equal(got, want)


def test_closed_forms():
    rng = np.random.default_rng(7)
    # K = 1: C = 2*a*b, both indices 0
    a = rng.standard_normal((5, 1)).astype(np.float32)
    b = rng.standard_normal((1, 4)).astype(np.float32)
    c, amax, amin = oracle.forward(a, b)
    assert_bits_equal(c, (a * b) + (a * b), "K=1")
    assert not amax.any() and not amin.any()
    # non-negative operands: max / min are the largest / smallest product
    a = np.abs(rng.standard_normal((4, 9))).astype(np.float32)
    b = np.abs(rng.standard_normal((9, 3))).astype(np.float32)
    c, amax, amin = oracle.forward(a, b)
    prod = a[:, :, None] * b[None, :, :]
    assert_bits_equal(c, prod.max(1) + prod.min(1), "non-negative")
    np.testing.assert_array_equal(amax, prod.argmax(1))
    np.testing.assert_array_equal(amin, prod.argmin(1))
    # one-hot columns of b with a > 0: the max sits at the hot row, the min at the first zero row
    K, M = 6, 6
    b = np.eye(K, M, dtype=np.float32)
    a = (np.abs(rng.standard_normal((3, K))) + 1).astype(np.float32)
    c, amax, amin = oracle.forward(a, b)
    np.testing.assert_array_equal(amax, np.tile(np.arange(M), (3, 1)))
    np.testing.assert_array_equal(amin, np.tile(np.array([1] + [0] * (M - 1)), (3, 1)))
    assert_bits_equal(c, a[:, :M], "one-hot")
    # scaling (a*s, b/s) by a power of two leaves everything unchanged
    a = rng.standard_normal((4, 11)).astype(np.float32)
    b = rng.standard_normal((11, 5)).astype(np.float32)
    r0 = oracle.forward(a, b)
    r1 = oracle.forward(a * np.float32(8), b / np.float32(8))
    assert_bits_equal(r1[0], r0[0], "scaling")
    np.testing.assert_array_equal(r1[1], r0[1])
    np.testing.assert_array_equal(r1[2], r0[2])
    # permuting k permutes the indices (no ties in continuous data)
    perm = rng.permutation(11)
    r2 = oracle.forward(a[:, perm], b[perm, :])
    assert_bits_equal(r2[0], r0[0], "permutation")
    np.testing.assert_array_equal(perm[r2[1]], r0[1])
    np.testing.assert_array_equal(perm[r2[2]], r0[2])


def test_backward_matches_autograd_of_gather_formulation():
    torch.manual_seed(3)
    N, K, M = 6, 13, 5
    a = torch.randn(N, K, dtype=torch.float64, requires_grad=True)
    b = torch.randn(K, M, dtype=torch.float64, requires_grad=True)
    g = torch.randn(N, M, dtype=torch.float64)
    prod = a[:, :, None] * b[None, :, :]
    y = prod.max(dim=1).values + prod.min(dim=1).values
    y.backward(g)
    a32, b32, g32 = a.detach().float().numpy(), b.detach().float().numpy(), g.float().numpy()
    _, amax, amin = oracle.forward(a32, b32)
    xg, bg = oracle.backward(a32, b32, g32, amax, amin)
    np.testing.assert_allclose(xg, a.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(bg, b.grad.numpy(), rtol=1e-5, atol=1e-6)
    # invariants: both gradients sum to sum g*(selected operand)
    sel_w = b32[amax, np.arange(M)[None, :]] + b32[amin, np.arange(M)[None, :]]
    np.testing.assert_allclose(xg.sum(), (g32 * sel_w).sum(), rtol=1e-5)
    sel_x = np.take_along_axis(a32, amax, 1) + np.take_along_axis(a32, amin, 1)
    np.testing.assert_allclose(bg.sum(), (g32 * sel_x).sum(), rtol=1e-5)


def test_backward_finite_differences_fp64():
    rng = np.random.default_rng(11)
    N, K, M = 3, 7, 4
    a = rng.standard_normal((N, K))
    b = rng.standard_normal((K, M))
    g = rng.standard_normal((N, M))

    def loss(a_, b_):
        p = a_[:, :, None] * b_[None, :, :]
        return ((p.max(1) + p.min(1)) * g).sum()

    _, amax, amin = oracle.forward(a.astype(np.float32), b.astype(np.float32))
    xg, bg = oracle.backward(a.astype(np.float32), b.astype(np.float32), g.astype(np.float32), amax, amin)
    eps = 1e-6
    for (i, j) in [(0, 0), (1, 3), (2, 6)]:
        d = np.zeros_like(a); d[i, j] = eps
        fd = (loss(a + d, b) - loss(a - d, b)) / (2 * eps)
        assert abs(fd - xg[i, j]) < 1e-4 * max(1.0, abs(fd))
    for (i, j) in [(0, 0), (4, 2), (6, 3)]:
        d = np.zeros_like(b); d[i, j] = eps
        fd = (loss(a, b + d) - loss(a, b - d)) / (2 * eps)
        assert abs(fd - bg[i, j]) < 1e-4 * max(1.0, abs(fd))


def test_config1_c_oracle_vs_torch_port():
    x, w, bias, grad = config1()
    c, amax, amin = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK, bias.numpy())
    ct, tmax, tmin = torch_port.forward(x, w.T.contiguous(), bias)
    assert_bits_equal(c, ct.numpy(), "config 1 c")
    assert_index_equal(amax, tmax.numpy(), "config 1 argmax")
    assert_index_equal(amin, tmin.numpy(), "config 1 argmin")
    xg, wg = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), amax, amin, oracle.W_MK)
    xt, bt = torch_port.backward(x, w.T.contiguous(), grad, tmax, tmin)
    np.testing.assert_allclose(xg, xt.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(wg, bt.numpy().T, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("density", [0.0, 0.1, 0.5, 1.0])
def test_csr_oracle_equals_dense_on_densified_weight(density):
    M, K, N = 12, 20, 5
    dense, crow, col, val = pruned_csr(M, K, density, seed=5, scale=1.0)
    if 0 < density < 1:
        val = val.clone(); val[: int(crow[1])] = -val[: int(crow[1])].abs()   # a row of negative weights
        dense = torch.zeros(M, K)
        for m in range(M):
            dense[m, col[crow[m]:crow[m + 1]]] = val[crow[m]:crow[m + 1]]
    g = torch.Generator().manual_seed(9)
    x = torch.randn(N, K, generator=g).abs()          # positive inputs: negative rows lose to the zeros
    x[0] = -x[0]
    c, amax, amin = oracle.csr_forward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), K)
    cd, dmax, dmin = oracle.forward(x.numpy(), dense.numpy(), oracle.W_MK)
    cb, bmax, bmin = brute.forward(x.numpy(), dense.numpy().T)
    assert_bits_equal(c, cd, "csr c"); assert_bits_equal(c, cb, "csr c brute")
    assert_index_equal(amax, dmax, "csr argmax"); assert_index_equal(amax, bmax, "csr argmax brute")
    assert_index_equal(amin, dmin, "csr argmin"); assert_index_equal(amin, bmin, "csr argmin brute")
    grad = torch.randn(N, M, generator=g)
    xg, vg = oracle.csr_backward(x.numpy(), crow.numpy(), col.numpy(), val.numpy(), grad.numpy(), amax, amin)
    xd, wd = oracle.backward(x.numpy(), dense.numpy(), grad.numpy(), amax, amin, oracle.W_MK)
    np.testing.assert_allclose(xg, xd, rtol=1e-6, atol=1e-7)
    rows = np.repeat(np.arange(M), np.diff(crow.numpy()))
    np.testing.assert_allclose(vg, wd[rows, col.numpy()], rtol=1e-6, atol=1e-7)


# ---- sum-of-products SpMM oracle (checker of mamtorch_kernel_sparsev1::cusparsemm) ----
def _random_sparse(rows, k, sparse_rate, seed):
    # the generator of the reference's own check, seeded (test/test_sparse.py:14-17)
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(rows, k, generator=g)
    return a * torch.bernoulli(torch.full((rows, k), 1 - sparse_rate), generator=g)


@pytest.mark.parametrize("rows,k,cols,rate", [(37, 53, 29, 0.9), (200, 310, 64, 0.7), (5, 1, 3, 0.0), (64, 64, 100, 0.99)])
def test_spmm_oracle_against_dense_matmul_and_scipy(rows, k, cols, rate):
    import scipy.sparse as sp

    a = _random_sparse(rows, k, rate, seed=rows)
    b = torch.randn(k, cols, generator=torch.Generator().manual_seed(k))
    csr = a.to_sparse_csr()
    got, floor = oracle.csr_spmm(csr.crow_indices().numpy(), csr.col_indices().numpy(), csr.values().numpy(), b.numpy())
    want = a.numpy().astype(np.float64) @ b.numpy().astype(np.float64)
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max() + 1e-30
    np.testing.assert_allclose(floor, np.abs(a.numpy()).astype(np.float64) @ np.abs(b.numpy()).astype(np.float64), rtol=1e-6)
    lib_result = sp.csr_matrix((csr.values().numpy().astype(np.float64), csr.col_indices().numpy(),
                                csr.crow_indices().numpy()), shape=(rows, k)) @ b.numpy().astype(np.float64)
    assert np.abs(got - lib_result).max() <= 1e-6 * np.abs(want).max() + 1e-30


def test_spmm_oracle_coo_any_order_and_duplicates():
    # hand-derived: [[1,0,2],[0,0,0],[0,3,0]] with the (0,2) entry given as 0.5 + 1.5 and shuffled order
    row = np.array([2, 0, 0, 0], dtype=np.int64)
    col = np.array([1, 2, 0, 2], dtype=np.int64)
    val = np.array([3.0, 0.5, 1.0, 1.5], dtype=np.float32)
    b = np.array([[1.0, 2.0], [3.0, 4.0], [5.0, -6.0]], dtype=np.float32)
    c, floor = oracle.coo_spmm(row, col, val, b, 3)
    np.testing.assert_array_equal(c, np.array([[11.0, -10.0], [0.0, 0.0], [9.0, 12.0]], dtype=np.float32))
    np.testing.assert_array_equal(floor, np.array([[11.0, 14.0], [0.0, 0.0], [9.0, 12.0]], dtype=np.float32))


# ---- pruning rule and dense -> CSR compaction oracle ----
def test_prune_oracle_hand_derived():
    from oracle import prune as po

    w = np.array([[0.5, -0.2, 0.0, 0.3], [-0.3, 0.31, 0.29, -1.0]], dtype=np.float32)
    crow, col, val = po.to_csr(w, 0.3)                     # |w| <= 0.3 goes: ties at the threshold go too
    np.testing.assert_array_equal(crow, [0, 1, 3])
    np.testing.assert_array_equal(col, [0, 1, 3])
    np.testing.assert_array_equal(val, np.array([0.5, 0.31, -1.0], dtype=np.float32))
    g = np.array([[1.0, 10.0, 5.0, -1.0], [0.0, 1.0, 2.0, 0.1]], dtype=np.float32)
    np.testing.assert_array_equal(po.apply(w, 0.3, po.WEIGHT_TIMES, g),
                                  np.array([[0.5, -0.2, 0.0, 0.0], [0.0, 0.31, 0.29, 0.0]], dtype=np.float32))
    a = np.array([[0, 2, 1, 0], [3, 0, 0, 1]], dtype=np.int32)
    b = np.array([[0, 0, 0, 1], [0, 0, 1, 0]], dtype=np.int32)
    np.testing.assert_array_equal(po.keep_mask(w, 1.0, po.COUNT, a, b),
                                  [[False, True, False, False], [True, False, False, False]])


@pytest.mark.parametrize("p", [0.0, 0.5, 0.9, 0.99])
def test_prune_oracle_against_the_literal_torch_rule(p):
    from oracle import prune as po

    g = torch.Generator().manual_seed(int(p * 100))
    w = torch.randn(37, 101, generator=g) * 0.02
    grad = torch.randn(37, 101, generator=g)
    for mode, score in ((po.MAGNITUDE, w), (po.WEIGHT_TIMES, w * grad)):
        thr = float(torch.quantile(score.flatten().abs(), p))      # pruning_utils.py:104
        want = w.clone()
        want[score.abs() <= thr] = 0                                # pruning_utils.py:105
        np.testing.assert_array_equal(po.apply(w.numpy(), thr, mode, grad.numpy()), want.numpy())
        crow, col, val = po.to_csr(w.numpy(), thr, mode, grad.numpy())
        csr = want.to_sparse_csr()                                  # drops the zeros the rule wrote
        kept_nonzero = val != 0
        np.testing.assert_array_equal(col[kept_nonzero], csr.col_indices().numpy())
        np.testing.assert_array_equal(val[kept_nonzero], csr.values().numpy())
        assert crow[-1] == len(col) and abs(len(col) / w.numel() - (1 - p)) < 0.02


def test_conv_oracle_known_answers_and_cross_checks():
    """The MAM convolution of the reference's retired kernels: hand-derived known answers
    (tests/golden/kat_conv.json), the numpy window builder + C oracle against the pure-Python scalar
    loops, the window matrix against torch's own unfold (other column order, permuted here), and the
    backward against autograd of the gather formulation."""
    import json
    import os

    import torch
    import torch.nn.functional as F
    from oracle import brute

    here = os.path.dirname(os.path.abspath(__file__))
    for kat in json.load(open(os.path.join(here, "golden", "kat_conv.json"))):
        x = np.array(kat["x"], np.float32)[:, :, None, :]
        w = np.array(kat["w"], np.float32)[:, :, None, :]
        for fn in (brute.conv_forward, oracle.conv_forward):
            y, amax, amin = fn(x, w, (1, kat["stride"]))
            assert y[:, :, 0].tolist() == kat["y"], kat["name"]
            assert amax[:, :, 0].tolist() == kat["argmax"] and amin[:, :, 0].tolist() == kat["argmin"], kat["name"]
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 6, 7)).astype(np.float32)
    w = rng.standard_normal((4, 3, 2, 3)).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    for stride in ((1, 1), (2, 1), (1, 3)):
        a = brute.conv_forward(x, w, stride, bias)
        b = oracle.conv_forward(x, w, stride, bias)
        assert all(np.array_equal(u.view(np.int32), v.view(np.int32)) for u, v in zip(a, b))
        # torch's unfold orders columns (c, j1, j2); ours is (j2, j1, c)
        cols = oracle.conv_windows(x, 2, 3, *stride)
        unf = F.unfold(torch.tensor(x), (2, 3), stride=stride)                     # (B, C*k1*k2, L)
        unf = unf.view(2, 3, 2, 3, -1).permute(0, 4, 3, 2, 1).reshape(cols.shape)   # (B, L, j2, j1, c)
        assert np.array_equal(cols, unf.numpy())
        # backward: autograd of y = p[argmax] + p[argmin] over the window matrix
        grad = rng.standard_normal(a[0].shape).astype(np.float32)
        xg, wg = brute.conv_backward(x, w, grad, a[1], a[2], stride)
        xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
        u = F.unfold(xt, (2, 3), stride=stride).view(2, 3, 2, 3, -1).permute(0, 4, 3, 2, 1).reshape(cols.shape[0], -1)
        wm = wt.permute(0, 3, 2, 1).reshape(4, -1)
        prods = u[:, None, :] * wm[None, :, :]                                      # (rows, F, q)
        L = a[1].shape[2] * a[1].shape[3]
        i1 = torch.tensor(a[1]).permute(0, 2, 3, 1).reshape(-1, 4, 1).long()
        i2 = torch.tensor(a[2]).permute(0, 2, 3, 1).reshape(-1, 4, 1).long()
        yy = prods.gather(2, i1) + prods.gather(2, i2)
        gflat = torch.tensor(grad, dtype=torch.float64).permute(0, 2, 3, 1).reshape(-1, 4, 1)
        (yy * gflat).sum().backward()
        assert np.allclose(xg, xt.grad.numpy(), rtol=1e-5, atol=1e-6) and np.allclose(wg, wt.grad.numpy(), rtol=1e-5, atol=1e-6)
        assert L > 0


# ---- NaN products: ignored by ordered compares, as by the reference kernel ----

def test_nan_products_known_answers():
    """Hand-derived.  (1) products [nan, 1, 2]: max 2 at k 2, min 1 at k 1, c = 3.  (2) products
    [3, nan, -1, nan]: max 3 at 0, min -1 at 2, c = 2.  (3) every product NaN: the extremes keep their
    starting values -inf / +inf (c = nan) and both indices stay 0.  (4) products [nan, -inf, -inf]: the
    max never rises above its start, index 0; the min is -inf, first held by k 1."""
    nan, inf = float("nan"), float("inf")
    cases = [
        ([[nan, 1, 2]], [[1], [1], [1]], 3.0, 2, 1),
        ([[3, 1, -1, 2]], [[1], [nan], [1], [nan]], 2.0, 0, 2),
        ([[nan, nan]], [[1], [2]], nan, 0, 0),
        ([[nan, -inf, -inf]], [[1], [1], [1]], -inf, 0, 1),
    ]
    for a, b, c_want, imax, imin in cases:
        a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
        for c, amax, amin in (oracle.forward(a, b), oracle.forward(a, np.ascontiguousarray(b.T), oracle.W_MK),
                              brute.forward(a, b)):
            assert_bits_equal(c, np.asarray([[c_want]], np.float32), "nan kat c")
            assert (int(amax[0, 0]), int(amin[0, 0])) == (imax, imin)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_nan_products_c_scan_equals_brute_force(seed):
    """The C scan against the pure-Python statement (values sorted out first, index found afterwards) on
    inputs with NaNs at k = 0, in the middle of rows, in whole rows of x, whole columns of w, and with
    infinities of both signs."""
    rng = np.random.default_rng(seed)
    N, K, M = 7, 19, 6
    x = rng.standard_normal((N, K)).astype(np.float32)
    w = rng.standard_normal((M, K)).astype(np.float32)
    x[0, 0] = np.nan
    x[1, 7] = np.nan
    x[2, :] = np.nan
    w[3, :] = np.nan
    w[4, 0] = np.nan
    x[5, 3] = np.inf
    x[6, 0] = -np.inf
    w[5, 3] = 0.0                     # inf * 0 = nan
    with np.errstate(invalid="ignore"):
        c, amax, amin = oracle.forward(x, w, oracle.W_MK)
        cb, bmax, bmin = brute.forward(x, np.ascontiguousarray(w.T))
    assert_bits_equal(c, cb, "nan c")
    assert_index_equal(amax, bmax, "nan argmax")
    assert_index_equal(amin, bmin, "nan argmin")
    assert np.isnan(c[2]).all() and (amax[2] == 0).all() and (amin[:, 3] == 0).all()
