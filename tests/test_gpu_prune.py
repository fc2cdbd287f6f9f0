"""GPU parity of pruning and dense -> CSR compaction through the C ABI: exact against the numpy oracle
(integer / bit work), plus the pipeline prune -> CSR -> sparse MAM forward against the dense forward."""
import numpy as np
import pytest
import torch

import oracle
from oracle import prune as po

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _case(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(M, K, generator=g) * 0.02
    grad = torch.randn(M, K, generator=g)
    a = torch.randint(0, 4, (M, K), generator=g, dtype=torch.int32)
    b = torch.randint(0, 2, (M, K), generator=g, dtype=torch.int32)
    return w, grad, a, b


@pytest.mark.parametrize("M,K", [(37, 101), (4, 64), (1, 1), (130, 63), (64, 4096), (300, 257)])
@pytest.mark.parametrize("p", [0.0, 0.5, 0.97])
def test_all_scores_against_oracle(M, K, p):
    from mamtorch_amd import capi

    w, grad, a, b = _case(M, K, M + K)
    cases = [(capi.PRUNE_MAGNITUDE, None, None, float(np.quantile(np.abs(w.numpy()), p))),
             (capi.PRUNE_WEIGHT_TIMES, grad, None, float(np.quantile(np.abs((w * grad).numpy()), p))),
             (capi.PRUNE_COUNT, a, None, 1.0), (capi.PRUNE_COUNT, a, b, 2.0)]
    for mode, aux, aux2, thr in cases:
        thr = float(np.float32(thr))
        np_aux = None if aux is None else aux.numpy()
        np_aux2 = None if aux2 is None else aux2.numpy()
        crow_w, col_w, val_w = po.to_csr(w.numpy(), thr, mode, np_aux, np_aux2)
        d_aux = None if aux is None else aux.to(DEV)
        d_aux2 = None if aux2 is None else aux2.to(DEV)
        crow, col, val = capi.prune_to_csr(w.to(DEV), thr, mode, d_aux, d_aux2)
        np.testing.assert_array_equal(crow.cpu().numpy(), crow_w)
        np.testing.assert_array_equal(col.cpu().numpy(), col_w)
        np.testing.assert_array_equal(val.cpu().numpy().view(np.int32), val_w.view(np.int32))
        wd = w.to(DEV).clone()
        capi.prune_apply(wd, thr, mode, d_aux, d_aux2)
        np.testing.assert_array_equal(wd.cpu().numpy().view(np.int32),
                                      po.apply(w.numpy(), thr, mode, np_aux, np_aux2).view(np.int32))


def test_strided_views_nan_scores_and_extremes():
    from mamtorch_amd import capi

    g = torch.Generator().manual_seed(5)
    wide = torch.randn(20, 200, generator=g)
    wide[3, 17] = float("nan")
    w = wide[:, 10:150]                                           # rows of 140 inside rows of 200
    grad = torch.randn(20, 300, generator=g)[:, 100:240]
    for mode, aux in ((capi.PRUNE_MAGNITUDE, None), (capi.PRUNE_WEIGHT_TIMES, grad)):
        for thr in (-1.0, 0.8, 1e30):                              # everything kept / some / only the NaN kept
            want = po.to_csr(w.numpy(), thr, mode, None if aux is None else aux.numpy())
            got = capi.prune_to_csr(wide.to(DEV)[:, 10:150], thr, mode, None if aux is None else _strided(aux))
            for gt, wt in zip(got, want):
                np.testing.assert_array_equal(gt.cpu().numpy().view(np.int32 if gt.dtype == torch.float32 else np.int64),
                                              wt.view(np.int32 if wt.dtype == np.float32 else np.int64))
    assert po.keep_mask(w.numpy(), 1e30)[3, 7]                     # the NaN entry survives any threshold


def _strided(t):
    """The same values on the device inside a wider allocation, so that the row stride exceeds the length."""
    wide = torch.zeros(t.shape[0], t.shape[1] + 24, device=DEV)
    wide[:, 8:8 + t.shape[1]] = t.to(DEV)
    return wide[:, 8:8 + t.shape[1]]


def test_empty_shapes():
    from mamtorch_amd import capi

    crow, col, val = capi.prune_to_csr(torch.empty(0, 8, device=DEV), 0.0)
    assert crow.tolist() == [0] and col.numel() == 0
    crow, col, val = capi.prune_to_csr(torch.empty(3, 0, device=DEV), 0.0)
    assert crow.tolist() == [0, 0, 0, 0] and val.numel() == 0


def test_thresholds_and_pipeline_into_the_sparse_forward():
    """Layer-wise magnitude pruning as in pruning_utils.py:103-105, compaction, CSR MAM forward: equal,
    bit for bit, to the dense MAM forward on the matrix the reference would have kept dense."""
    import mamtorch_amd as mt
    from mamtorch_amd.sparse import prune

    g = torch.Generator().manual_seed(9)
    M, K, N = 256, 512, 48
    w = (torch.randn(M, K, generator=g) * 0.02).to(DEV)
    x = torch.randn(N, K, generator=g).to(DEV)
    thr = prune.layer_threshold(w, 0.9)
    assert thr == float(torch.quantile(w.flatten().abs(), 0.9))
    assert prune.global_threshold([w[:100], w[100:]], 0.9) == float(torch.sort(w.flatten().abs())[0][int(0.9 * w.numel())])
    w_csr = prune.dense_to_csr(w, thr)
    dense = w.clone()
    prune.prune_(dense, thr)
    want_dense = w.clone()
    want_dense[w.abs() <= thr] = 0
    assert torch.equal(dense, want_dense)
    assert torch.equal(w_csr.to_dense(), want_dense)
    assert abs(w_csr.values().numel() / w.numel() - 0.1) < 0.01
    c, amax, amin = mt.sparse.fullyconnected(x, w_csr)
    cd, dmax, dmin = mt.kernel.v4.fullyconnected(x, dense.T.contiguous())
    assert torch.equal(c.view(torch.int32), cd.view(torch.int32)) and torch.equal(amax, dmax) and torch.equal(amin, dmin)
    # selection-count driven: keep what was selected at least once in this batch
    max_count = torch.zeros(M, K, dtype=torch.int32, device=DEV)
    min_count = torch.zeros(M, K, dtype=torch.int32, device=DEV)
    _, fmax, fmin = mt.kernel.v4.fullyconnected(x, w.T.contiguous())
    mt.kernel.v4.selection_count(fmax, fmin, max_count, min_count, mode=1)   # true hit counts
    sel_csr = prune.dense_to_csr(w, 0.0, counts=(max_count, min_count))
    assert sel_csr.values().numel() == int(((max_count + min_count) > 0).sum())
    c2, _, _ = mt.sparse.fullyconnected(x, sel_csr)
    full, _, _ = mt.kernel.v4.fullyconnected(x, w.T.contiguous())
    # every selected weight survived, so wherever no implicit zero wins the result is unchanged
    same = (c2 == full)
    assert float(same.float().mean()) > 0.5


def test_full_size_counts_and_order():
    from mamtorch_amd import capi

    M = K = 4096
    w = torch.randn(M, K, generator=torch.Generator().manual_seed(1)).to(DEV) * 0.02
    thr = 0.02 * 1.6449        # ~10 % of a normal distribution lies beyond 1.645 sigma
    crow, col, val = capi.prune_to_csr(w, thr)
    keep = w.abs() > thr
    assert torch.equal(crow[1:], torch.cumsum(keep.sum(1), 0))
    assert torch.equal(val, w[keep]) and torch.equal(col, keep.nonzero()[:, 1])
    idem = torch.sparse_csr_tensor(crow, col, val, size=(M, K)).to_dense()
    crow2, col2, val2 = capi.prune_to_csr(idem, thr)               # idempotence
    assert torch.equal(crow2, crow) and torch.equal(col2, col) and torch.equal(val2, val)


# ---- thresholds by radix select: no sort, bit-equal to the reference's sort-based rules ----

def _sorted_abs(*tensors):
    return torch.sort(torch.cat([t.detach().abs().float().flatten() for t in tensors]))[0]


def _quantile_by_sort(ordered, p):
    """torch.quantile's linear rule written out (rank formed in fp32, floor / ceil neighbours, lerp), on the
    CPU: it also covers inputs above torch.quantile's size limit."""
    n = ordered.numel()
    rank = torch.tensor(p, dtype=torch.float32) * (n - 1)
    lo, hi = int(torch.floor(rank)), int(torch.ceil(rank))
    return float(torch.lerp(ordered[lo].cpu(), ordered[hi].cpu(), rank - torch.floor(rank)))


@pytest.mark.parametrize("p", [0.0, 0.5, 0.9, 0.97, 0.999, 1.0])
def test_layer_threshold_equals_torch_quantile(p):
    from mamtorch_amd.sparse import prune

    w = (torch.randn(4000, 4000, generator=torch.Generator().manual_seed(2)) * 0.02).to(DEV)   # torch's limit
    got = prune.layer_threshold(w, p)
    want = float(torch.quantile(w.flatten().abs().cpu(), p))
    assert np.float32(got).view(np.int32) == np.float32(want).view(np.int32), (got, want)
    assert abs(got - float(torch.quantile(w.flatten().abs(), p))) <= 1.2e-7 * abs(want)


@pytest.mark.parametrize("p", [0.1, 0.9, 0.99])
def test_layer_threshold_at_4096_squared(p):
    """16.8 M scores: above torch.quantile's size limit; the same rule by a full sort is the yardstick."""
    from mamtorch_amd.sparse import prune

    w = (torch.randn(4096, 4096, generator=torch.Generator().manual_seed(3)) * 0.02).to(DEV)
    ordered = _sorted_abs(w)
    got = prune.layer_threshold(w, p)
    want = _quantile_by_sort(ordered, p)
    assert np.float32(got).view(np.int32) == np.float32(want).view(np.int32), (got, want)


def test_global_threshold_over_three_tensors():
    """The reference's global rule (sort of the concatenated |scores|, element int(p * n)) over tensors of
    different shapes, one of them a strided view with an unaligned start."""
    from mamtorch_amd.sparse import prune

    g = torch.Generator().manual_seed(4)
    a = (torch.randn(768, 3072, generator=g) * 0.03).to(DEV)
    b = (torch.randn(3072, 768, generator=g) * 0.01).to(DEV)
    c = (torch.randn(301, 1031, generator=g)).to(DEV)[:, 3:1001]
    ordered = _sorted_abs(a, b, c)
    for p in (0.0, 0.3, 0.9, 0.9999, 1.0):
        index = max(0, min(int(p * ordered.numel()), ordered.numel() - 1))
        got = prune.global_threshold([a, b, c], p)
        assert np.float32(got).view(np.int32) == ordered[index].cpu().numpy().view(np.int32), p


def test_thresholds_of_product_and_count_scores_and_corner_cases():
    from mamtorch_amd.sparse import prune

    g = torch.Generator().manual_seed(5)
    w = torch.randn(257, 1000, generator=g).to(DEV)
    grad = torch.randn(257, 1000, generator=g).to(DEV)
    ordered = _sorted_abs(w * grad)
    for p in (0.25, 0.9):
        got = prune.layer_threshold(w, p, factor=grad)
        assert np.float32(got).view(np.int32) == np.float32(_quantile_by_sort(ordered, p)).view(np.int32)
        index = int(p * ordered.numel())
        assert np.float32(prune.global_threshold([w], p, factors=[grad])).view(np.int32) == \
            ordered[index].cpu().numpy().view(np.int32)
    cmax = torch.randint(0, 40, (257, 1000), generator=g, dtype=torch.int32).to(DEV)
    cmin = torch.randint(0, 40, (257, 1000), generator=g, dtype=torch.int32).to(DEV)
    ordered = torch.sort((cmax + cmin).flatten().float())[0]
    for p in (0.1, 0.5, 0.95):
        assert prune.global_threshold([w], p, counts=[(cmax, cmin)]) == float(ordered[int(p * ordered.numel())])
    # ties, signed zeros, a single element, NaN scores (they order above infinity, where torch.sort puts them)
    t = torch.tensor([[0.0, -0.0, 1.0, -1.0, 1.0, float("inf"), float("nan"), -2.0]], device=DEV)
    ordered = torch.sort(t.abs().flatten())[0]
    for index in range(8):
        got = prune.global_threshold([t], (index + 0.5) / 8)
        want = float(ordered[index])
        assert (got != got and want != want) or got == want, (index, got, want)
    assert prune.global_threshold([torch.tensor([[-3.5]], device=DEV)], 0.7) == 3.5
    assert prune.layer_threshold(torch.tensor([[-3.5]], device=DEV), 0.7) == 3.5
    same = torch.full((64, 64), -0.25, device=DEV)
    assert prune.layer_threshold(same, 0.33) == 0.25 and prune.global_threshold([same, same], 0.99) == 0.25
