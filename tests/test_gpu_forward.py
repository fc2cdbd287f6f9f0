"""GPU parity of the dense MAM forward, driven through the C ABI (mamtorch_amd.capi).
Bar: values bit-exact (fp32 bit patterns), argmax/argmin exactly equal, against the CPU oracle."""
import contextlib
import json
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal, config1, random_case

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _dev():
    return torch.device("cuda:0")


@contextlib.contextmanager
def forward_tiling(name):
    """Option MAM_OPT_FORWARD_TILING of the library for the calls inside the block."""
    from mamtorch_amd import capi

    if name:
        assert name == "wide"
        capi.set_option(capi.OPT_FORWARD_TILING, capi.FORWARD_TILING_WIDE)
    try:
        yield
    finally:
        capi.set_option(capi.OPT_FORWARD_TILING, capi.FORWARD_TILING_AUTO)


def _run_both_layouts(x, w_mk, bias=None, what=""):
    """x (N,K), w_mk (M,K) CPU tensors.  Checks forward (+values-only) in both layouts vs the oracle."""
    from mamtorch_amd import capi

    dev = _dev()
    want = oracle.forward(x.numpy(), w_mk.numpy(), oracle.W_MK, None if bias is None else bias.numpy())
    xd = x.to(dev)
    bd = None if bias is None else bias.to(dev)
    # the (M,K) layout twice: the library picks its wave-uniform-rows tiling where the shape allows it;
    # option MAM_FORWARD_TILING_WIDE keeps it on the first tiling
    # the (K,M) operand twice as well: transposed once into the workspace and run on the (M,K) tilings where
    # the shape allows it, and as it is on the general tiling
    for layout, w, tiling in ((capi.W_MK, w_mk.contiguous(), None), (capi.W_MK, w_mk.contiguous(), "wide"),
                              (capi.W_KM, w_mk.T.contiguous(), None), (capi.W_KM, w_mk.T.contiguous(), "wide")):
        wd = w.to(dev)
        with forward_tiling(tiling):
            c, amax, amin = capi.fc_forward(xd, wd, layout, bd)
            cv = capi.fc_forward_values(xd, wd, layout, bd)
            torch.cuda.synchronize()
        tag = "%s layout=%d tiling=%s" % (what, layout, tiling or "default")
        assert_bits_equal(c.cpu().numpy(), want[0], tag + " c")
        assert_index_equal(amax.cpu().numpy(), want[1], tag + " argmax")
        assert_index_equal(amin.cpu().numpy(), want[2], tag + " argmin")
        assert_bits_equal(cv.cpu().numpy(), want[0], tag + " values-only c")
    return want


def test_known_answers():
    def conv(v):
        return [conv(e) for e in v] if isinstance(v, list) else float(v)
    for kat in json.load(open(os.path.join(GOLDEN, "kat.json"))):
        if "a" not in kat:
            continue
        a = torch.tensor(conv(kat["a"]), dtype=torch.float32)
        b = torch.tensor(conv(kat["b"]), dtype=torch.float32)
        c, amax, amin = _run_both_layouts(a, b.T.contiguous(), what=kat["name"])
        assert_bits_equal(c, np.asarray(conv(kat["c"]), np.float32), kat["name"])
        assert amax.tolist() == kat["argmax"] and amin.tolist() == kat["argmin"]


def test_golden_brute_fixtures():
    data = np.load(os.path.join(GOLDEN, "brute_small.npz"))
    for i in range(5):
        f = lambda n: torch.tensor(data["case%d_%s" % (i, n)])
        c, amax, amin = _run_both_layouts(f("x"), f("b").T.contiguous(), f("bias"), "fixture %d" % i)
        assert_bits_equal(c, data["case%d_c" % i], "fixture %d c" % i)
        assert_index_equal(amax, data["case%d_argmax" % i], "fixture %d argmax" % i)
        assert_index_equal(amin, data["case%d_argmin" % i], "fixture %d argmin" % i)


def test_config1_bit_exact():
    x, w, bias, _ = config1()
    _run_both_layouts(x, w, bias, "config 1")
    _run_both_layouts(x, w, None, "config 1 no bias")


@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 7, 1), (2, 3, 5), (63, 31, 127), (64, 32, 128), (65, 33, 129),
                                   (130, 257, 70), (17, 1001, 19), (300, 8, 300), (5, 4097, 9)])
def test_ragged_shapes(shape):
    N, K, M = shape
    x, w, _ = random_case(N, K, M, seed=N + K + M)
    _run_both_layouts(x, w, None, "shape %s" % (shape,))


@pytest.mark.parametrize("seed", range(4))
def test_random_shapes_like_the_reference_test(seed):
    # the reference draws n, m, l uniformly from [10, 1000] (test/test.py:12-14)
    rng = np.random.default_rng(100 + seed)
    N, K, M = (int(v) for v in rng.integers(10, 1001, 3))
    x, w, _ = random_case(N, K, M, seed)
    _run_both_layouts(x, w, None, "random %d,%d,%d" % (N, K, M))


def test_ties_take_the_lowest_index():
    g = torch.Generator().manual_seed(1)
    N, K, M = 70, 200, 140
    # coarse values: products collide constantly, including exact zeros and +-0
    x = torch.round(torch.randn(N, K, generator=g) * 2)
    w = torch.round(torch.randn(M, K, generator=g) * 2)
    want = _run_both_layouts(x, w, None, "quantised")
    prod = x.numpy()[:, :, None] * w.numpy().T[None, :, :]
    tied = (prod == prod.max(axis=1, keepdims=True)).sum(axis=1) > 1
    assert tied.mean() > 0.15                    # a good share of the maxima really are tied
    # all products equal
    _run_both_layouts(torch.ones(9, 50), torch.full((11, 50), 5.0), None, "all equal")
    # a zero row of x: every product is +-0, the sign comes from the first product
    x = torch.randn(6, 40, generator=g); x[2] = 0.0; x[4] = -0.0
    w = torch.randn(9, 40, generator=g)
    _run_both_layouts(x, w, None, "zero rows")
    # duplicate columns of k far apart (different LDS tiles, different groups of 8)
    x = torch.randn(20, 300, generator=g); w = torch.randn(33, 300, generator=g)
    x[:, 290] = x[:, 3]; w[:, 290] = w[:, 3]; x[:, 3] *= 50; x[:, 290] *= 50
    want = _run_both_layouts(x, w, None, "far duplicates")
    assert not (want[1] == 290).any() and not (want[2] == 290).any()


def test_extremes_that_the_reference_kernel_gets_wrong():
    g = torch.Generator().manual_seed(2)
    # all products negative (the reference's max accumulator starts at +1.18e-38)
    x = torch.rand(10, 64, generator=g) + 0.5
    w = -(torch.rand(12, 64, generator=g) + 0.5)
    want = _run_both_layouts(x, w, None, "all negative")
    assert (want[0] < 0).all()
    # subnormal products must not be flushed
    x = torch.full((4, 16), 1e-20) * (torch.rand(4, 16, generator=g) + 0.5)
    w = torch.full((5, 16), 1e-20) * (torch.rand(5, 16, generator=g) - 0.5)
    want = _run_both_layouts(x, w, None, "subnormal")
    assert np.abs(want[0]).max() < 1.2e-38 and np.abs(want[0]).max() > 0
    # huge dynamic range and infinities of the same sign
    x = torch.randn(8, 40, generator=g) * 1e30
    w = torch.randn(7, 40, generator=g) * 1e30
    want = _run_both_layouts(x, w, None, "overflow to inf")
    assert np.isinf(want[0]).any() or np.isnan(want[0]).any()


def test_pruned_dense_weight_with_many_zeros():
    g = torch.Generator().manual_seed(3)
    N, K, M = 96, 512, 160
    x = torch.randn(N, K, generator=g)
    w = torch.randn(M, K, generator=g) * (torch.rand(M, K, generator=g) < 0.05)
    w[0] = 0.0
    w[1] = -w[1].abs()
    _run_both_layouts(x, w, None, "95% zeros")


@pytest.mark.parametrize("shape", [(1, 64, 1), (33, 128, 130), (70, 192, 300), (31, 640, 127), (257, 4096, 129),
                                   (40, 8192, 260)])
def test_ragged_batch_and_neurons_on_whole_k_tiles(shape):
    # K is a multiple of 64, so the (M,K) layout takes the wave-uniform-rows tiling: batch sizes that are no
    # multiple of its 32 rows, neuron counts that are no multiple of its 128, with and without a split of K
    N, K, M = shape
    x, w, _ = random_case(N, K, M, seed=N + M, w_scale=1.0 / K ** 0.5)
    bias = torch.randn(M, generator=torch.Generator().manual_seed(K))
    _run_both_layouts(x, w, bias, "whole k tiles %s" % (shape,))


@pytest.mark.parametrize("shape", [(1, 16, 1), (33, 48, 130), (70, 208, 300), (64, 784, 256), (31, 1072, 127),
                                   (257, 4112, 129), (40, 8240, 260), (256, 4144, 512)])
def test_partial_last_k_tile(shape):
    """K a multiple of 16 but not of 64: the wave-uniform-rows tiling ends on a partial tile of one, two or
    three 16-k groups, alone (K < 64), after whole tiles, and at the end of the last range of a split K.  The
    second case plants the extremes inside that partial tile and ties them with earlier columns."""
    N, K, M = shape
    x, w, _ = random_case(N, K, M, seed=N + K, w_scale=1.0 / K ** 0.5)
    bias = torch.randn(M, generator=torch.Generator().manual_seed(K))
    _run_both_layouts(x, w, bias, "partial tile %s" % (shape,))
    x2, w2 = x.clone(), w.clone()
    tail0 = K - K % 64
    x2[:, K - 1] = 50.0
    w2[:, K - 1] = torch.where(torch.arange(M) % 2 == 0, 1.0, -1.0)
    x2[:, tail0] = 50.0
    w2[:, tail0] = w2[:, K - 1]
    if tail0 >= 64:
        x2[N // 2:, 3] = 50.0
        w2[:, 3] = w2[:, K - 1]
    _run_both_layouts(x2, w2, None, "partial tile, planted %s" % (shape,))


def test_aligned_views_with_longer_rows_on_whole_k_tiles():
    """Aligned 128-k windows of wider x and weight matrices (module splits > 1): row strides exceed K."""
    from mamtorch_amd import capi

    dev = _dev()
    g = torch.Generator().manual_seed(14)
    N, M, Kfull = 45, 200, 384
    x = torch.randn(N, Kfull, generator=g); w = torch.randn(M, Kfull, generator=g)
    xd, wd = x.to(dev), w.to(dev)
    for k0 in (0, 128, 256):
        c, amax, amin = capi.fc_forward(xd.narrow(1, k0, 128), wd.narrow(1, k0, 128), capi.W_MK)
        cv = capi.fc_forward_values(xd.narrow(1, k0, 128), wd.narrow(1, k0, 128), capi.W_MK)
        torch.cuda.synchronize()
        want = oracle.forward(x[:, k0:k0 + 128].contiguous().numpy(), w[:, k0:k0 + 128].contiguous().numpy(), oracle.W_MK)
        assert_bits_equal(c.cpu().numpy(), want[0], "window %d c" % k0)
        assert_index_equal(amax.cpu().numpy(), want[1], "window %d argmax" % k0)
        assert_index_equal(amin.cpu().numpy(), want[2], "window %d argmin" % k0)
        assert_bits_equal(cv.cpu().numpy(), want[0], "window %d values-only c" % k0)


def test_strided_rows_and_unaligned_views():
    from mamtorch_amd import capi

    dev = _dev()
    g = torch.Generator().manual_seed(4)
    N, K, M, off, sub = 50, 96, 70, 5, 37
    x = torch.randn(N, K, generator=g); w = torch.randn(M, K, generator=g)
    xd, wd = x.to(dev), w.to(dev)
    # narrow along K: row stride stays K, base pointer is only 4-byte aligned
    xv, wv = xd.narrow(1, off, sub), wd.narrow(1, off, sub)
    c, amax, amin = capi.fc_forward(xv, wv, capi.W_MK)
    want = oracle.forward(x[:, off:off + sub].numpy(), w[:, off:off + sub].numpy(), oracle.W_MK)
    torch.cuda.synchronize()
    assert_bits_equal(c.cpu().numpy(), want[0], "narrow c")
    assert_index_equal(amax.cpu().numpy(), want[1], "narrow argmax")
    assert_index_equal(amin.cpu().numpy(), want[2], "narrow argmin")
    # (K, M) operand narrowed along K (rows) and along M (row stride > M)
    b = w.T.contiguous().to(dev)
    c, amax, amin = capi.fc_forward(xv, b.narrow(0, off, sub), capi.W_KM)
    torch.cuda.synchronize()
    assert_bits_equal(c.cpu().numpy(), want[0], "narrow KM c")
    bm = b.narrow(1, 3, 41)
    c, amax, amin = capi.fc_forward(xd, bm, capi.W_KM)
    want = oracle.forward(x.numpy(), w[3:44].numpy(), oracle.W_MK)
    torch.cuda.synchronize()
    assert_bits_equal(c.cpu().numpy(), want[0], "column-narrowed KM c")
    assert_index_equal(amax.cpu().numpy(), want[1], "column-narrowed KM argmax")


@pytest.mark.parametrize("shape", [(256, 4096, 512), (64, 8192, 128), (100, 1000, 257), (256, 2048, 1024)])
def test_split_k_path(shape):
    from mamtorch_amd import capi

    N, K, M = shape
    assert capi.lib().mam_fc_forward_workspace(N, K, M) > 0, "shape no longer exercises split-K"
    x, w, _ = random_case(N, K, M, seed=7, w_scale=1.0 / K ** 0.5)
    bias = torch.randn(M, generator=torch.Generator().manual_seed(8))
    _run_both_layouts(x, w, bias, "split-K %s" % (shape,))
    # ties across splits: one dominant column of k planted again in every K range
    x2, w2 = x.clone(), w.clone()
    x2[:, 5] *= 100
    planted = list(range(100, K, K // 8))
    for k in planted:
        x2[:, k] = x2[:, 5]
        w2[:, k] = w2[:, 5]
    want = _run_both_layouts(x2, w2, None, "split-K ties %s" % (shape,))
    assert (want[1] == 5).mean() > 0.3 and (want[2] == 5).mean() > 0.3
    assert not np.isin(want[1], planted).any() and not np.isin(want[2], planted).any()


def test_workspace_is_required_and_checked():
    from mamtorch_amd import capi

    dev = _dev()
    N, K, M = 256, 4096, 512
    x, w, _ = random_case(N, K, M, seed=1)
    need = capi.lib().mam_fc_forward_workspace(N, K, M)
    small = torch.empty(need // 2, dtype=torch.uint8, device=dev)
    with pytest.raises(capi.MamError) as e:
        capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK, workspace=small)
    assert e.value.code == -3 and "workspace" in str(e.value)


def test_headline_config2_full_size():
    """N256 K4096 M4096, x~N(0,1), W~U(+-1/64): every value and index against the C oracle."""
    g = torch.Generator().manual_seed(0)
    N, K, M = 256, 4096, 4096
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / 64
    _run_both_layouts(x, w, None, "config 2")


@pytest.mark.parametrize("dims", [(768, 3072), (3072, 768)])
def test_vit_mlp_config3_shapes(dims):
    """N = 64 x 197 = 12608 token rows; oracle on a fixed sample of rows, size-independent
    properties on all rows."""
    from mamtorch_amd import capi

    dev = _dev()
    K, M = dims
    N = 12608
    g = torch.Generator().manual_seed(K)
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / K ** 0.5
    xd, wd = x.to(dev), w.to(dev)
    c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK)
    cv = capi.fc_forward_values(xd, wd, capi.W_MK)
    torch.cuda.synchronize()
    rows = torch.arange(0, N, 13)
    want = oracle.forward(x[rows].numpy(), w.numpy(), oracle.W_MK)
    assert_bits_equal(c[rows.to(dev)].cpu().numpy(), want[0], "config 3 c")
    assert_index_equal(amax[rows.to(dev)].cpu().numpy(), want[1], "config 3 argmax")
    assert_index_equal(amin[rows.to(dev)].cpu().numpy(), want[2], "config 3 argmin")
    assert torch.equal(c, cv)
    # the selected products reproduce c on every row
    pm = torch.gather(xd, 1, amax.long()) * wd[torch.arange(M, device=dev)[None, :], amax.long()]
    pn = torch.gather(xd, 1, amin.long()) * wd[torch.arange(M, device=dev)[None, :], amin.long()]
    assert torch.equal(pm + pn, c)
    # permuting the batch rows permutes the outputs
    perm = torch.randperm(N, generator=g).to(dev)
    c2, amax2, amin2 = capi.fc_forward(xd[perm].contiguous(), wd, capi.W_MK)
    assert torch.equal(c2, c[perm]) and torch.equal(amax2, amax[perm]) and torch.equal(amin2, amin[perm])


@pytest.mark.parametrize("shape", [(64, 2048, 256), (40, 2112, 72), (256, 4096, 128), (2048, 2048, 1024), (2080, 2240, 1000)])
@pytest.mark.parametrize("data", ["ties", "plain", "zeros"])
def test_indices_recorded_per_32_products(shape, data):
    """From K = 2048 on (whole 64-k tiles) the wave-uniform-rows tiling records the group of an extreme once per
    32 products instead of 16, and the resolve scans 32: the small shapes take the K split and the merge kernel,
    the large ones the kernel's own epilogue.  Quantised operands make most products tie, also across the two
    halves of a span and across spans; the first index must still win.  Oracle on a sample of the rows, the
    selected products reproduce c on all of them, and the general tiling (groups of 16) agrees bit for bit."""
    from mamtorch_amd import capi

    dev = _dev()
    N, K, M = shape
    g = torch.Generator().manual_seed(N + K + M)
    x = torch.randn(N, K, generator=g)
    w = torch.randn(M, K, generator=g)
    if data == "ties":
        x, w = torch.round(x), torch.round(w * 2) / 2
    elif data == "zeros":                       # extremes that are zeros of either sign
        x = torch.where(torch.rand(N, K, generator=g) < 0.5, torch.zeros(()), -x.abs())
        w = torch.where(torch.rand(M, K, generator=g) < 0.5, -torch.zeros(()), w.abs())
    xd, wd = x.to(dev), w.to(dev)
    text = capi.fc_forward_describe(xd, wd, capi.W_MK)
    assert "indices per 32 k" in text, text
    w_sel = torch.empty(2, N, M, device=dev)
    x_sel = torch.empty(2, N, M, device=dev)
    c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK, w_sel=w_sel, x_sel=x_sel)
    cv = capi.fc_forward_values(xd, wd, capi.W_MK)
    torch.cuda.synchronize()
    rows = torch.arange(0, N, max(1, N // 48))
    want = oracle.forward(x[rows].numpy(), w.numpy(), oracle.W_MK)
    assert_bits_equal(c[rows.to(dev)].cpu().numpy(), want[0], "c")
    assert_index_equal(amax[rows.to(dev)].cpu().numpy(), want[1], "argmax")
    assert_index_equal(amin[rows.to(dev)].cpu().numpy(), want[2], "argmin")
    assert torch.equal(c.view(torch.int32), cv.view(torch.int32))
    cols = torch.arange(M, device=dev)[None, :]
    assert torch.equal(w_sel[0], wd[cols, amax.long()]) and torch.equal(w_sel[1], wd[cols, amin.long()])
    assert torch.equal(x_sel[0], torch.gather(xd, 1, amax.long())) and torch.equal(x_sel[1], torch.gather(xd, 1, amin.long()))
    assert torch.equal((w_sel[0] * x_sel[0] + w_sel[1] * x_sel[1]).view(torch.int32), c.view(torch.int32))
    with forward_tiling("wide"):
        c2, amax2, amin2 = capi.fc_forward(xd, wd, capi.W_MK)
        torch.cuda.synchronize()
    assert torch.equal(c2.view(torch.int32), c.view(torch.int32))
    assert torch.equal(amax2, amax) and torch.equal(amin2, amin)


@pytest.mark.parametrize("M", [1024, 4096])
def test_large_batch_inference_config4(M):
    """N16384 K4096, x~U(-1,1), W~N(0,0.02): oracle on sampled rows + properties on all."""
    from mamtorch_amd import capi

    dev = _dev()
    N, K = 16384, 4096
    g = torch.Generator().manual_seed(M)
    x = torch.rand(N, K, generator=g) * 2 - 1
    w = torch.randn(M, K, generator=g) * 0.02
    xd, wd = x.to(dev), w.to(dev)
    c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK)
    torch.cuda.synchronize()
    rows = torch.arange(5, N, 257)
    want = oracle.forward(x[rows].numpy(), w.numpy(), oracle.W_MK)
    assert_bits_equal(c[rows.to(dev)].cpu().numpy(), want[0], "config 4 c")
    assert_index_equal(amax[rows.to(dev)].cpu().numpy(), want[1], "config 4 argmax")
    assert_index_equal(amin[rows.to(dev)].cpu().numpy(), want[2], "config 4 argmin")
    cols = torch.arange(M, device=dev)[None, :]
    pm = torch.gather(xd, 1, amax.long()) * wd[cols, amax.long()]
    pn = torch.gather(xd, 1, amin.long()) * wd[cols, amin.long()]
    assert torch.equal(pm + pn, c)
    assert bool((pm >= pn).all())
    # the (K, M) operand gives the same answer
    c2, amax2, amin2 = capi.fc_forward(xd[:2048], wd.T.contiguous(), capi.W_KM)
    assert torch.equal(c2, c[:2048]) and torch.equal(amax2, amax[:2048]) and torch.equal(amin2, amin[:2048])


def test_large_batch_inference_config4_out16384():
    """The largest forward of the configurations: N16384 K4096 M16384 (1.1 T triples, 3 x 1 GiB of outputs,
    a 256 MiB weight): oracle on sampled rows (bits and indices), and on ALL rows, in slabs of 2048 rows,
    the selected products reproduce c, max >= min, indices in range, values-only forward equal."""
    from mamtorch_amd import capi

    dev = _dev()
    N, K, M = 16384, 4096, 16384
    g = torch.Generator().manual_seed(16384)
    x = torch.rand(N, K, generator=g) * 2 - 1
    w = torch.randn(M, K, generator=g) * 0.02
    xd, wd = x.to(dev), w.to(dev)
    assert capi.lib().mam_fc_forward_workspace(N, K, M) == 0
    c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK)
    torch.cuda.synchronize()
    rows = torch.arange(7, N, 1021)       # 17 rows, among them rows of the first and of the last row tile
    rows = torch.cat([rows, torch.tensor([0, N - 1])])
    want = oracle.forward(x[rows].numpy(), w.numpy(), oracle.W_MK)
    assert_bits_equal(c[rows.to(dev)].cpu().numpy(), want[0], "config 4 out 16384 c")
    assert_index_equal(amax[rows.to(dev)].cpu().numpy(), want[1], "config 4 out 16384 argmax")
    assert_index_equal(amin[rows.to(dev)].cpu().numpy(), want[2], "config 4 out 16384 argmin")
    del want
    cols = torch.arange(M, device=dev)[None, :]
    for r0 in range(0, N, 2048):
        sl = slice(r0, r0 + 2048)
        i1, i2 = amax[sl].long(), amin[sl].long()
        assert int(i1.min()) >= 0 and int(i1.max()) < K and int(i2.min()) >= 0 and int(i2.max()) < K
        pm = torch.gather(xd[sl], 1, i1) * wd[cols, i1]
        pn = torch.gather(xd[sl], 1, i2) * wd[cols, i2]
        assert torch.equal(pm + pn, c[sl]), "rows %d.." % r0
        assert bool((pm >= pn).all())
        del i1, i2, pm, pn
    del amax, amin
    cv = capi.fc_forward_values(xd, wd, capi.W_MK)
    torch.cuda.synchronize()
    assert torch.equal(cv, c)


@pytest.mark.parametrize("shape", [(64, 784, 256), (256, 4096, 512), (70, 123, 45), (300, 2048, 200)])
def test_selected_weights_output(shape):
    """w_sel[0] = w[argmax[n,m], m], w_sel[1] = w[argmin[n,m], m], x_sel[0] = x[n, argmax[n,m]],
    x_sel[1] = x[n, argmin[n,m]] (exact copies), both layouts, both tilings."""
    from mamtorch_amd import capi

    dev = _dev()
    N, K, M = shape
    x, w, _ = random_case(N, K, M, seed=11)
    want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
    cols = np.arange(M)[None, :]
    rows = np.arange(N)[:, None]
    for layout, wl, tiling in ((capi.W_MK, w.contiguous(), None), (capi.W_MK, w.contiguous(), "wide"),
                               (capi.W_KM, w.T.contiguous(), None)):
        w_sel = torch.full((2, N, M), float("nan"), device=dev)
        x_sel = torch.full((2, N, M), float("nan"), device=dev)
        with forward_tiling(tiling):
            c, amax, amin = capi.fc_forward(x.to(dev), wl.to(dev), layout, w_sel=w_sel, x_sel=x_sel)
            torch.cuda.synchronize()
        what = "layout %d tiling %s" % (layout, tiling)
        assert_bits_equal(c.cpu().numpy(), want[0], "c " + what)
        assert_index_equal(amax.cpu().numpy(), want[1], "argmax " + what)
        assert_bits_equal(w_sel[0].cpu().numpy(), w.numpy()[cols, want[1]], "w_sel max " + what)
        assert_bits_equal(w_sel[1].cpu().numpy(), w.numpy()[cols, want[2]], "w_sel min " + what)
        assert_bits_equal(x_sel[0].cpu().numpy(), x.numpy()[rows, want[1]], "x_sel max " + what)
        assert_bits_equal(x_sel[1].cpu().numpy(), x.numpy()[rows, want[2]], "x_sel min " + what)
        # only one of the two asked for
        x_only = torch.full((2, N, M), float("nan"), device=dev)
        with forward_tiling(tiling):
            capi.fc_forward(x.to(dev), wl.to(dev), layout, x_sel=x_only)
            torch.cuda.synchronize()
        assert torch.equal(x_only, x_sel)


def test_nan_products_are_ignored():
    """NaN products never win and never stick (ordered compares, as in the reference kernel): NaN at k = 0,
    in mid-row, a whole row of x and a whole weight row, on both tilings, unsplit and with K split."""
    g = torch.Generator().manual_seed(21)
    for N, K, M in ((40, 128, 70), (48, 2048, 256)):        # the second shape splits K
        x = torch.randn(N, K, generator=g)
        w = torch.randn(M, K, generator=g)
        x[0, 0] = float("nan")
        x[1, K // 2 + 3] = float("nan")
        x[2, :] = float("nan")
        w[3, :] = float("nan")
        w[4, 0] = float("nan")
        w[5, K - 1] = float("nan")
        x[6, 17] = float("nan")
        w[6, 17] = float("nan")
        _run_both_layouts(x, w, None, "nan products %dx%dx%d" % (N, K, M))


def test_merge_inside_the_forward_launch_gives_the_same_bits():
    """MAM_FORWARD_TILING_FUSED_MERGE: the last of a tile's workgroups to finish combines the K ranges and resolves
    in its own epilogue (no merge kernel).  Kept for comparisons (it is slower: 0.234 against 0.212 ms at
    256 x 4096 x 4096); its results must be those of the shipped pair, and of the oracle."""
    from mamtorch_amd import capi

    dev = _dev()
    g = torch.Generator().manual_seed(31)
    for N, K, M in ((48, 2048, 256), (100, 4096, 200)):
        x = torch.randn(N, K, generator=g)
        w = torch.randn(M, K, generator=g)
        x[3, :] = 0.0                       # ties and zero signs across the K ranges
        w[5, K // 2:] = w[5, :K // 2]
        want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)
        xd, wd = x.to(dev), w.to(dev)
        ws = torch.empty(2, N, M, device=dev)
        xs = torch.empty(2, N, M, device=dev)
        capi.set_option(capi.OPT_FORWARD_TILING, 3)
        try:
            assert "split" in capi.fc_forward_describe(xd, wd, capi.W_MK)
            for _ in range(2):              # the tickets are cleared per call
                c, amax, amin = capi.fc_forward(xd, wd, capi.W_MK, w_sel=ws, x_sel=xs)
                torch.cuda.synchronize()
                assert_bits_equal(c.cpu().numpy(), want[0], "fused merge c")
                assert_index_equal(amax.cpu().numpy(), want[1], "fused merge argmax")
                assert_index_equal(amin.cpu().numpy(), want[2], "fused merge argmin")
        finally:
            capi.set_option(capi.OPT_FORWARD_TILING, capi.FORWARD_TILING_AUTO)
        cols = torch.arange(M)[None, :]
        assert torch.equal(ws[0].cpu(), w[cols, torch.tensor(want[1]).long()])
        assert torch.equal(xs[1].cpu(), x[torch.arange(N)[:, None], torch.tensor(want[2]).long()])
