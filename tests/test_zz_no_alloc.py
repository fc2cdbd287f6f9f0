"""The entry point that allocates nothing (mam_fc_forward_static) against mam_fc_forward through the C ABI:
two calls in a row, the second with a smaller input, every output compared bit for bit."""
import ctypes

import pytest
import torch

from mamtorch_amd import capi

pytestmark = pytest.mark.gpu


def _inputs(N, K, M, seed):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(N, K, generator=gen)
    w = (torch.rand(M, K, generator=gen) * 2 - 1) / K ** 0.5
    b = torch.randn(M, generator=gen)
    return x, w, b


def _both(dev, N, K, M, seed, layout):
    x, w, b = (t.to(dev) for t in _inputs(N, K, M, seed))
    if layout == capi.W_KM:
        w = w.T.contiguous()
    ws_ref = torch.empty((2, N, M), dtype=torch.float32, device=dev)
    xs_ref = torch.empty((2, N, M), dtype=torch.float32, device=dev)
    c_ref, amax_ref, amin_ref = capi.fc_forward(x, w, layout, bias=b, w_sel=ws_ref, x_sel=xs_ref)
    c = torch.full((N, M), float("nan"), dtype=torch.float32, device=dev)
    amax = torch.full((N, M), -7, dtype=torch.int32, device=dev)
    amin = torch.full((N, M), -7, dtype=torch.int32, device=dev)
    ws = torch.full((2, N, M), float("nan"), dtype=torch.float32, device=dev)
    xs = torch.full((2, N, M), float("nan"), dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    capi.fc_forward_static(x, w, c, amax, amin, layout, bias=b, w_sel=ws, x_sel=xs)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before   # torch's allocator untouched
    assert torch.equal(c.view(torch.int32), c_ref.view(torch.int32))
    assert torch.equal(amax, amax_ref) and torch.equal(amin, amin_ref)
    assert torch.equal(ws.view(torch.int32), ws_ref.view(torch.int32))
    assert torch.equal(xs.view(torch.int32), xs_ref.view(torch.int32))


def test_static_forward_matches_workspace_forward_on_two_calls_in_a_row():
    dev = torch.device("cuda:0")
    l = capi.lib()
    limit = l.mam_fc_forward_static_limit()
    # first call: K split in two, 24 MiB of partials in the scratch array; second: smaller, K split further
    big, small = (256, 4096, 4096), (96, 2048, 640)
    for N, K, M in (big, small):
        # the query covers the worst alignment (the general tiling splits K further); aligned (out, in)
        # weights take the wave-uniform-rows tiling, whose partials are what has to fit
        assert l.mam_fc_forward_workspace(N, K, M) > 0, "the shapes of this test must use the scratch array"
    assert 2 * 3 * 256 * 4096 * 4 <= limit
    _both(dev, *big, seed=0, layout=capi.W_MK)
    _both(dev, *small, seed=1, layout=capi.W_MK)
    # the general tiling (operand b in (K, M) layout) and a shape that needs no partials at all
    _both(dev, 64, 1100, 200, seed=2, layout=capi.W_KM)
    assert l.mam_fc_forward_workspace(4096, 512, 2048) == 0
    _both(dev, 4096, 512, 2048, seed=3, layout=capi.W_MK)
    # and again the big one after the small ones: what the earlier calls left in the array does not matter
    _both(dev, *big, seed=4, layout=capi.W_MK)


def test_static_forward_refuses_what_does_not_fit():
    l = capi.lib()
    N, K, M = 224, 4096, 4224      # 3 ranges of K x 3 planes x N*M words = 34 MB of partials
    assert l.mam_fc_forward_workspace(N, K, M) > l.mam_fc_forward_static_limit()
    one = ctypes.c_void_p(16)      # never dereferenced: the size check comes before any launch
    rc = l.mam_fc_forward_static(one, K, one, K, capi.W_MK, None, one, one, one, None, None, N, K, M, None)
    assert rc == -2
    assert b"scratch" in l.mam_last_error()
