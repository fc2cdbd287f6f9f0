"""GPU parity of the selection-count kernel through the C ABI (exact integer equality)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_port

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _run(amax, amin, mc, nc, mode):
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    md, nd = torch.tensor(mc).to(dev), torch.tensor(nc).to(dev)
    capi.selection_count(torch.tensor(amax).to(dev), torch.tensor(amin).to(dev), md, nd, mode)
    torch.cuda.synchronize()
    return md.cpu().numpy(), nd.cpu().numpy()


def test_known_answer():
    kat = [k for k in json.load(open(os.path.join(GOLDEN, "kat.json"))) if k["name"] == "selection_count"][0]
    amax, amin = np.asarray(kat["sel_argmax"], np.int32), np.asarray(kat["sel_argmin"], np.int32)
    z = np.zeros((kat["M"], kat["K"]), np.int32)
    mc, nc = _run(amax, amin, z, z, 0)
    assert mc.tolist() == kat["ref_max_count"] and not nc.any()
    mc, nc = _run(amax, amin, z, z, 1)
    assert mc.tolist() == kat["hits_max_count"] and nc.tolist() == kat["hits_min_count"]


@pytest.mark.parametrize("shape", [(1, 1, 1), (4, 3, 4), (64, 256, 784), (300, 77, 100), (50, 33, 4099), (9, 5, 70001)])
@pytest.mark.parametrize("mode", [0, 1])
def test_random_indices(shape, mode):
    N, M, K = shape
    g = torch.Generator().manual_seed(N * 7 + M)
    # concentrated picks: many batch rows choose the same weight
    amax = (torch.randint(0, K, (N, M), generator=g) % max(1, K // 3)).to(torch.int32).numpy()
    amin = torch.randint(0, K, (N, M), generator=g, dtype=torch.int32).numpy()
    mc = torch.randint(0, 5, (M, K), generator=g, dtype=torch.int32).numpy()
    nc = torch.randint(0, 5, (M, K), generator=g, dtype=torch.int32).numpy()
    want = oracle.selection_count(amax, amin, mc, nc, mode)
    got = _run(amax, amin, mc, nc, mode)
    np.testing.assert_array_equal(got[0], want[0])
    np.testing.assert_array_equal(got[1], want[1])
    if mode == 0:
        lit = torch_port.selection_count_reference(torch.tensor(amax), torch.tensor(amin), torch.tensor(mc).clone())
        np.testing.assert_array_equal(got[0], lit.numpy())
    else:
        assert int(got[0].sum() - mc.sum()) == N * M and int(got[1].sum() - nc.sum()) == N * M


@pytest.mark.parametrize("M", [4, 5])
def test_more_hits_on_one_cell_than_a_16_bit_field_holds(M):
    """Hits mode counts in 16-bit LDS fields; batches above 32768 rows are walked in passes so that a field
    cannot overflow.  70000 rows that all pick the same weight must add exactly 70000 (both the 16-byte path,
    M a multiple of 4, and the element path)."""
    N, K = 70000, 8
    amax = np.full((N, M), 3, np.int32)
    amin = np.full((N, M), 5, np.int32)
    amin[:, 0] = 3                      # one neuron picks the same weight as max and as min
    z = np.zeros((M, K), np.int32)
    for mode in (1, 0, 2):
        mc, nc = _run(amax, amin, z, z, mode)
        want = oracle.selection_count(amax, amin, z, z, mode) if mode != 2 else None
        if mode == 1:
            assert mc[:, 3].tolist() == [N] * M and nc[1:, 5].tolist() == [N] * (M - 1) and nc[0, 3] == N
            assert int(mc.sum()) == N * M and int(nc.sum()) == N * M
        if want is not None:
            np.testing.assert_array_equal(mc, want[0])
            np.testing.assert_array_equal(nc, want[1])
        if mode == 2:                   # flags, max and min apart: one per picked cell
            assert int(mc.sum()) == M and int(nc.sum()) == M and mc[0, 3] == 1 and nc[0, 3] == 1


def test_headline_config2_accumulates_over_batches():
    from mamtorch_amd import capi

    dev = torch.device("cuda:0")
    N, K, M = 256, 4096, 4096
    g = torch.Generator().manual_seed(0)
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) / 64
    _, amax, amin = capi.fc_forward(x.to(dev), w.to(dev), capi.W_MK)
    a1, a2 = amax.cpu().numpy(), amin.cpu().numpy()
    for mode in (0, 1):
        mc = torch.zeros((M, K), dtype=torch.int32, device=dev)
        nc = torch.zeros((M, K), dtype=torch.int32, device=dev)
        z = np.zeros((M, K), np.int32)
        want = (z, z)
        for _ in range(2):   # two batches: the counters accumulate across calls
            capi.selection_count(amax, amin, mc, nc, mode)
            want = oracle.selection_count(a1, a2, want[0], want[1], mode)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(mc.cpu().numpy(), want[0])
        np.testing.assert_array_equal(nc.cpu().numpy(), want[1])
