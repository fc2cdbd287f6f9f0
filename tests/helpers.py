"""Shared input generators and comparison helpers for the parity tests."""
import numpy as np
import torch


def bits(a):
    """fp32 array as its int32 bit pattern: bit-exact comparison that tells +0 from -0."""
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.int32)


def assert_bits_equal(got, want, what):
    got, want = np.asarray(got), np.asarray(want)
    # NaN payload / sign is not part of the contract (inf - inf): NaN matches NaN
    bad = np.argwhere((bits(got) != bits(want)) & ~(np.isnan(got) & np.isnan(want)))
    assert bad.size == 0, "%s: %d mismatches, first at %s: got %r want %r" % (
        what, len(bad), bad[0].tolist(), got[tuple(bad[0])], want[tuple(bad[0])])


def assert_index_equal(got, want, what):
    got, want = np.asarray(got), np.asarray(want)
    bad = np.argwhere(got != want)
    assert bad.size == 0, "%s: %d mismatches, first at %s: got %r want %r" % (
        what, len(bad), bad[0].tolist(), got[tuple(bad[0])], want[tuple(bad[0])])


def config1(seed=0):
    """The small CPU-runnable configuration: N64 K784 M256, bias on, Kaiming-uniform weight, seeded on the CPU."""
    g = torch.Generator().manual_seed(seed)
    N, K, M = 64, 784, 256
    bound = 1.0 / K ** 0.5
    x = torch.randn(N, K, generator=g)
    w = (torch.rand(M, K, generator=g) * 2 - 1) * bound   # weight (out, in)
    bias = (torch.rand(M, generator=g) * 2 - 1) * bound
    grad = torch.randn(N, M, generator=g)
    return x, w, bias, grad


def random_case(N, K, M, seed, w_scale=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, K, generator=g)
    w = torch.randn(M, K, generator=g) * (w_scale if w_scale is not None else 1.0)
    grad = torch.randn(N, M, generator=g)
    return x, w, grad


def pruned_csr(M, K, density, seed, scale=0.02):
    """Per-row seeded uniform-random keep mask; surviving W ~ N(0, scale).  Returns dense W and CSR parts."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(M, K, generator=g) * scale
    keep_n = int(round(density * K))
    mask = torch.zeros(M, K, dtype=torch.bool)
    for m in range(M):
        mask[m, torch.randperm(K, generator=g)[:keep_n]] = True
    dense = torch.where(mask, w, torch.zeros_like(w))
    counts = mask.sum(dim=1)
    crow = torch.zeros(M + 1, dtype=torch.int64)
    crow[1:] = torch.cumsum(counts, 0)
    col = mask.nonzero()[:, 1].to(torch.int64).contiguous()
    val = w[mask].contiguous()
    return dense, crow, col, val
