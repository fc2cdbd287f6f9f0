"""Pure-PyTorch CPU restatement of the reference's MAM oracle -- TEST INFRASTRUCTURE ONLY.

Semantics of test/reference.py:3-10 (forward, beta = 0) and test/reference.py:12-25
(backward, beta = 0 branch) of SSIGPRO/mamtorch, re-expressed so that the N*K*M product
tensor is never materialised: rows of the batch are independent, so the batch is processed
in chunks (identical results).  The backward uses index_put with accumulation instead of
the reference's per-row dense mask; the sums are the same terms.

This is the "cpu_baseline" (kind "port") that bench.py times on the host cores.
"""
import torch


def forward(a, b, bias=None, chunk_elems=1 << 26):
    """a (N,K), b (K,M) CPU fp32 -> y (N,M), argmax (N,M) int32, argmin (N,M) int32."""
    N, K = a.shape
    M = b.shape[1]
    rows = max(1, min(N, chunk_elems // max(1, K * M)))
    y = torch.empty((N, M), dtype=torch.float32)
    amax = torch.empty((N, M), dtype=torch.int32)
    amin = torch.empty((N, M), dtype=torch.int32)
    for r0 in range(0, N, rows):
        v = a[r0:r0 + rows, :, None] * b[None, :, :]
        hi, ih = torch.max(v, dim=1)
        lo, il = torch.min(v, dim=1)
        y[r0:r0 + rows] = hi + lo
        amax[r0:r0 + rows] = ih.to(torch.int32)
        amin[r0:r0 + rows] = il.to(torch.int32)
    if bias is not None:
        y = y + bias
    return y, amax, amin


def backward(a, b, grad, argmax, argmin):
    """-> a_grad (N,K), b_grad (K,M).  fp32 accumulation in index order."""
    N, K = a.shape
    M = b.shape[1]
    a_grad = torch.zeros_like(a)
    b_grad = torch.zeros_like(b)
    rows = torch.arange(N).view(N, 1).expand(N, M)
    cols = torch.arange(M).view(1, M).expand(N, M)
    for arg in (argmax, argmin):
        k = arg.long()
        a_grad.index_put_((rows, k), b[k, cols] * grad, accumulate=True)
        b_grad.index_put_((k, cols), a[rows, k] * grad, accumulate=True)
    return a_grad, b_grad


def selection_count_reference(argmax, argmin, max_count):
    """Literal mamtorch/nn/v4/fullyconnected.py:123-129: non-accumulating '+= 1', twice."""
    N, M = argmax.shape
    col = torch.arange(M).repeat(N)
    max_count[col, argmax.flatten().long()] += 1
    max_count[col, argmin.flatten().long()] += 1
    return max_count
