"""Pure-Python brute force of the MAM path for tiny inputs -- TEST INFRASTRUCTURE ONLY.

Written from the scalar definition (one numpy.float32 multiply per product, a scan in
ascending k with strict comparisons), so that it shares no code with mam_oracle.c or
torch_port.py and can pin both.  Follows mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:126-143
(scan order and tie-break) and mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:54-75.
"""
import numpy as np

f32 = np.float32


def forward(x, b, bias=None):
    """x (N,K), b (K,M) -> c, argmax, argmin"""
    x = np.asarray(x, f32)
    b = np.asarray(b, f32)
    N, K = x.shape
    M = b.shape[1]
    c = np.zeros((N, M), f32)
    amax = np.zeros((N, M), np.int32)
    amin = np.zeros((N, M), np.int32)
    for n in range(N):
        for m in range(M):
            prods = [f32(x[n, k]) * f32(b[k, m]) for k in range(K)]
            hi, lo, ih, il = prods[0], prods[0], 0, 0
            for k in range(1, K):
                if prods[k] > hi:
                    hi, ih = prods[k], k
                if prods[k] < lo:
                    lo, il = prods[k], k
            s = f32(hi + lo)
            if bias is not None:
                s = f32(s + f32(bias[m]))
            c[n, m], amax[n, m], amin[n, m] = s, ih, il
    return c, amax, amin


def backward(x, b, grad, argmax, argmin):
    """-> x_grad (N,K), b_grad (K,M); python floats (fp64) accumulate fp32 terms."""
    x = np.asarray(x, f32)
    b = np.asarray(b, f32)
    grad = np.asarray(grad, f32)
    N, K = x.shape
    M = b.shape[1]
    xg = [[0.0] * K for _ in range(N)]
    bg = [[0.0] * M for _ in range(K)]
    for n in range(N):
        for m in range(M):
            for k in (int(argmax[n, m]), int(argmin[n, m])):
                xg[n][k] += float(f32(b[k, m]) * f32(grad[n, m]))
                bg[k][m] += float(f32(x[n, k]) * f32(grad[n, m]))
    return np.asarray(xg, f32), np.asarray(bg, f32)


def selection_count(argmax, argmin, max_count, min_count, mode=0):
    mc = np.array(max_count, np.int32, copy=True)
    nc = np.array(min_count, np.int32, copy=True)
    N, M = np.asarray(argmax).shape
    if mode == 1:
        for n in range(N):
            for m in range(M):
                mc[m, argmax[n, m]] += 1
                nc[m, argmin[n, m]] += 1
        return mc, nc
    for arg in (argmax, argmin):
        cells = {(m, int(arg[n, m])) for n in range(N) for m in range(M)}
        for (m, k) in cells:
            mc[m, k] += 1
    return mc, nc
