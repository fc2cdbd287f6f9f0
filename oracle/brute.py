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
            # NaN products take no part (the reference kernel compares with ordered > and <).  Among the
            # rest the extreme is the largest / smallest value and its index the lowest k that holds it;
            # an extreme that does not rise above -inf (fall below +inf) -- no candidates at all, or only
            # that infinity -- keeps the scan's starting index 0.
            real = [(k, p) for k, p in enumerate(prods) if p == p]
            hi = max([p for _, p in real], default=f32(-np.inf))
            lo = min([p for _, p in real], default=f32(np.inf))
            ih = min([k for k, p in real if p == hi], default=0) if hi > -np.inf else 0
            il = min([k for k, p in real if p == lo], default=0) if lo < np.inf else 0
            # a zero extreme carries the sign of the FIRST zero product
            if hi == 0:
                hi = prods[ih]
            if lo == 0:
                lo = prods[il]
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


def conv_forward(x, w, stride=(1, 1), bias=None):
    """MAM convolution by its scalar definition.  x (B, C, H, W), w (F, C, k1, k2), no padding ->
    y, argmax, argmin of shape (B, F, L1, L2).  Products are scanned in ascending
    q = (j2 * k1 + j1) * C + c (window column outermost, then window row, channel innermost) with strict
    comparisons, the order in which the reference's kernels walk a window
    (mamtorch/kernel/backup/mamconv1d_forward.txt:74-139: blocks of k over position * C + channel;
    index decoding in mamtorch/nn/backup/mamconv2d.txt:97-103).  A 1-D convolution is H = k1 = 1."""
    x = np.asarray(x, f32)
    w = np.asarray(w, f32)
    B, C, H, W = x.shape
    Fo, _, k1, k2 = w.shape
    s1, s2 = stride
    L1, L2 = (H - k1) // s1 + 1, (W - k2) // s2 + 1
    y = np.zeros((B, Fo, L1, L2), f32)
    amax = np.zeros((B, Fo, L1, L2), np.int32)
    amin = np.zeros((B, Fo, L1, L2), np.int32)
    for b in range(B):
        for f in range(Fo):
            for l1 in range(L1):
                for l2 in range(L2):
                    hi = lo = None
                    ih = il = 0
                    for j2 in range(k2):
                        for j1 in range(k1):
                            for c in range(C):
                                q = (j2 * k1 + j1) * C + c
                                p = f32(x[b, c, l1 * s1 + j1, l2 * s2 + j2]) * f32(w[f, c, j1, j2])
                                if hi is None or p > hi:
                                    hi, ih = p, q
                                if lo is None or p < lo:
                                    lo, il = p, q
                    s = f32(hi + lo)
                    if bias is not None:
                        s = f32(s + f32(bias[f]))
                    y[b, f, l1, l2], amax[b, f, l1, l2], amin[b, f, l1, l2] = s, ih, il
    return y, amax, amin


def conv_backward(x, w, grad, argmax, argmin, stride=(1, 1)):
    """-> x_grad like x, w_grad like w (fp64 accumulation of fp32 terms): the gradient goes to the two
    selected (input, weight) pairs of every output position, twice when they coincide
    (mamtorch/kernel/backup/mamconv1d_backward.txt)."""
    x = np.asarray(x, f32)
    w = np.asarray(w, f32)
    grad = np.asarray(grad, f32)
    B, C, H, W = x.shape
    Fo, _, k1, k2 = w.shape
    s1, s2 = stride
    xg = np.zeros(x.shape, np.float64)
    wg = np.zeros(w.shape, np.float64)
    _, _, L1, L2 = grad.shape
    for b in range(B):
        for f in range(Fo):
            for l1 in range(L1):
                for l2 in range(L2):
                    g = grad[b, f, l1, l2]
                    for q in (int(argmax[b, f, l1, l2]), int(argmin[b, f, l1, l2])):
                        c, pos = q % C, q // C
                        j1, j2 = pos % k1, pos // k1
                        h, ww = l1 * s1 + j1, l2 * s2 + j2
                        xg[b, c, h, ww] += float(f32(w[f, c, j1, j2]) * g)
                        wg[f, c, j1, j2] += float(f32(x[b, c, h, ww]) * g)
    return xg.astype(f32), wg.astype(f32)
