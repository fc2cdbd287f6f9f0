"""CPU oracle for the MAM fully-connected hot path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package, and only as the checker.  The shipped package never imports it.

Three independent statements of the same algorithm live here:
  * ``mam_oracle.c``   -- plain C triple loops (ctypes wrappers below); fast enough for
                          the medium-size parity cases.
  * ``torch_port.py``  -- pure-PyTorch, batch-chunked restatement of the reference's
                          test/reference.py:3-25; it is the CPU baseline timed by bench.py.
  * ``brute.py``       -- pure-Python loops over numpy float32 scalars for tiny inputs;
                          it pins the other two.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmam_oracle.so")
_lib = None

W_KM = 0  # w is (K, M): the operator's ``b`` operand
W_MK = 1  # w is (M, K): the module's ``weight`` (out, in)


def build(force=False):
    """Compile mam_oracle.c with gcc (oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libmam_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def _i64(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int64))


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


_I64 = ctypes.c_int64


def forward(x, w, layout=W_KM, bias=None):
    """Returns (c, argmax, argmin) as numpy arrays; x (N,K), w (K,M) or (M,K)."""
    x, w = _f32(x), _f32(w)
    N, K = x.shape
    M = w.shape[1] if layout == W_KM else w.shape[0]
    assert (w.shape[0] if layout == W_KM else w.shape[1]) == K
    b = None if bias is None else _f32(bias)
    c = np.empty((N, M), np.float32)
    amax = np.empty((N, M), np.int32)
    amin = np.empty((N, M), np.int32)
    lib().mam_oracle_forward(_p(x), _I64(K), _p(w), _I64(w.shape[1]), ctypes.c_int(layout), _p(b),
                             _p(c), _p(amax), _p(amin), _I64(N), _I64(K), _I64(M))
    return c, amax, amin


def backward(x, w, grad, argmax, argmin, layout=W_KM):
    """Returns (x_grad (N,K), w_grad in the layout of w)."""
    x, w, grad = _f32(x), _f32(w), _f32(grad)
    argmax, argmin = _i32(argmax), _i32(argmin)
    N, K = x.shape
    M = grad.shape[1]
    xg = np.empty((N, K), np.float32)
    wg = np.empty(w.shape, np.float32)
    lib().mam_oracle_backward(_p(x), _I64(K), _p(w), _I64(w.shape[1]), ctypes.c_int(layout), _p(grad),
                              _p(argmax), _p(argmin), _p(xg), _p(wg), _I64(N), _I64(K), _I64(M))
    return xg, wg


def selection_count(argmax, argmin, max_count, min_count, mode=0):
    """Adds to copies of the (M,K) int32 counters and returns them."""
    argmax, argmin = _i32(argmax), _i32(argmin)
    mc, nc = _i32(max_count).copy(), _i32(min_count).copy()
    N, M = argmax.shape
    K = mc.shape[1]
    lib().mam_oracle_selection_count(_p(argmax), _p(argmin), _p(mc), _p(nc), _I64(N), _I64(M), _I64(K),
                                     ctypes.c_int(mode))
    return mc, nc


def csr_forward(x, crow, col, val, K, bias=None):
    x, val = _f32(x), _f32(val)
    crow, col = _i64(crow), _i64(col)
    N = x.shape[0]
    M = crow.shape[0] - 1
    b = None if bias is None else _f32(bias)
    c = np.empty((N, M), np.float32)
    amax = np.empty((N, M), np.int32)
    amin = np.empty((N, M), np.int32)
    lib().mam_oracle_csr_forward(_p(x), _I64(K), _p(crow), _p(col), _p(val), _p(b), _p(c), _p(amax),
                                 _p(amin), _I64(N), _I64(K), _I64(M))
    return c, amax, amin


def csr_backward(x, crow, col, val, grad, argmax, argmin):
    x, val, grad = _f32(x), _f32(val), _f32(grad)
    crow, col = _i64(crow), _i64(col)
    argmax, argmin = _i32(argmax), _i32(argmin)
    N, K = x.shape
    M = crow.shape[0] - 1
    xg = np.empty((N, K), np.float32)
    vg = np.empty(val.shape, np.float32)
    lib().mam_oracle_csr_backward(_p(x), _I64(K), _p(crow), _p(col), _p(val), _p(grad), _p(argmax),
                                  _p(argmin), _p(xg), _p(vg), _I64(N), _I64(K), _I64(M))
    return xg, vg


def coo_spmm(row, col, val, b, R):
    """(c, abs_sum) for c = A @ b with A given as COO triples (any order, duplicates add up); fp64
    accumulation.  abs_sum[r, j] = sum of |val * b| of the cell: the scale of its rounding floor."""
    row, col, val = _i64(row), _i64(col), _f32(val)
    b = _f32(b)
    K, C = b.shape
    c = np.empty((R, C), np.float32)
    ab = np.empty((R, C), np.float32)
    lib().mam_oracle_coo_spmm(_p(row), _p(col), _p(val), _I64(val.shape[0]), _p(b), _I64(C), _p(c), _p(ab),
                              _I64(R), _I64(C))
    return c, ab


def csr_spmm(crow, col, val, b):
    """(c, abs_sum) for c = A @ b with A in CSR (int64 crow / col)."""
    crow = _i64(crow)
    R = crow.shape[0] - 1
    row = np.repeat(np.arange(R, dtype=np.int64), np.diff(crow))
    return coo_spmm(row, col, val, b, R)


def conv_windows(x, k1, k2, s1, s2):
    """x (B, C, H, W) -> the (B * L1 * L2, k2 * k1 * C) matrix of windows, column
    q = (j2 * k1 + j1) * C + c, built by plain numpy slicing (one slice per window position): the operand on
    which forward() gives the MAM convolution of brute.conv_forward at sizes the pure-Python loops cannot
    reach.  Pinned against brute.conv_forward in tests/test_oracle.py."""
    x = np.asarray(x, dtype=np.float32)
    B, C, H, W = x.shape
    L1, L2 = (H - k1) // s1 + 1, (W - k2) // s2 + 1
    cols = np.empty((B, L1, L2, k2, k1, C), dtype=np.float32)
    for j2 in range(k2):
        for j1 in range(k1):
            # x[b, c, l1 * s1 + j1, l2 * s2 + j2] for all (b, c, l1, l2)
            win = x[:, :, j1:j1 + (L1 - 1) * s1 + 1:s1, j2:j2 + (L2 - 1) * s2 + 1:s2]
            cols[:, :, :, j2, j1, :] = win.transpose(0, 2, 3, 1)
    return cols.reshape(B * L1 * L2, k2 * k1 * C)


def conv_forward(x, w, stride=(1, 1), bias=None):
    """MAM convolution through conv_windows + forward(): y, argmax, argmin of shape (B, F, L1, L2)."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    B, C, H, W = x.shape
    Fo, _, k1, k2 = w.shape
    s1, s2 = stride
    L1, L2 = (H - k1) // s1 + 1, (W - k2) // s2 + 1
    wm = np.ascontiguousarray(w.transpose(0, 3, 2, 1).reshape(Fo, k2 * k1 * C))
    c, amax, amin = forward(conv_windows(x, k1, k2, s1, s2), wm, W_MK, bias)
    shape = (B, L1, L2, Fo)
    return tuple(np.ascontiguousarray(t.reshape(shape).transpose(0, 3, 1, 2)) for t in (c, amax, amin))
