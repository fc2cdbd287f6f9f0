"""The C ABI of libmam_hip.so (include/mam_hip.h) through ctypes, for torch GPU tensors.

Thin argument marshalling only: device pointers come from ``Tensor.data_ptr()``, the stream from
``torch.cuda.current_stream()``, outputs and workspace from torch's allocator.  This is the path
the GPU parity tests drive, and what a non-PyTorch host would bind.
"""
import ctypes

import torch

from . import _native

W_KM = 0
W_MK = 1
PRUNE_MAGNITUDE = 0
PRUNE_WEIGHT_TIMES = 1
PRUNE_COUNT = 2
OPT_FORWARD_TILING = 0
OPT_BACKWARD_FORK = 1
OPT_BACKWARD_ONE_LAUNCH = 2
OPT_BACKWARD_EXACT = 3
FORWARD_TILING_AUTO = 0
FORWARD_TILING_WIDE = 1
FORWARD_TILING_GROUPS16 = 2
BACKWARD_FORK_AUTO = -1
COUNT_REFERENCE = 0
COUNT_HITS = 1
COUNT_FLAGS = 2

EXPORTS = (
    "mam_version", "mam_error_string", "mam_last_error", "mam_init", "mam_set_option", "mam_device_info",
    "mam_fc_forward_static_limit", "mam_fc_forward_static", "mam_fc_forward_describe",
    "mam_fc_forward_workspace", "mam_fc_forward_workspace_for", "mam_fc_forward",
    "mam_fc_forward_values_workspace", "mam_fc_forward_values",
    "mam_fc_backward", "mam_fc_backward_count", "mam_selection_count",
    "mam_fc_forward_ranges_workspace", "mam_fc_forward_ranges", "mam_fc_backward_ranges",
    "mam_csr_fc_forward_workspace", "mam_csr_fc_forward", "mam_csr_fc_backward", "mam_csr_validate",
    "mam_csr_spmm", "mam_coo_spmm", "mam_csr_to_dense", "mam_coo_to_dense",
    "mam_blend", "mam_bias_grad_workspace", "mam_bias_grad", "mam_apply_keep", "mam_im2col", "mam_col2im",
    "mam_prune_row_offsets", "mam_prune_fill_csr", "mam_prune_apply",
    "mam_select_workspace", "mam_select_begin", "mam_select_accumulate", "mam_select_advance", "mam_select_result",
)

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_size = ctypes.c_size_t
_configured = False


def lib():
    global _configured
    l = _native.hip_library()
    if not _configured:
        l.mam_error_string.restype = ctypes.c_char_p
        l.mam_error_string.argtypes = [_int]
        l.mam_last_error.restype = ctypes.c_char_p
        for name in ("mam_fc_forward_workspace", "mam_fc_forward_values_workspace",
                     "mam_csr_fc_forward_workspace"):
            fn = getattr(l, name)
            fn.restype = _size
            fn.argtypes = [_i64, _i64, _i64]
        l.mam_fc_forward_workspace_for.restype = _size
        l.mam_fc_forward_workspace_for.argtypes = [_i64, _i64, _i64, _int, _int]
        l.mam_fc_forward.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64,
                                     _i64, _i64, _ptr, _size, _ptr]
        l.mam_fc_forward_static_limit.restype = _size
        l.mam_fc_forward_static_limit.argtypes = []
        l.mam_fc_forward_static.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64,
                                            _i64, _i64, _ptr]
        l.mam_set_option.argtypes = [_int, _int]
        l.mam_fc_forward_describe.argtypes = [_ptr, _i64, _ptr, _i64, _int, _i64, _i64, _i64, _int, ctypes.c_char_p,
                                              _size]
        l.mam_fc_forward_values.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _i64, _i64, _i64,
                                            _ptr, _size, _ptr]
        l.mam_fc_backward.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                      _i64, _i64, _i64, _ptr]
        l.mam_fc_forward_ranges_workspace.restype = _size
        l.mam_fc_forward_ranges_workspace.argtypes = [_i64, _i64, _i64, _i64, _int]
        l.mam_fc_forward_ranges.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64,
                                            _i64, _ptr, _size, _ptr]
        l.mam_fc_backward_count.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                            _ptr, _int, _i64, _i64, _i64, _ptr]
        l.mam_fc_backward_ranges.argtypes = [_ptr, _i64, _ptr, _i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64,
                                             _i64, _i64, _ptr]
        l.mam_selection_count.argtypes = [_ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _int, _ptr]
        l.mam_csr_fc_forward.argtypes = [_ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                         _i64, _i64, _i64, _i64, _ptr, _size, _ptr]
        l.mam_csr_fc_backward.argtypes = [_ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                          _ptr, _ptr, _i64, _i64, _i64, _i64, _ptr]
        l.mam_blend.argtypes = [_ptr, _ptr, _ptr, ctypes.c_float, ctypes.c_float, _ptr, _i64, _i64, _ptr]
        l.mam_apply_keep.argtypes = [_ptr, _i64, _ptr, _ptr, _i64, _i64, _ptr]
        l.mam_im2col.argtypes = [_ptr, _ptr] + [_i64] * 8 + [_ptr]
        l.mam_col2im.argtypes = [_ptr, _ptr] + [_i64] * 8 + [_ptr]
        l.mam_csr_validate.argtypes = [_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr]
        l.mam_csr_spmm.argtypes = [_ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _i64, _i64, _ptr]
        l.mam_coo_spmm.argtypes = [_ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i64, _i64, _i64, _ptr]
        l.mam_csr_to_dense.argtypes = [_ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr]
        l.mam_coo_to_dense.argtypes = [_ptr, _ptr, _ptr, _i64, _ptr, _i64, _i64, _i64, _ptr]
        _f = ctypes.c_float
        l.mam_prune_row_offsets.argtypes = [_ptr, _i64, _int, _ptr, _ptr, _i64, _f, _ptr, _i64, _i64, _ptr]
        l.mam_prune_fill_csr.argtypes = [_ptr, _i64, _int, _ptr, _ptr, _i64, _f, _ptr, _ptr, _ptr, _i64, _i64, _ptr]
        l.mam_prune_apply.argtypes = [_ptr, _i64, _int, _ptr, _ptr, _i64, _f, _i64, _i64, _ptr]
        _configured = True
    return l


class MamError(RuntimeError):
    def __init__(self, code):
        self.code = code
        l = lib()
        super().__init__("%s (%s)" % (l.mam_error_string(code).decode(), l.mam_last_error().decode()))


def _check(rc):
    if rc != 0:
        raise MamError(rc)


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dims(x, w, layout):
    N, K = x.shape
    M = w.shape[0] if layout == W_MK else w.shape[1]
    return N, K, M


def _ld(t):
    return t.stride(0) if t.size(0) > 1 else max(t.size(1), 1)


def fc_forward(x, w, layout=W_KM, bias=None, workspace=None, w_sel=None, x_sel=None):
    """-> (c, argmax, argmin) on x.device.  ``workspace`` (uint8 tensor) is allocated if None.
    ``w_sel`` / ``x_sel``: optional (2, N, M) fp32 tensors that receive the selected weights / inputs."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    c = torch.empty((N, M), dtype=torch.float32, device=x.device)
    amax = torch.empty((N, M), dtype=torch.int32, device=x.device)
    amin = torch.empty((N, M), dtype=torch.int32, device=x.device)
    need = l.mam_fc_forward_workspace_for(N, K, M, layout, 1)
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _check(l.mam_fc_forward(_p(x), _ld(x), _p(w), _ld(w), layout, _p(bias), _p(c), _p(amax), _p(amin),
                                _p(w_sel), _p(x_sel), N, K, M, _p(workspace), 0 if workspace is None else workspace.numel(),
                                _stream(x)))
    return c, amax, amin


def fc_forward_static(x, w, c, argmax, argmin, layout=W_KM, bias=None, w_sel=None, x_sel=None):
    """mam_fc_forward_static into caller-provided outputs: nothing is allocated anywhere on the way (the
    split-K partials live in the library's file-scope device array)."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    with torch.cuda.device(x.device):
        _check(l.mam_fc_forward_static(_p(x), _ld(x), _p(w), _ld(w), layout, _p(bias), _p(c), _p(argmax), _p(argmin),
                                       _p(w_sel), _p(x_sel), N, K, M, _stream(x)))


def set_option(option, value):
    _check(lib().mam_set_option(option, value))


def fc_forward_describe(x, w, layout=W_KM, with_indices=True):
    """Text naming the kernels and the tiling that mam_fc_forward would launch for these operands."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    buf = ctypes.create_string_buffer(320)
    _check(l.mam_fc_forward_describe(_p(x), _ld(x), _p(w), _ld(w), layout, N, K, M, 1 if with_indices else 0, buf, 320))
    return buf.value.decode()


def fc_forward_values(x, w, layout=W_KM, bias=None, workspace=None):
    l = lib()
    N, K, M = _dims(x, w, layout)
    c = torch.empty((N, M), dtype=torch.float32, device=x.device)
    need = l.mam_fc_forward_workspace_for(N, K, M, layout, 0)
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _check(l.mam_fc_forward_values(_p(x), _ld(x), _p(w), _ld(w), layout, _p(bias), _p(c), N, K, M,
                                       _p(workspace), 0 if workspace is None else workspace.numel(),
                                       _stream(x)))
    return c


def fc_backward(x, w, grad, argmax, argmin, layout=W_KM, want_x=True, want_w=True, w_sel=None, x_sel=None):
    """-> (x_grad or None, w_grad or None); w_grad has the shape and layout of w."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    xg = torch.empty((N, K), dtype=torch.float32, device=x.device) if want_x else None
    wg = torch.empty(tuple(w.shape), dtype=torch.float32, device=x.device) if want_w else None
    with torch.cuda.device(x.device):
        _check(l.mam_fc_backward(_p(x), _ld(x), _p(w), _ld(w), layout, _p(grad), _p(argmax), _p(argmin),
                                 _p(w_sel), _p(x_sel), _p(xg), _p(wg), N, K, M, _stream(x)))
    return xg, wg


def fc_backward_count(x, w, grad, argmax, argmin, max_count, min_count, mode=COUNT_HITS, layout=W_KM, want_x=True,
                      want_w=True, w_sel=None, x_sel=None):
    """fc_backward and selection_count (in place on the (M, K) int32 counters) as one call."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    xg = torch.empty((N, K), dtype=torch.float32, device=x.device) if want_x else None
    wg = torch.empty(tuple(w.shape), dtype=torch.float32, device=x.device) if want_w else None
    with torch.cuda.device(x.device):
        _check(l.mam_fc_backward_count(_p(x), _ld(x), _p(w), _ld(w), layout, _p(grad), _p(argmax), _p(argmin),
                                       _p(w_sel), _p(x_sel), _p(xg), _p(wg), _p(max_count), _p(min_count), mode,
                                       N, K, M, _stream(x)))
    return xg, wg


def fc_forward_ranges(x, w, range_len, layout=W_KM, bias=None, with_indices=True):
    """-> (c, argmax, argmin) with argmax / argmin of shape (ranges, N, M) holding absolute k (None, None
    when with_indices is false): the module's `splits` as one call."""
    l = lib()
    N, K, M = _dims(x, w, layout)
    ranges = max(1, -(-K // range_len))
    c = torch.empty((N, M), dtype=torch.float32, device=x.device)
    amax = torch.empty((ranges, N, M), dtype=torch.int32, device=x.device) if with_indices else None
    amin = torch.empty((ranges, N, M), dtype=torch.int32, device=x.device) if with_indices else None
    need = l.mam_fc_forward_ranges_workspace(N, K, M, range_len, int(with_indices))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _check(l.mam_fc_forward_ranges(_p(x), _ld(x), _p(w), _ld(w), layout, _p(bias), _p(c), _p(amax), _p(amin),
                                       N, K, M, range_len, _p(ws), need, _stream(x)))
    return c, amax, amin


def fc_backward_ranges(x, w, grad, argmax, argmin, range_len, layout=W_KM, want_x=True, want_w=True):
    l = lib()
    N, K, M = _dims(x, w, layout)
    xg = torch.empty((N, K), dtype=torch.float32, device=x.device) if want_x else None
    wg = torch.empty(tuple(w.shape), dtype=torch.float32, device=x.device) if want_w else None
    with torch.cuda.device(x.device):
        _check(l.mam_fc_backward_ranges(_p(x), _ld(x), _p(w), _ld(w), layout, _p(grad), _p(argmax), _p(argmin),
                                        _p(xg), _p(wg), N, K, M, range_len, _stream(x)))
    return xg, wg


def selection_count(argmax, argmin, max_count, min_count, mode=COUNT_REFERENCE):
    """In place on the (M, K) int32 counters."""
    l = lib()
    N, M = argmax.shape
    K = max_count.shape[1]
    with torch.cuda.device(argmax.device):
        _check(l.mam_selection_count(_p(argmax), _p(argmin), _p(max_count), _p(min_count), N, M, K, mode,
                                     _stream(argmax)))


def csr_fc_forward(x, crow, col, val, M, bias=None, w_sel=None, pos_sel=None, x_sel=None):
    """Returns (c, argmax, argmin); fills the optional (2,N,M) hand-over arrays for the backward."""
    l = lib()
    N, K = x.shape
    c = torch.empty((N, M), dtype=torch.float32, device=x.device)
    amax = torch.empty((N, M), dtype=torch.int32, device=x.device)
    amin = torch.empty((N, M), dtype=torch.int32, device=x.device)
    need = l.mam_csr_fc_forward_workspace(N, K, M)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _check(l.mam_csr_fc_forward(_p(x), _ld(x), _p(crow), _p(col), _p(val), _p(bias), _p(c), _p(amax),
                                    _p(amin), _p(w_sel), _p(pos_sel), _p(x_sel), N, K, M, val.numel(), _p(ws), need,
                                    _stream(x)))
    return c, amax, amin


def csr_validate(crow, col, K):
    """0 when the CSR parts satisfy what the sparse kernels assume, else a mask of violations
    (1 row-offset ends, 2 row offsets decreasing, 4 column out of range, 8 columns not ascending in a row).
    Synchronises to read the verdict back."""
    l = lib()
    M = crow.numel() - 1
    status = torch.zeros(1, dtype=torch.int32, device=crow.device)
    with torch.cuda.device(crow.device):
        _check(l.mam_csr_validate(_p(crow), _p(col), M, K, col.numel(), _p(status), _stream(crow)))
    return int(status.item())


def csr_fc_backward(x, crow, col, val, grad, argmax, argmin, w_sel=None, pos_sel=None, x_sel=None):
    l = lib()
    N, K = x.shape
    M = crow.numel() - 1
    xg = torch.empty((N, K), dtype=torch.float32, device=x.device)
    vg = torch.empty_like(val)
    with torch.cuda.device(x.device):
        _check(l.mam_csr_fc_backward(_p(x), _ld(x), _p(crow), _p(col), _p(val), _p(grad), _p(argmax),
                                     _p(argmin), _p(w_sel), _p(pos_sel), _p(x_sel), _p(xg), _p(vg), N, K, M, val.numel(),
                                     _stream(x)))
    return xg, vg


def csr_spmm(crow, col, val, b, R):
    """c (R, C) = A (R, K) in CSR @ b (K, C) dense (rows may be strided)."""
    l = lib()
    K, C = b.shape
    c = torch.empty((R, C), dtype=torch.float32, device=b.device)
    with torch.cuda.device(b.device):
        _check(l.mam_csr_spmm(_p(crow), _p(col), _p(val), _p(b), _ld(b), _p(c), R, K, C, _stream(b)))
    return c


def coo_spmm(row, col, val, b, R):
    """c (R, C) = A (R, K) in COO (any order, duplicates add up) @ b (K, C) dense."""
    l = lib()
    K, C = b.shape
    c = torch.empty((R, C), dtype=torch.float32, device=b.device)
    with torch.cuda.device(b.device):
        _check(l.mam_coo_spmm(_p(row), _p(col), _p(val), val.numel(), _p(b), _ld(b), _p(c), R, K, C, _stream(b)))
    return c


def csr_to_dense(crow, col, val, R, K):
    """(R, K) dense fp32 matrix of a CSR operand (repeated coordinates add up)."""
    l = lib()
    dense = torch.empty((R, K), dtype=torch.float32, device=val.device)
    with torch.cuda.device(val.device):
        _check(l.mam_csr_to_dense(_p(crow), _p(col), _p(val), _p(dense), K, R, K, _stream(val)))
    return dense


def coo_to_dense(row, col, val, R, K):
    l = lib()
    dense = torch.empty((R, K), dtype=torch.float32, device=val.device)
    with torch.cuda.device(val.device):
        _check(l.mam_coo_to_dense(_p(row), _p(col), _p(val), val.numel(), _p(dense), K, R, K, _stream(val)))
    return dense


def _prune_operands(w, mode, aux, aux2):
    if mode == PRUNE_MAGNITUDE:
        return None, None, max(w.size(1), 1)
    want = torch.float32 if mode == PRUNE_WEIGHT_TIMES else torch.int32
    for t in (aux, aux2):
        if t is not None and (t.dtype != want or t.shape != w.shape or t.device != w.device or t.stride(1) != 1):
            raise ValueError("score operand must be a %s tensor shaped and placed like the weight" % want)
    if aux is None or (aux2 is not None and (mode != PRUNE_COUNT or _ld(aux2) != _ld(aux))):
        raise ValueError("score operand missing or second operand not allowed")
    return aux, aux2, _ld(aux)


def prune_to_csr(w, threshold, mode=PRUNE_MAGNITUDE, aux=None, aux2=None):
    """CSR parts (crow, col, val) of the entries of w (M, K) whose score is above `threshold`.
    Reads crow[M] back to size col / val: the only host synchronisation."""
    l = lib()
    M, K = w.shape
    aux, aux2, ld_aux = _prune_operands(w, mode, aux, aux2)
    crow = torch.empty(M + 1, dtype=torch.int64, device=w.device)
    with torch.cuda.device(w.device):
        _check(l.mam_prune_row_offsets(_p(w), _ld(w), mode, _p(aux), _p(aux2), ld_aux, threshold, _p(crow), M, K,
                                       _stream(w)))
        nnz = int(crow[M].item())
        col = torch.empty(nnz, dtype=torch.int64, device=w.device)
        val = torch.empty(nnz, dtype=torch.float32, device=w.device)
        _check(l.mam_prune_fill_csr(_p(w), _ld(w), mode, _p(aux), _p(aux2), ld_aux, threshold, _p(crow), _p(col),
                                    _p(val), M, K, _stream(w)))
    return crow, col, val


def select_abs_ranks(operands, ranks):
    """The elements of the given 0-based `ranks` (one or two, ascending) among the absolute scores of all
    `operands`, each (w, mode, aux, aux2) as for prune_apply (w (M, K) fp32 with contiguous rows): what a
    full ascending sort of the concatenated |scores| would hold there.  Returns a DEVICE float tensor with
    one element per rank (reading it is the caller's synchronisation)."""
    l = lib()
    l.mam_select_workspace.restype = _size
    first = operands[0][0]
    dev = first.device
    nbytes = l.mam_select_workspace()
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    out = torch.empty(len(ranks), dtype=torch.float32, device=dev)
    rk = (ctypes.c_int64 * len(ranks))(*[int(r) for r in ranks])
    mode0 = operands[0][1]
    with torch.cuda.device(dev):
        st = _stream(first)
        _check(l.mam_select_begin(_p(ws), _size(nbytes), rk, len(ranks), st))
        for ps in range(3):
            for w, mode, aux, aux2 in operands:
                if mode != mode0:
                    raise ValueError("all operands of one selection must use the same score")
                M, K = w.shape
                aux, aux2, ld_aux = _prune_operands(w, mode, aux, aux2)
                _check(l.mam_select_accumulate(_p(ws), _p(w), _i64(_ld(w)), mode, _p(aux), _p(aux2), _i64(ld_aux),
                                               _i64(M), _i64(K), ps, st))
            _check(l.mam_select_advance(_p(ws), ps, st))
        _check(l.mam_select_result(_p(ws), mode0, _p(out), st))
    return out


def prune_apply(w, threshold, mode=PRUNE_MAGNITUDE, aux=None, aux2=None):
    """In place: entries of w whose score is not above `threshold` become 0."""
    l = lib()
    M, K = w.shape
    aux, aux2, ld_aux = _prune_operands(w, mode, aux, aux2)
    with torch.cuda.device(w.device):
        _check(l.mam_prune_apply(_p(w), _ld(w), mode, _p(aux), _p(aux2), ld_aux, threshold, M, K, _stream(w)))
    return w
