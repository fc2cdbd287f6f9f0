"""CPU oracle of the pruning rule and the dense -> CSR compaction -- TEST INFRASTRUCTURE ONLY.

Restates examples/vitb16_imagenet1k/pruning_utils.py:103-111 (magnitude), :190-203 (weight x gradient):
``w[score.abs() <= threshold] = 0``; with selection counts (mamtorch/nn/v4/fullyconnected.py:107-131) as the
third score.  A NaN score compares false and is therefore kept, as by the reference's masked assignment.
Pinned in tests/test_oracle.py against the literal torch statement of the rule followed by
``Tensor.to_sparse_csr()`` and against a hand-derived case.
"""
import numpy as np

MAGNITUDE, WEIGHT_TIMES, COUNT = 0, 1, 2


def keep_mask(w, threshold, mode=MAGNITUDE, aux=None, aux2=None):
    w = np.asarray(w, dtype=np.float32)
    if mode == MAGNITUDE:
        score = np.abs(w)
    elif mode == WEIGHT_TIMES:
        score = np.abs(w * np.asarray(aux, dtype=np.float32))     # one fp32 multiply, as on the device
    else:
        cnt = np.asarray(aux, dtype=np.int32)
        if aux2 is not None:
            cnt = cnt + np.asarray(aux2, dtype=np.int32)
        score = cnt.astype(np.float32)
    with np.errstate(invalid="ignore"):
        return ~(score <= np.float32(threshold))


def apply(w, threshold, mode=MAGNITUDE, aux=None, aux2=None):
    out = np.array(w, dtype=np.float32, copy=True)
    out[~keep_mask(w, threshold, mode, aux, aux2)] = 0.0
    return out


def to_csr(w, threshold, mode=MAGNITUDE, aux=None, aux2=None):
    """(crow int64 (M+1), col int64 (nnz) ascending per row, val fp32 (nnz)) of the kept entries."""
    w = np.asarray(w, dtype=np.float32)
    keep = keep_mask(w, threshold, mode, aux, aux2)
    crow = np.zeros(w.shape[0] + 1, dtype=np.int64)
    crow[1:] = np.cumsum(keep.sum(axis=1))
    rows, cols = np.nonzero(keep)           # row-major order: ascending columns within a row
    return crow, cols.astype(np.int64), w[rows, cols]
