"""Loads the native libraries of the MAM hot path and fails loudly when they are missing.

``libmam_hip.so``    -- HIP kernels for gfx950 behind a C ABI (include/mam_hip.h).
``mam_torch_ops.so`` -- torch.ops registration (mamtorch_kernel_v1 / _v4 / _sparsev1) over that ABI.

There is no CPU or eager-PyTorch fallback: if a library is absent the import raises, and the
operators exist for GPU tensors only.
"""
import ctypes
import os

import torch

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
HIP_LIB_PATH = os.path.join(_LIB_DIR, "libmam_hip.so")
OPS_LIB_PATH = os.path.join(_LIB_DIR, "mam_torch_ops.so")

_hip = None
_ops_loaded = False


def _require(path):
    if not os.path.exists(path):
        raise ImportError(
            "%s is not built; run `python -m mamtorch_amd.build` (needs hipcc, targets gfx950)" % path)


def hip_library():
    """ctypes handle of libmam_hip.so."""
    global _hip
    if _hip is None:
        _require(HIP_LIB_PATH)
        _hip = ctypes.CDLL(HIP_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    return _hip


def load_ops():
    """Registers the torch.ops namespaces (idempotent)."""
    global _ops_loaded
    if not _ops_loaded:
        hip_library()
        _require(OPS_LIB_PATH)
        torch.ops.load_library(OPS_LIB_PATH)
        _ops_loaded = True
