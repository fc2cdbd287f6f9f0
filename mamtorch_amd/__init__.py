"""MI355X-native Multiply-And-Max/min (MAM) fully-connected hot path.

Mirrors the interface of SSIGPRO/mamtorch for this path (mamtorch/__init__.py:1-3):
``kernel`` (operator wrappers), ``nn`` (FullyConnected), ``sparse`` (CSR-sparse MAM), plus
``capi`` (the C ABI through ctypes).
"""
import sys

from . import _native

# `python -m mamtorch_amd.build` imports this package on its way to the build module: it must work
# before the libraries exist and while they are stale, so nothing native is loaded for it.
if "mamtorch_amd.build" not in getattr(sys, "orig_argv", []):
    _native.load_ops()

    from . import kernel  # noqa: E402
    from . import nn  # noqa: E402
    from . import sparse  # noqa: E402
    from . import capi  # noqa: E402
    from .nn.legacy import MAMDense  # noqa: E402  (mamtorch/__init__.py:7: backwards compatibility)

__version__ = "0.1.0"
