"""``import mamtorch`` -- the import name of SSIGPRO/mamtorch, served by the MI355X-native build.

Every module path the reference's callers use resolves onto the corresponding module of ``mamtorch_amd``
(the same module objects, registered under both names), so ``import mamtorch`` followed by the
reference's own call patterns -- ``mamtorch.nn.FullyConnected``, ``mamtorch.kernel.v4.fullyconnected``,
``torch.ops.mamtorch_kernel_v1.fullyconnected``, ``mamtorch.MAMDense`` -- runs on the HIP kernels:

    mamtorch.kernel, .kernel.v1, .kernel.v1.fullyconnected,
    .kernel.v4, .kernel.v4.fullyconnected, .kernel.v4.fullyconnected_fast      (mamtorch/kernel/__init__.py:1-4)
    mamtorch.nn, .nn.v1, .nn.v1.fullyconnected, .nn.v4, .nn.v4.fullyconnected,
    .nn.compat                                                                  (mamtorch/nn/__init__.py:1-6)
    mamtorch.sparse, .sparse.kernel, .sparse.kernel.v1, .sparse.kernel.v1.cusparsemm
    mamtorch.MAMDense (star-import of nn.compat)                                (mamtorch/__init__.py:1-7)

The reference's v2 / v3 generations are not importable upstream either (commented out there).
"""
import importlib
import sys

import mamtorch_amd as _impl

_PATHS = (
    "kernel", "kernel.v1", "kernel.v1.fullyconnected", "kernel.v4", "kernel.v4.fullyconnected",
    "kernel.v4.fullyconnected_fast",
    "nn", "nn.compat", "nn.v1", "nn.v1.fullyconnected", "nn.v4", "nn.v4.fullyconnected",
    "sparse", "sparse.kernel", "sparse.kernel.v1", "sparse.kernel.v1.cusparsemm",
)
for _path in _PATHS:
    sys.modules[__name__ + "." + _path] = importlib.import_module("mamtorch_amd." + _path)
del _path

kernel = sys.modules[__name__ + ".kernel"]
nn = sys.modules[__name__ + ".nn"]
sparse = sys.modules[__name__ + ".sparse"]
capi = _impl.capi

# backwards compatibility (mamtorch/__init__.py:5-7)
from mamtorch_amd.nn.compat import *  # noqa: E402,F401,F403

__version__ = _impl.__version__
