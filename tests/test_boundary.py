"""CPU-only checks of the drop-in boundary: the C ABI library loads and exports every symbol that
include/mam_hip.h declares, the torch operator schemas equal the reference's strings, fake
kernels propagate shapes, the module's host logic follows the reference, and nothing falls
back to a CPU implementation."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import mamtorch_amd as mt
from mamtorch_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mam_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mam_[a-z_0-9]+)\s*\(", text)))


def test_c_abi_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 12
    assert set(names) == set(capi.EXPORTS)
    lib = ctypes.CDLL(mt._native.HIP_LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libmam_hip.so does not export %s" % n
    assert lib.mam_version() >= 100
    capi.lib()
    assert capi.lib().mam_error_string(-3).decode() == "workspace missing or too small"


def test_workspace_queries_are_pure_host_calls():
    l = capi.lib()
    assert l.mam_fc_forward_workspace(12608, 768, 3072) == 0          # enough tiles: no split-K
    ws = l.mam_fc_forward_workspace(256, 4096, 4096)
    assert ws > 0 and ws % (256 * 4096 * 12) == 0                     # splits x (max, min, packed groups) x N*M x 4 B
    assert l.mam_fc_forward_values_workspace(256, 4096, 4096) * 3 == ws * 2
    assert l.mam_fc_forward_workspace(0, 5, 5) == 0


def test_argument_validation_without_a_gpu():
    l = capi.lib()
    # invalid arguments are rejected on the host before anything is launched
    assert l.mam_fc_forward(None, 4, None, 4, 7, None, None, None, None, None, None, 2, 4, 2, None, 0, None) == -1
    assert b"w_layout" in l.mam_last_error()
    assert l.mam_fc_forward(None, 4, None, 4, 0, None, None, None, None, None, None, -1, 4, 2, None, 0, None) == -1
    assert l.mam_fc_forward(None, 4, None, 4, 0, None, None, None, None, None, None, 2, 4, 2, None, 0, None) == -1
    assert b"null" in l.mam_last_error()
    assert l.mam_selection_count(None, None, None, None, 2, 2, 2, 9, None) == -1
    # sizes beyond what the kernels index are refused, not truncated (pointers never dereferenced)
    one = ctypes.c_void_p(16)
    big = 2 ** 30 + 1
    assert l.mam_fc_forward(one, big, one, big, 0, None, one, one, one, None, None, 2, big, 2, None, 0, None) == -2
    assert b"2^30" in l.mam_last_error()
    assert l.mam_fc_backward(one, 4, one, 4, 1, one, one, one, None, None, one, one, big, 4, 2, None) == -2
    assert l.mam_selection_count(one, one, one, one, 2, big, 2, 1, None) == -2
    assert l.mam_fc_forward(one, 2, one, 4, 0, None, one, one, one, None, None, 2, 4, 2, None, 0, None) == -1
    assert b"leading dimension" in l.mam_last_error()
    # empty problems are a no-op
    assert l.mam_fc_forward(None, 4, None, 4, 0, None, None, None, None, None, None, 0, 4, 2, None, 0, None) == 0
    assert l.mam_selection_count(None, None, None, None, 0, 2, 2, 0, None) == 0


REFERENCE_SCHEMAS = {
    # mamtorch/kernel/v1/csrc/register_functions.cpp:21-24
    ("mamtorch_kernel_v1", "fullyconnected"): "mamtorch_kernel_v1::fullyconnected(Tensor a, Tensor b) -> Tensor[]",
    ("mamtorch_kernel_v1", "fullyconnected_backward"):
        "mamtorch_kernel_v1::fullyconnected_backward(Tensor a, Tensor b, Tensor grad, Tensor argmax, Tensor argmin) -> Tensor[]",
    # mamtorch/kernel/v4/csrc/register_functions.cpp:10-14
    ("mamtorch_kernel_v4", "fullyconnected"): "mamtorch_kernel_v4::fullyconnected(Tensor a, Tensor b) -> Tensor[]",
    ("mamtorch_kernel_v4", "fullyconnected_fast"): "mamtorch_kernel_v4::fullyconnected_fast(Tensor a, Tensor b) -> Tensor",
    ("mamtorch_kernel_v4", "fullyconnected_backward"):
        "mamtorch_kernel_v4::fullyconnected_backward(Tensor a, Tensor b, Tensor grad, Tensor argmax, Tensor argmin) -> Tensor[]",
}


@pytest.mark.parametrize("key", sorted(REFERENCE_SCHEMAS))
def test_operator_schemas_match_the_reference(key):
    ns, name = key
    op = getattr(getattr(torch.ops, ns), name).default
    assert str(op._schema) == REFERENCE_SCHEMAS[key]


def test_python_surface_matches_reference_layout():
    assert callable(mt.kernel.v1.fullyconnected)
    assert callable(mt.kernel.v4.fullyconnected)
    assert callable(mt.kernel.v4.fullyconnected_fast)
    assert mt.nn.FullyConnected.__name__ == "FullyConnected"
    assert callable(mt.sparse.fullyconnected)


def test_no_cpu_fallback():
    a, b = torch.randn(3, 4), torch.randn(4, 5)
    with pytest.raises(NotImplementedError):
        mt.kernel.v1.fullyconnected(a, b)
    with pytest.raises(NotImplementedError):
        mt.kernel.v4.fullyconnected_fast(a, b)
    layer = mt.nn.FullyConnected(4, 5)
    with pytest.raises(NotImplementedError):
        layer(a)


def test_fake_kernels_propagate_shapes():
    a = torch.empty(7, 11, device="meta")
    b = torch.empty(11, 5, device="meta")
    w = torch.empty(5, 11, device="meta")
    c, amax, amin = torch.ops.mamtorch_kernel_v4.fullyconnected(a, b)
    assert c.shape == (7, 5) and c.dtype == torch.float32
    assert amax.dtype == torch.int32 and amin.shape == (7, 5)
    assert torch.ops.mamtorch_kernel_v4.fullyconnected_fast(a, b).shape == (7, 5)
    c, amax, amin = torch.ops.mamtorch_kernel_v1.fullyconnected(a, b)
    assert c.shape == (7, 5)
    c, amax, amin, sel = torch.ops.mamtorch_kernel_v4.fullyconnected_wt(a, w, None, False)
    assert sel.shape == (0, 7, 5)
    c, amax, amin, sel = torch.ops.mamtorch_kernel_v4.fullyconnected_wt(a, w, None, True)
    assert c.shape == (7, 5) and sel.shape == (4, 7, 5)
    g = torch.empty(7, 5, device="meta")
    ag, bg = torch.ops.mamtorch_kernel_v4.fullyconnected_backward(a, b, g, amax, amin)
    assert ag.shape == (7, 11) and bg.shape == (11, 5)
    ag, wg = torch.ops.mamtorch_kernel_v4.fullyconnected_wt_backward(a, w, g, amax, amin, sel)
    assert ag.shape == (7, 11) and wg.shape == (5, 11)
    with pytest.raises(RuntimeError):
        torch.ops.mamtorch_kernel_v4.fullyconnected(a, torch.empty(12, 5, device="meta"))


def test_module_constructor_and_repr():
    torch.manual_seed(0)
    layer = mt.nn.FullyConnected(784, 256)
    assert layer.weight.shape == (256, 784) and layer.bias.shape == (256,)
    # the draws are fp32: the largest one can round up to the fp32 value of the bound
    bound = float(np.float32(1 / 784 ** 0.5))
    assert float(layer.weight.detach().abs().max()) <= bound and float(layer.bias.detach().abs().max()) <= bound
    assert (layer.beta, layer.alpha) == (0.0, 1.0)
    assert repr(layer) == "MAM@FullyConnected(in_features=784, out_features=256, bias=True)"
    layer = mt.nn.FullyConnected(8, 4, bias=False, splits=3, relu_in=True, vcon_steps=10, vcon_expand=True)
    assert layer.bias is None
    assert (layer.in_subfeatures, layer.in_subfeatures_last) == (3, 2)
    assert repr(layer) == ("MAM@FullyConnected(in_features=8, out_features=4, bias=False, vcon_steps=10, "
                           "vcon_type=linear, splits=3, vcon_expand=True, relu_in=True)")
    assert sorted(n for n, _ in mt.nn.FullyConnected(3, 2).state_dict().items()) == ["bias", "weight"]


def test_vanishing_contribution_schedule():
    layer = mt.nn.FullyConnected(8, 4, vcon_steps=4)
    assert (layer.beta, layer.alpha) == (1.0, 0.0)
    betas = []
    for _ in range(5):
        layer.vcon_step()
        betas.append(layer.beta)
    assert betas[:3] == [0.75, 0.5, 0.25] and betas[3] == 0 and betas[4] == 0
    assert layer.alpha == 1.0
    layer = mt.nn.FullyConnected(8, 4, vcon_steps=3, vcon_type="exponential", vcon_eps=1e-3)
    layer.vcon_step()
    assert abs(layer.beta - 0.1) < 1e-12 and abs(layer.alpha - 0.9) < 1e-12
    layer.vcon_step(); layer.vcon_step()
    assert layer.beta == 0 or abs(layer.beta - 1e-3) < 1e-15   # gamma**3 lands on eps up to rounding
    layer.vcon_step()
    assert layer.beta == 0
    layer = mt.nn.FullyConnected(8, 4, vcon_steps=2, vcon_expand=True, splits=2)
    layer.vcon_step()
    assert layer.alpha == 0.5 * 8 / 4
    layer = mt.nn.FullyConnected(8, 4, vcon_steps=2, vcon_type="cosine")
    with pytest.raises(Exception, match="vcon_type 'cosine' is not supported"):
        layer.vcon_step()
    layer = mt.nn.FullyConnected(8, 4, vcon_steps=-1)
    with pytest.raises(Exception, match="Invalid value for vcon_steps"):
        layer.vcon_step()


def test_selection_count_requires_store_args():
    layer = mt.nn.FullyConnected(8, 4)
    with pytest.raises(Exception, match="store_args is False"):
        layer.reset_selection_count()
    with pytest.raises(Exception, match="store_args is False"):
        layer.update_selection_count()
    layer = mt.nn.FullyConnected(8, 4, store_args=True)
    with pytest.raises(Exception, match="No argmax or argmin"):
        layer.update_selection_count()
    layer.reset_selection_count()
    assert layer.max_selection_count.dtype == torch.int32 and layer.max_selection_count.shape == (4, 8)
    assert int(layer.min_selection_count.sum()) == 0


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU: any other --gpus value exits with a message before touching torch."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--workload", "nonsense"], capture_output=True,
                       text=True)
    assert r.returncode != 0


def test_legacy_layers_constructors_schedules_and_names():
    """mamtorch.nn.v1.FullyConnected, mamtorch.nn.v4.FullyConnected and mamtorch.MAMDense under their
    reference names (mamtorch/nn/__init__.py:1-6, mamtorch/__init__.py:7)."""
    assert mt.nn.v4.FullyConnected is mt.nn.FullyConnected
    layer = mt.nn.v1.FullyConnected(12, 6, vcon_steps=4, init_mode="normal")
    assert repr(layer) == "MAM@FullyConnected(in_features=12, out_features=6, bias=True, vcon_steps=4, vcon_type=linear)"
    assert layer.weight.shape == (6, 12) and bool((layer.bias == 0).all()) and layer.beta == 1.0
    for want in (0.75, 0.5, 0.25, 0):
        layer.vcon_step()
        assert layer.beta == want
    bound = float(np.float32((6 / (2 + 6)) ** 0.5))
    torch.manual_seed(0)
    uniform = mt.nn.v1.FullyConnected(50, 6)
    assert float(uniform.weight.abs().max()) <= bound and uniform.beta == 0.0
    with pytest.raises(Exception, match="not supported"):
        mt.nn.v1.FullyConnected(4, 4, vcon_steps=2, vcon_type="cubic").vcon_step()
    with pytest.raises(Exception, match="No argmax"):
        uniform.update_selection_count()
    dense = mt.MAMDense(10, 3, beta=True, beta_decay="descending-parabola", beta_epochs=4)
    assert dense.input_features == 10 and dense.state_size == 3 and dense.beta == 1.0
    dense.adjust_beta(2)
    assert dense.beta == 0.75
    dense.adjust_beta(4)
    assert dense.beta == 0
    asc = mt.MAMDense(10, 3, beta=True, beta_decay="ascending-parabola", beta_epochs=4)
    asc.adjust_beta(1)
    assert abs(asc.beta - 0.5625) < 1e-12


def test_resolve_row_offsets_at_a_weight_beyond_4_gib(tmp_path):
    """The 32-bit weight-row offsets of the index-resolving code (mamtorch_amd/csrc/mam_offsets.h), checked
    by a host-only C++ program at M = 262150, ldw = 4096, where (M - 1) * ldw * 4 wraps in 32 bits."""
    import subprocess

    exe = str(tmp_path / "offsets_host")
    subprocess.run(["g++", "-O1", "-std=c++17", os.path.join(ROOT, "tests", "offsets_host.cpp"), "-o", exe], check=True)
    r = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stdout[-2000:]


def test_static_forward_limit_is_checked_on_the_host():
    l = capi.lib()
    N, K, M = 224, 4096, 4224      # 3 ranges of K x 3 planes x N*M words = 34 MB of partials
    assert l.mam_fc_forward_workspace(N, K, M) > l.mam_fc_forward_static_limit() >= 24 * 2 ** 20
    one = ctypes.c_void_p(16)       # never dereferenced: the size check precedes every launch
    assert l.mam_fc_forward_static(one, K, one, K, capi.W_MK, None, one, one, one, None, None, N, K, M, None) == -2
    assert b"scratch" in l.mam_last_error()
    assert l.mam_set_option(99, 0) == -1
    # a value outside the option's range is refused and leaves the option as it was
    assert l.mam_set_option(capi.OPT_BACKWARD_ONE_LAUNCH, 3) == -1
    assert l.mam_set_option(capi.OPT_FORWARD_TILING, -1) == -1
    assert l.mam_set_option(capi.OPT_FORWARD_TILING, capi.FORWARD_TILING_AUTO) == 0


def test_the_reference_import_name():
    import mamtorch
    import mamtorch.kernel.v4.fullyconnected_fast  # noqa: F401
    import mamtorch.nn.compat
    import mamtorch.nn.v1.fullyconnected
    import mamtorch.nn.v4.fullyconnected
    import mamtorch.sparse.kernel.v1.cusparsemm  # noqa: F401

    assert mamtorch.nn.FullyConnected is mt.nn.FullyConnected is mamtorch.nn.v4.fullyconnected.FullyConnected
    assert mamtorch.nn.v1.fullyconnected.FullyConnected is mt.nn.FullyConnectedV1
    assert mamtorch.MAMDense is mamtorch.nn.compat.MAMDense
    assert mamtorch.kernel.v4.fullyconnected is mt.kernel.v4.fullyconnected
