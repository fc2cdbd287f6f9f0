"""`import mamtorch`: the reference's import name and module paths, and its own call patterns (restated
from test/test.py:21-35 v1 operator + opcheck, :130-180 v4 / fast / backward operators, and
test/test_sparse.py:33-44 cusparsemm; the reference draws n, m, l in [10, 1000] unseeded, here seeded),
checked against the oracle instead of printed."""
import random

import numpy as np
import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_index_equal

pytestmark = pytest.mark.gpu
device = torch.device("cuda:0")


def _random_abc(seed):
    rng = random.Random(seed)
    n, m, l = rng.randint(10, 1000), rng.randint(10, 1000), rng.randint(10, 1000)
    g = torch.Generator().manual_seed(seed)
    a = torch.randn((n, m), dtype=torch.float32, generator=g)
    b = torch.randn((m, l), dtype=torch.float32, generator=g)
    c = torch.randn((n, l), dtype=torch.float32, generator=g)
    return a, b, c


def test_module_paths_of_the_reference_resolve():
    import importlib

    import mamtorch
    import mamtorch.nn.compat as compat
    import mamtorch.nn.v1.fullyconnected as nn_v1_module
    import mamtorch.nn.v4.fullyconnected as nn_v4_module
    from mamtorch.kernel.v4 import fullyconnected, fullyconnected_fast   # noqa: F401

    # as in the reference, the attribute `fullyconnected` of the package is the function (it shadows the
    # submodule of the same name), so the submodules are taken from the import system
    k1_module = importlib.import_module("mamtorch.kernel.v1.fullyconnected")
    k4_fast_module = importlib.import_module("mamtorch.kernel.v4.fullyconnected_fast")
    spmm_module = importlib.import_module("mamtorch.sparse.kernel.v1.cusparsemm")

    assert mamtorch.nn.FullyConnected is nn_v4_module.FullyConnected is mamtorch.nn.v4.FullyConnected
    assert mamtorch.nn.v1.FullyConnected is nn_v1_module.FullyConnected
    assert mamtorch.MAMDense is compat.MAMDense and compat.__all__ == ["MAMDense"]
    assert callable(k1_module.fullyconnected) and callable(k4_fast_module.fullyconnected_fast)
    assert callable(spmm_module.cusparsemm) and callable(mamtorch.sparse.kernel.v1.cusparsemm)
    assert mamtorch.kernel.v1.fullyconnected is k1_module.fullyconnected


@pytest.mark.parametrize("seed", [0, 1])
def test_reference_operator_call_patterns(seed):
    import mamtorch   # noqa: F401  (registers torch.ops.mamtorch_kernel_*)

    a_cpu, b_cpu, c_cpu = _random_abc(seed)
    a, b, c = a_cpu.to(device), b_cpu.to(device), c_cpu.to(device)
    want = oracle.forward(a_cpu.numpy(), b_cpu.numpy(), oracle.W_KM)

    # test/test.py:26-35
    torch.library.opcheck(torch.ops.mamtorch_kernel_v1.fullyconnected, (a, b))
    res, argmax, argmin = torch.ops.mamtorch_kernel_v1.fullyconnected(a, b)
    assert_bits_equal(res.cpu().numpy(), want[0], "v1 res")
    assert_index_equal(argmax.cpu().numpy(), want[1], "v1 argmax")
    assert_index_equal(argmin.cpu().numpy(), want[2], "v1 argmin")

    # test/test.py:131-149: the reference's v4 kernel is approximate; this one has error zero
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected, (a, b))
    res, argmax, argmin = torch.ops.mamtorch_kernel_v4.fullyconnected(a, b)
    assert_bits_equal(res.cpu().numpy(), want[0], "v4 res")
    assert_index_equal(argmax.cpu().numpy(), want[1], "v4 argmax")
    assert_index_equal(argmin.cpu().numpy(), want[2], "v4 argmin")

    # test/test.py:165-173
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_fast, (a, b))
    res = torch.ops.mamtorch_kernel_v4.fullyconnected_fast(a, b)
    assert_bits_equal(res.cpu().numpy(), want[0], "v4 fast res")

    # test/test.py:175-180
    agrad, bgrad = torch.ops.mamtorch_kernel_v4.fullyconnected_backward(a, b, c, argmax, argmin)
    ag_want, bg_want = oracle.backward(a_cpu.numpy(), b_cpu.numpy(), c_cpu.numpy(), want[1], want[2], oracle.W_KM)
    np.testing.assert_allclose(agrad.cpu().numpy(), ag_want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(bgrad.cpu().numpy(), bg_want, rtol=1e-5, atol=1e-5)


def test_reference_layer_and_wrappers_under_the_reference_name():
    import mamtorch

    a_cpu, b_cpu, _ = _random_abc(2)
    K, M = b_cpu.shape
    layer = mamtorch.nn.FullyConnected(K, M, bias=True, store_args=True)
    x = a_cpu.to(device)
    want = oracle.forward(a_cpu.numpy(), layer.weight.detach().numpy(), oracle.W_MK, layer.bias.detach().numpy())
    layer = layer.to(device)
    y = layer(x)
    assert_bits_equal(y.detach().cpu().numpy(), want[0], "layer output")
    assert_index_equal(layer.argmax.cpu().numpy(), want[1], "layer argmax")
    res, argmax, argmin = mamtorch.kernel.v4.fullyconnected(x, b_cpu.to(device))
    w2 = oracle.forward(a_cpu.numpy(), b_cpu.numpy(), oracle.W_KM)
    assert_bits_equal(res.cpu().numpy(), w2[0], "wrapper res")
    assert_bits_equal(mamtorch.kernel.v4.fullyconnected_fast(x, b_cpu.to(device)).cpu().numpy(), w2[0], "fast wrapper")
    assert_bits_equal(mamtorch.kernel.v1.fullyconnected(x, b_cpu.to(device))[0].cpu().numpy(), w2[0], "v1 wrapper")


@pytest.mark.parametrize("layout", [torch.sparse_csr, torch.sparse_coo])
def test_reference_sparse_call_pattern(layout):
    import mamtorch   # noqa: F401

    # test/test_sparse.py:13-16,22-44
    rng = random.Random(3)
    n, l, m = rng.randint(10, 1000), rng.randint(10, 1000), rng.randint(10, 1000)
    g = torch.Generator().manual_seed(3)
    a = torch.randn((n, l), dtype=torch.float32, generator=g)
    a = a * torch.bernoulli(torch.full_like(a, 1 - 0.9), generator=g)
    b = torch.randn((l, m), dtype=torch.float32, generator=g)
    asparse = a.to(device).to_sparse(layout=layout)
    res = torch.ops.mamtorch_kernel_sparsev1.cusparsemm(asparse, b.to(device))
    want = a.double() @ b.double()
    floor = (a.abs().double() @ b.abs().double()) * 2.0 ** -22
    err = (res.cpu().double() - want).abs()
    assert bool((err <= 1e-5 * want.abs() + floor).all())
    res2 = mamtorch.sparse.kernel.v1.cusparsemm(asparse, b.to(device))
    assert torch.equal(res2, res) or layout == torch.sparse_coo   # COO accumulates with atomics
