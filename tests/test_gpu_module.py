"""GPU tests of the PyTorch-facing boundary: torch.ops operators (schemas of the reference),
autograd wiring, torch.library.opcheck (as test/test.py:28,134,168 of the reference does), and
the FullyConnected module against the oracle."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import mamtorch_amd as mt
import oracle
from helpers import assert_bits_equal, assert_index_equal, config1, pruned_csr, random_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _oracle_kmb(a, b):
    return oracle.forward(a.cpu().numpy(), b.cpu().numpy(), oracle.W_KM)


@pytest.mark.parametrize("ns", ["mamtorch_kernel_v1", "mamtorch_kernel_v4"])
def test_reference_operators_forward_backward(ns):
    ops = getattr(torch.ops, ns)
    x, w, grad = random_case(70, 123, 45, seed=1)
    a = x.to(DEV).requires_grad_(True)
    b = w.T.contiguous().to(DEV).requires_grad_(True)
    c, amax, amin = ops.fullyconnected(a, b)
    want = _oracle_kmb(x, w.T.contiguous())
    assert_bits_equal(c.detach().cpu().numpy(), want[0], ns + " c")
    assert_index_equal(amax.cpu().numpy(), want[1], ns + " argmax")
    assert_index_equal(amin.cpu().numpy(), want[2], ns + " argmin")
    assert amax.dtype == torch.int32 and c.dtype == torch.float32
    c.backward(grad.to(DEV))
    xo, bo = oracle.backward(x.numpy(), w.T.contiguous().numpy(), grad.numpy(), want[1], want[2], oracle.W_KM)
    np.testing.assert_allclose(a.grad.cpu().numpy(), xo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(b.grad.cpu().numpy(), bo, rtol=1e-5, atol=1e-6)
    ag, bg = ops.fullyconnected_backward(a.detach(), b.detach(), grad.to(DEV), amax, amin)
    np.testing.assert_allclose(ag.cpu().numpy(), xo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(bg.cpu().numpy(), bo, rtol=1e-5, atol=1e-6)


def test_fast_operator_values_and_mac_gradient():
    x, w, grad = random_case(33, 65, 20, seed=2)
    a = x.to(DEV).requires_grad_(True)
    b = w.T.contiguous().to(DEV).requires_grad_(True)
    c = mt.kernel.v4.fullyconnected_fast(a, b)
    assert_bits_equal(c.detach().cpu().numpy(), _oracle_kmb(x, w.T.contiguous())[0], "fast c")
    c.backward(grad.to(DEV))
    # registered backward of the fast operator is the dense MAC gradient
    # (mamtorch/kernel/v4/fullyconnected_fast.py:22-28)
    assert torch.allclose(a.grad, grad.to(DEV) @ b.detach().T, rtol=1e-4, atol=1e-4)
    assert torch.allclose(b.grad, a.detach().T @ grad.to(DEV), rtol=1e-4, atol=1e-4)


def test_opcheck():
    x, w, grad = random_case(20, 37, 11, seed=3)
    a = x.to(DEV).requires_grad_(True)
    b = w.T.contiguous().to(DEV).requires_grad_(True)
    wt = w.to(DEV).requires_grad_(True)
    bias = torch.randn(11, device=DEV, requires_grad=True)
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.mamtorch_kernel_v1.fullyconnected, (a, b), test_utils=tests)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected, (a, b), test_utils=tests)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_fast, (a, b), test_utils=tests)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_wt, (a, wt, bias, True), test_utils=tests)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_fast_wt, (a, wt, None), test_utils=tests)
    _, amax, amin = torch.ops.mamtorch_kernel_v4.fullyconnected(a.detach(), b.detach())
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.fullyconnected_backward,
                          (a.detach(), b.detach(), grad.to(DEV), amax, amin), test_utils=("test_schema", "test_faketensor"))
    keep = torch.rand(11, 37, device=DEV) < 0.5
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.apply_keep, (wt, keep), test_utils=tests)


def test_operator_errors_are_runtime_errors():
    a = torch.randn(4, 6, device=DEV)
    b = torch.randn(6, 5, device=DEV)
    with pytest.raises(RuntimeError, match="float32"):
        torch.ops.mamtorch_kernel_v4.fullyconnected(a.double(), b.double())
    with pytest.raises(RuntimeError, match="inner dimensions"):
        torch.ops.mamtorch_kernel_v4.fullyconnected(a, torch.randn(7, 5, device=DEV))
    with pytest.raises(RuntimeError, match="unit stride"):
        torch.ops.mamtorch_kernel_v4.fullyconnected(a.T.contiguous().T, b)
    with pytest.raises(RuntimeError):
        torch.ops.mamtorch_kernel_v4.fullyconnected(a, b.cpu())
    c, amax, amin = torch.ops.mamtorch_kernel_v4.fullyconnected(a, b)
    with pytest.raises(RuntimeError, match="int32"):
        torch.ops.mamtorch_kernel_v4.fullyconnected_backward(a, b, c, amax.long(), amin)
    with pytest.raises(RuntimeError, match="shape"):
        torch.ops.mamtorch_kernel_v4.fullyconnected_backward(a, b, c, amax[:2], amin)
    # empty batch is fine
    c, amax, amin = torch.ops.mamtorch_kernel_v4.fullyconnected(a[:0], b)
    assert c.shape == (0, 5)


def _layer_from(w, bias, **kw):
    layer = mt.nn.FullyConnected(w.shape[1], w.shape[0], bias=bias is not None, **kw)
    with torch.no_grad():
        layer.weight.copy_(w)
        if bias is not None:
            layer.bias.copy_(bias)
    return layer.to(DEV)


def test_module_config1_training_step_and_selection_count():
    x, w, bias, grad = config1()
    layer = _layer_from(w, bias, store_args=True).train()
    xin = x.to(DEV).requires_grad_(True)
    y = layer(xin)
    want = oracle.forward(x.numpy(), w.numpy(), oracle.W_MK, bias.numpy())
    assert_bits_equal(y.detach().cpu().numpy(), want[0], "module y")
    assert_index_equal(layer.argmax.cpu().numpy(), want[1], "module argmax")
    assert_index_equal(layer.argmin.cpu().numpy(), want[2], "module argmin")
    y.backward(grad.to(DEV))
    xo, wo = oracle.backward(x.numpy(), w.numpy(), grad.numpy(), want[1], want[2], oracle.W_MK)
    np.testing.assert_allclose(xin.grad.cpu().numpy(), xo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(layer.weight.grad.cpu().numpy(), wo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(layer.bias.grad.cpu().numpy(), grad.numpy().sum(0), rtol=1e-5, atol=1e-5)
    # selection counting, literal reference rule (default) over two batches
    layer.update_selection_count()
    layer.update_selection_count()
    z = np.zeros(w.shape, np.int32)
    mc, _ = oracle.selection_count(want[1], want[2], z, z, 0)
    np.testing.assert_array_equal(layer.max_selection_count.cpu().numpy(), 2 * mc)
    assert int(layer.min_selection_count.sum()) == 0
    layer.selection_count_mode = "hits"
    layer.reset_selection_count()
    layer.update_selection_count()
    mc, nc = oracle.selection_count(want[1], want[2], z, z, 1)
    np.testing.assert_array_equal(layer.max_selection_count.cpu().numpy(), mc)
    np.testing.assert_array_equal(layer.min_selection_count.cpu().numpy(), nc)


def test_module_eval_path_3d_input_relu_and_no_bias():
    x, w, _ = random_case(6 * 7, 50, 30, seed=4)
    layer = _layer_from(w, None, relu_in=True).eval()
    xin = x.view(6, 7, 50).to(DEV)
    with torch.no_grad():
        y = layer(xin)
    assert y.shape == (6, 7, 30)
    want = oracle.forward(torch.relu(x).numpy(), w.numpy(), oracle.W_MK)
    assert_bits_equal(y.reshape(42, 30).cpu().numpy(), want[0], "eval relu y")
    assert layer.argmax is None


def test_module_splits_sum_of_slices():
    x, w, grad = random_case(25, 50, 12, seed=5)
    bias = torch.randn(12, generator=torch.Generator().manual_seed(5))
    layer = _layer_from(w, bias, splits=3).train()
    xin = x.to(DEV).requires_grad_(True)
    y = layer(xin)
    # slices of ceil(50/3) = 17, 17 and 16 input features
    bounds = [(0, 17), (17, 34), (34, 50)]
    total = None
    xo = np.zeros((25, 50), np.float32)
    wo = np.zeros((12, 50), np.float32)
    for lo, hi in bounds:
        c, amax, amin = oracle.forward(x[:, lo:hi].numpy(), w[:, lo:hi].numpy(), oracle.W_MK)
        total = c if total is None else (total + c).astype(np.float32)
        gx, gw = oracle.backward(x[:, lo:hi].numpy(), w[:, lo:hi].numpy(), grad.numpy(), amax, amin, oracle.W_MK)
        xo[:, lo:hi], wo[:, lo:hi] = gx, gw
    assert_bits_equal(y.detach().cpu().numpy(), (total + bias.numpy()).astype(np.float32), "splits y")
    y.backward(grad.to(DEV))
    np.testing.assert_allclose(xin.grad.cpu().numpy(), xo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(layer.weight.grad.cpu().numpy(), wo, rtol=1e-5, atol=1e-6)


def test_module_vanishing_contribution_blend():
    x, w, grad = random_case(16, 40, 10, seed=6)
    bias = torch.randn(10, generator=torch.Generator().manual_seed(6))
    layer = _layer_from(w, bias, vcon_steps=4).train()
    xin = x.to(DEV)
    mac = F.linear(xin, layer.weight, None)
    y = layer(xin)                       # beta = 1: pure MAC + bias
    assert torch.allclose(y, mac + layer.bias, rtol=1e-6, atol=1e-6)
    layer.vcon_step()                    # beta = 0.75
    mam = torch.tensor(oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)[0]).to(DEV)
    y = layer(xin)
    assert torch.allclose(y, 0.25 * mam + 0.75 * mac + layer.bias, rtol=1e-5, atol=1e-6)
    for _ in range(3):
        layer.vcon_step()
    assert layer.beta == 0
    y = layer(xin)
    assert_bits_equal(y.detach().cpu().numpy(), (mam + layer.bias).detach().cpu().numpy(), "beta=0 y")


def test_module_weight_dropout_and_output_dropout_run():
    x, w, _ = random_case(8, 20, 6, seed=7)
    layer = _layer_from(w, None, wdrop_rate=0.5, drop_rate=0.5).train()
    torch.manual_seed(0)
    y = layer(x.to(DEV))
    assert y.shape == (8, 6) and torch.isfinite(y).all()
    layer.wdrop_rate = 1.5
    with pytest.raises(Exception, match="wdrop_rate must be between 0 and 1"):
        layer(x.to(DEV))


@pytest.mark.parametrize("shape", [(6, 20), (45, 123), (256, 784), (130, 4096)])
def test_apply_keep_is_the_reference_expression_on_a_fixed_mask(shape):
    """weight * mask with the mask as bytes: bit-equal to the reference's float expression
    (mamtorch/nn/v4/fullyconnected.py:143-148), signed zeros and non-finite weights included; strided weight
    views; the gradient is the same masking."""
    M, Kin = shape
    g = torch.Generator().manual_seed(M + Kin)
    w = torch.randn(M, Kin, generator=g)
    w[0, 0], w[M - 1, Kin - 1], w[M // 2, 1] = float("inf"), -0.0, float("nan")
    keep = torch.rand(M, Kin, generator=g) < 0.6
    keep[0, 0] = True
    w[1, 2], keep[1, 2] = float("-inf"), False      # inf * 0: NaN here as in the reference (its sign is the platform's)
    want = w * keep.to(torch.float32)
    wd = w.to(DEV).requires_grad_(True)
    got = mt.kernel.v4.apply_keep(wd, keep.to(DEV))
    assert torch.isnan(got[1, 2]) and torch.isnan(want[1, 2])
    want[1, 2] = got[1, 2].item()
    want = torch.where(torch.isnan(want), got.detach().cpu(), want)
    assert torch.isnan(got[M // 2, 1])
    assert_bits_equal(got.detach().cpu().numpy(), want.numpy(), "apply_keep %s" % (shape,))
    grad = torch.randn(M, Kin, generator=g)
    got.backward(grad.to(DEV))
    assert_bits_equal(wd.grad.cpu().numpy(), (grad * keep.to(torch.float32)).numpy(), "apply_keep gradient")
    # a view with a longer row stride and an unaligned base
    wide = torch.randn(M, Kin + 7, generator=g).to(DEV)
    got = mt.kernel.v4.apply_keep(wide[:, 3:3 + Kin], keep.to(DEV))
    assert_bits_equal(got.cpu().numpy(), (wide[:, 3:3 + Kin].cpu() * keep.to(torch.float32)).numpy(), "strided view")
    got8 = mt.kernel.v4.apply_keep(wd.detach(), keep.to(DEV).to(torch.uint8))
    assert_bits_equal(got8.cpu().numpy(), want.numpy(), "uint8 mask")


def test_module_weight_dropout_against_the_oracle():
    """Training-time weight dropout: the layer's output is the MAM of x and weight * mask for the mask the
    layer drew (same generator state, same call), bit for bit; dropped weights get no gradient."""
    x, w, grad = random_case(33, 128, 40, seed=17)
    layer = _layer_from(w, None, wdrop_rate=0.3).train()
    torch.manual_seed(5)
    y = layer(x.to(DEV))
    torch.manual_seed(5)
    keep = torch.empty(w.shape, dtype=torch.bool, device=DEV).bernoulli_(1 - 0.3)
    assert 0.5 < keep.float().mean().item() < 0.9
    wm = (w * keep.cpu().to(torch.float32))
    want = oracle.forward(x.numpy(), wm.numpy(), oracle.W_MK)
    assert_bits_equal(y.detach().cpu().numpy(), want[0], "weight dropout y")
    y.backward(grad.to(DEV))
    _, wo = oracle.backward(x.numpy(), wm.numpy(), grad.numpy(), want[1], want[2], oracle.W_MK)
    wo = wo * keep.cpu().numpy()
    np.testing.assert_allclose(layer.weight.grad.cpu().numpy(), wo, rtol=1e-5, atol=1e-6)
    assert (layer.weight.grad[~keep] == 0).all()
    layer.eval()
    y = layer(x.to(DEV))
    assert_bits_equal(y.detach().cpu().numpy(), oracle.forward(x.numpy(), w.numpy(), oracle.W_MK)[0], "eval: no dropout")


def test_sparse_operator_and_autograd_function():
    M, K, N = 90, 200, 17
    dense, crow, col, val = pruned_csr(M, K, 0.1, seed=8)
    x = torch.randn(N, K, generator=torch.Generator().manual_seed(8))
    w_csr = dense.to(DEV).to_sparse_csr()
    c, amax, amin = mt.sparse.fullyconnected(x.to(DEV), w_csr)
    want = oracle.forward(x.numpy(), dense.numpy(), oracle.W_MK)
    assert_bits_equal(c.cpu().numpy(), want[0], "sparse op c")
    assert_index_equal(amax.cpu().numpy(), want[1], "sparse op argmax")
    assert_index_equal(amin.cpu().numpy(), want[2], "sparse op argmin")
    # prune_to_csr keeps explicitly stored zeros, to_sparse_csr drops them: same dense matrix
    w2 = mt.sparse.prune_to_csr(dense.to(DEV), (dense != 0).to(DEV))
    c2, _, _ = mt.sparse.fullyconnected(x.to(DEV), w2)
    assert torch.equal(c2, c)
    grad = torch.randn(N, M, generator=torch.Generator().manual_seed(9))
    xin = x.to(DEV).requires_grad_(True)
    vals = w2.values().clone().requires_grad_(True)
    cc, _, _ = mt.sparse.SparseFullyConnectedFunction.apply(xin, vals, w2.crow_indices(), w2.col_indices(), M)
    cc.backward(grad.to(DEV))
    xo, vo = oracle.csr_backward(x.numpy(), w2.crow_indices().cpu().numpy(), w2.col_indices().cpu().numpy(),
                                 w2.values().cpu().numpy(), grad.numpy(), want[1], want[2])
    np.testing.assert_allclose(xin.grad.cpu().numpy(), xo, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(vals.grad.cpu().numpy(), vo, rtol=1e-5, atol=1e-6)


def test_linear_layers_swapped_for_mam_and_vit_mlp_block():
    """examples/vitb16_imagenet1k/utils.py:67-77: the swapped layer starts from the Linear's weight and
    bias; the ViT-B/16 MLP block (768 -> 3072 -> 768) on 2 x 197 tokens against the oracle, layer by layer."""
    torch.manual_seed(0)
    model = torch.nn.Sequential()
    model.add_module("encoder", torch.nn.Module())
    model.encoder.intermediate = torch.nn.Linear(64, 96)
    model.encoder.output = torch.nn.Linear(96, 64, bias=False)
    model.encoder.keep = torch.nn.Linear(8, 8)
    w1, b1 = model.encoder.intermediate.weight.data.clone(), model.encoder.intermediate.bias.data.clone()
    mt.nn.add_mam_to_model(model, ["encoder.intermediate", "encoder.output"], vcon_steps=4, store_args=True)
    assert isinstance(model.encoder.intermediate, mt.nn.FullyConnected)
    assert isinstance(model.encoder.output, mt.nn.FullyConnected) and model.encoder.output.bias is None
    assert isinstance(model.encoder.keep, torch.nn.Linear)
    assert torch.equal(model.encoder.intermediate.weight.data, w1) and torch.equal(model.encoder.intermediate.bias.data, b1)
    assert model.encoder.intermediate.beta == 1.0 and model.encoder.intermediate.vcon_steps == 4
    assert mt.nn.get_layers(model, ["encoder.keep"])[0] is model.encoder.keep
    with pytest.raises(TypeError):
        mt.nn.add_mam_to_model(model, ["encoder.output"])

    block = mt.nn.MAMMlp().to(DEV)
    tokens = torch.randn(2, 197, 768, generator=torch.Generator().manual_seed(1)).to(DEV).requires_grad_(True)
    out = block(tokens)
    assert out.shape == tokens.shape
    normed = block.norm(tokens.detach()).detach().reshape(-1, 768)
    c1 = oracle.forward(normed.cpu().numpy(), block.intermediate.weight.detach().cpu().numpy(), oracle.W_MK,
                        block.intermediate.bias.detach().cpu().numpy())[0]
    h = F.gelu(torch.from_numpy(c1).to(DEV))
    c2 = oracle.forward(h.cpu().numpy(), block.output.weight.detach().cpu().numpy(), oracle.W_MK,
                        block.output.bias.detach().cpu().numpy())[0]
    want = tokens.detach().reshape(-1, 768) + torch.from_numpy(c2).to(DEV)
    assert_bits_equal(out.detach().reshape(-1, 768).cpu().numpy(), want.cpu().numpy(), "MLP block output")
    out.sum().backward()
    assert tokens.grad is not None and block.intermediate.weight.grad is not None
    assert torch.isfinite(tokens.grad).all()


def test_legacy_layers_against_the_oracle():
    """nn.v1.FullyConnected and MAMDense: pure MAM output bit-exact (bias added after max + min), blended
    output against the same expression on the oracle's MAM term, gradients of both, literal selection count."""
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 7, 40, generator=g)
    for make in (lambda: mt.nn.v1.FullyConnected(40, 24), lambda: mt.MAMDense(40, 24)):
        layer = make()
        with torch.no_grad():
            layer.bias.copy_(torch.randn(24, generator=g))
        w, b = layer.weight.detach().clone(), layer.bias.detach().clone()
        layer = layer.to(dev)
        c_ref, amax, amin = oracle.forward(x.reshape(-1, 40).numpy(), w.numpy(), oracle.W_MK, b.numpy())
        xd = x.to(dev).requires_grad_(True)
        y = layer(xd)
        assert y.shape == (5, 7, 24)
        assert_bits_equal(y.detach().cpu().numpy().reshape(-1, 24), c_ref, "legacy pure MAM output")
        assert_index_equal(layer.argmax.cpu().numpy(), amax, "argmax")
        grad = torch.randn(5, 7, 24, generator=g)
        y.backward(grad.to(dev))
        xg, wg = oracle.backward(x.reshape(-1, 40).numpy(), w.numpy(), grad.reshape(-1, 24).numpy(), amax, amin, oracle.W_MK)
        assert np.allclose(xd.grad.cpu().numpy().reshape(-1, 40), xg, rtol=1e-5, atol=1e-6)
        assert np.allclose(layer.weight.grad.cpu().numpy(), wg, rtol=1e-5, atol=1e-6)
        assert np.allclose(layer.bias.grad.cpu().numpy(), grad.reshape(-1, 24).sum(0).numpy(), rtol=1e-5, atol=1e-5)
        layer.update_selection_count()
        zeros = np.zeros((24, 40), np.int32)
        want_count, _ = oracle.selection_count(amax, amin, zeros, zeros, mode=0)
        assert np.array_equal(layer.max_selection_count.cpu().numpy(), want_count)
        assert not layer.min_selection_count.any()
        # blended: (1 - beta) * MAM + bias + beta * MAC
        layer.beta = 0.25
        y2 = layer(x.to(dev)).cpu()
        c_mam = oracle.forward(x.reshape(-1, 40).numpy(), w.numpy(), oracle.W_MK)[0]
        want = (0.75 * torch.from_numpy(c_mam) + b.view(1, -1)).view(5, 7, 24) + 0.25 * torch.nn.functional.linear(x, w)
        assert torch.allclose(y2, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("N,M", [(1, 1), (64, 256), (256, 4096), (513, 70), (1300, 333), (12608, 768)])
def test_bias_gradient_is_the_column_sum(N, M):
    """The layer's bias gradient (autograd of the `+ bias` after max + min, mamtorch/nn/v4/fullyconnected.py:197-198)
    as one kernel: column sums in a fixed order, the same bits on every call, against the fp64 sum."""
    g = torch.randn(N, M, generator=torch.Generator().manual_seed(N + M)).to(DEV)
    got = torch.ops.mamtorch_kernel_v4.bias_grad(g)
    again = torch.ops.mamtorch_kernel_v4.bias_grad(g)
    want = g.double().sum(dim=0)
    floor = g.abs().double().sum(dim=0)
    assert got.shape == (M,) and torch.equal(got, again)
    assert bool(((got.double() - want).abs() <= 1e-5 * want.abs() + 2.0 ** -22 * floor).all())
    # a strided view (every other column block of a wider matrix)
    wide = torch.randn(N, 2 * M + 3, generator=torch.Generator().manual_seed(7)).to(DEV)
    view = wide[:, 3:3 + M]
    assert bool(((torch.ops.mamtorch_kernel_v4.bias_grad(view).double() - view.double().sum(dim=0)).abs()
                 <= 1e-5 * view.double().sum(dim=0).abs() + 2.0 ** -22 * view.abs().double().sum(dim=0)).all())


def test_bias_gradient_through_the_module():
    layer = mt.nn.FullyConnected(96, 40, bias=True).to(DEV).train()
    x = torch.randn(50, 96, generator=torch.Generator().manual_seed(3)).to(DEV).requires_grad_(True)
    g = torch.randn(50, 40, generator=torch.Generator().manual_seed(4)).to(DEV)
    layer(x).backward(g)
    torch.testing.assert_close(layer.bias.grad, g.sum(dim=0), rtol=1e-5, atol=1e-5)
