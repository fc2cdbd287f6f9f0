"""MAM convolutions (MAMConv1d / MAMConv2d: window gather + the dense MAM kernels) against the oracle's
scalar definition of the reference's retired conv kernels: forward values bit-exact, indices exact,
gradients within rtol 1e-5 (plus the fp32 summation floor where windows overlap), the MAC blend and the
selection counts against the reference's literal formulas."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import mamtorch_amd as mt
import oracle
from oracle import brute
from helpers import assert_bits_equal, assert_index_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _conv1d(w, bias=None, **kw):
    layer = mt.nn.MAMConv1d(w.shape[1], w.shape[0], w.shape[2], bias=bias is not None, **kw)
    with torch.no_grad():
        layer.weight.copy_(w)
        if bias is not None:
            layer.bias.copy_(bias)
    return layer.to(DEV)


def _conv2d(w, bias=None, **kw):
    layer = mt.nn.MAMConv2d(w.shape[1], w.shape[0], (w.shape[2], w.shape[3]), bias=bias is not None, **kw)
    with torch.no_grad():
        layer.weight.copy_(w)
        if bias is not None:
            layer.bias.copy_(bias)
    return layer.to(DEV)


def test_hand_derived_known_answers():
    for kat in json.load(open(os.path.join(GOLDEN, "kat_conv.json"))):
        x = torch.tensor(kat["x"], dtype=torch.float32)
        w = torch.tensor(kat["w"], dtype=torch.float32)
        layer = _conv1d(w, stride=kat["stride"])
        y = layer(x.to(DEV))
        assert y.shape == torch.Size(np.shape(kat["y"]))
        assert_bits_equal(y.detach().cpu().numpy(), np.array(kat["y"], np.float32), kat["name"] + " y")
        assert_index_equal(layer.argmax.cpu().numpy(), np.array(kat["argmax"]), kat["name"] + " argmax")
        assert_index_equal(layer.argmin.cpu().numpy(), np.array(kat["argmin"]), kat["name"] + " argmin")


@pytest.mark.parametrize("B,C,L,Fo,k,stride", [(3, 5, 40, 7, 3, 1), (2, 33, 70, 65, 5, 2), (1, 1, 9, 1, 9, 1),
                                               (4, 16, 128, 32, 4, 3)])
def test_conv1d_forward_and_backward(B, C, L, Fo, k, stride):
    g = torch.Generator().manual_seed(B * 100 + k)
    x = torch.randn(B, C, L, generator=g)
    w = torch.randn(Fo, C, k, generator=g)
    bias = torch.randn(Fo, generator=g)
    want = oracle.conv_forward(x.numpy()[:, :, None, :], w.numpy()[:, :, None, :], (1, stride), bias.numpy())
    layer = _conv1d(w, bias, stride=stride)
    xd = x.to(DEV).requires_grad_(True)
    y = layer(xd)
    assert_bits_equal(y.detach().cpu().numpy(), want[0][:, :, 0], "conv1d y")
    assert_index_equal(layer.argmax.cpu().numpy(), want[1][:, :, 0], "conv1d argmax")
    assert_index_equal(layer.argmin.cpu().numpy(), want[2][:, :, 0], "conv1d argmin")
    if B * Fo * L * k * C > 400000:
        return
    grad = torch.randn(y.shape, generator=g)
    y.backward(grad.to(DEV))
    xg, wg = brute.conv_backward(x.numpy()[:, :, None, :], w.numpy()[:, :, None, :], grad.numpy()[:, :, None, :],
                                 want[1], want[2], (1, stride))
    xa, wa = brute.conv_backward(x.abs().numpy()[:, :, None, :], w.abs().numpy()[:, :, None, :],
                                 grad.abs().numpy()[:, :, None, :], want[1], want[2], (1, stride))
    for got, wanted, floor, name in ((xd.grad, xg[:, :, 0], xa[:, :, 0], "x_grad"),
                                     (layer.weight.grad, wg[:, :, 0], wa[:, :, 0], "w_grad")):
        err = np.abs(got.cpu().numpy().astype(np.float64) - wanted)
        assert (err <= 1e-5 * np.abs(wanted) + 2.0 ** -22 * floor + 1e-30).all(), name
    np.testing.assert_allclose(layer.bias.grad.cpu().numpy(), grad.sum(dim=(0, 2)).numpy(), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("B,C,H,W,Fo,k1,k2,stride", [(2, 3, 6, 7, 4, 2, 3, (1, 1)), (1, 8, 12, 10, 5, 3, 3, (2, 1)),
                                                     (2, 4, 9, 9, 3, 1, 2, (1, 2)), (3, 32, 14, 14, 64, 3, 3, 1)])
def test_conv2d_forward_and_backward(B, C, H, W, Fo, k1, k2, stride):
    g = torch.Generator().manual_seed(H * 10 + W)
    x = torch.randn(B, C, H, W, generator=g)
    w = torch.randn(Fo, C, k1, k2, generator=g)
    st = stride if isinstance(stride, tuple) else (stride, stride)
    want = oracle.conv_forward(x.numpy(), w.numpy(), st)
    layer = _conv2d(w, None, stride=stride)
    xd = x.to(DEV).requires_grad_(True)
    y = layer(xd)
    assert_bits_equal(y.detach().cpu().numpy(), want[0], "conv2d y")
    assert_index_equal(layer.argmax.cpu().numpy(), want[1], "conv2d argmax")
    assert_index_equal(layer.argmin.cpu().numpy(), want[2], "conv2d argmin")
    if y.numel() * k1 * k2 * C > 400000:
        return
    grad = torch.randn(y.shape, generator=g)
    y.backward(grad.to(DEV))
    xg, wg = brute.conv_backward(x.numpy(), w.numpy(), grad.numpy(), want[1], want[2], st)
    xa, wa = brute.conv_backward(x.abs().numpy(), w.abs().numpy(), grad.abs().numpy(), want[1], want[2], st)
    for got, wanted, floor, name in ((xd.grad, xg, xa, "x_grad"), (layer.weight.grad, wg, wa, "w_grad")):
        err = np.abs(got.cpu().numpy().astype(np.float64) - wanted)
        assert (err <= 1e-5 * np.abs(wanted) + 2.0 ** -22 * floor + 1e-30).all(), name


@pytest.mark.parametrize("padding,mode", [(3, "zeros"), ("same", "zeros"), ((2, 1), "replicate"), ("valid", "zeros"),
                                          (4, "reflect")])
def test_conv1d_padding_follows_the_reference(padding, mode):
    """The reference pads with F.pad before its kernel (an int p adds p cells in total, p // 2 on the left)."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 3, 20, generator=g)
    w = torch.randn(4, 3, 5, generator=g)
    layer = _conv1d(w, None, padding=padding, padding_mode=mode)
    pm = "constant" if mode == "zeros" else mode
    if isinstance(padding, tuple):
        xp = F.pad(x, padding, mode=pm)
    elif padding == "same":
        xp = F.pad(x, (2, 2), mode=pm)
    elif padding == "valid":
        xp = x
    else:
        xp = F.pad(x, (padding // 2, padding - padding // 2), mode=pm)
    want = oracle.conv_forward(xp.numpy()[:, :, None, :], w.numpy()[:, :, None, :])
    y = layer(x.to(DEV))
    assert_bits_equal(y.detach().cpu().numpy(), want[0][:, :, 0], "padded conv1d")
    if padding == "same":
        assert y.shape[-1] == x.shape[-1]


@pytest.mark.parametrize("beta", [0.25, 1.0])
def test_mac_blend_of_the_conv_modules(beta):
    """(1 - beta) * Y + beta * conv + bias (mamtorch/nn/backup/mamconv1d.txt:134-140) in that rounding order."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 6, 30, generator=g)
    w = torch.randn(5, 6, 3, generator=g)
    bias = torch.randn(5, generator=g)
    layer = _conv1d(w, bias, stride=2, beta=True)
    layer.beta = beta
    xd = x.to(DEV)
    y = layer(xd)
    mam = torch.tensor(oracle.conv_forward(x.numpy()[:, :, None, :], w.numpy()[:, :, None, :], (1, 2))[0][:, :, 0]).to(DEV)
    yb = F.conv1d(xd, w.to(DEV), stride=2)
    ref = (1 - beta) * mam + beta * yb + bias.to(DEV)[None, :, None]
    assert torch.equal(y, ref)
    x2 = torch.randn(2, 3, 8, 9, generator=g)
    w2 = torch.randn(4, 3, 2, 2, generator=g)
    l2 = _conv2d(w2, None, beta=True)
    l2.beta = beta
    y2 = l2(x2.to(DEV))
    mam2 = torch.tensor(oracle.conv_forward(x2.numpy(), w2.numpy())[0]).to(DEV)
    assert torch.equal(y2, (1 - beta) * mam2 + beta * F.conv2d(x2.to(DEV), w2.to(DEV)))


def test_selection_counts_follow_the_literal_rule():
    """mamtorch/nn/backup/mamconv2d.txt:86-113 restated: two advanced-index `+= 1` (duplicates count once
    per call), the index decoded as channel = arg % C, element = arg // C, row = element % k1, column =
    element // k1; max and min go to their own counters."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 4, 9, 8, generator=g)
    w = torch.randn(6, 4, 2, 3, generator=g)
    layer = _conv2d(w, None)
    want_max = torch.zeros(w.shape, dtype=torch.int32)
    want_min = torch.zeros(w.shape, dtype=torch.int32)
    for rep in range(2):
        layer(x.to(DEV) * (rep + 1))
        layer.update_selection_count()
        for arg, counter in ((layer.argmax.cpu(), want_max), (layer.argmin.cpu(), want_min)):
            nb, nf, n1, n2 = arg.shape
            filt = torch.arange(nf).repeat_interleave(n1 * n2).repeat(nb)
            flat = arg.flatten().long()
            chan, elem = flat % w.shape[1], flat // w.shape[1]
            counter[filt, chan, elem % w.shape[2], elem // w.shape[2]] += 1
    assert torch.equal(layer.max_selection_count.cpu(), want_max)
    assert torch.equal(layer.min_selection_count.cpu(), want_min)
    l1 = _conv1d(torch.randn(5, 3, 4, generator=g), None)
    l1(torch.randn(2, 3, 17, generator=g).to(DEV))
    l1.update_selection_count()
    arg = l1.argmax.cpu()
    nb, nf, ne = arg.shape
    filt = torch.arange(nf).repeat_interleave(ne).repeat(nb)
    want = torch.zeros(5, 3, 4, dtype=torch.int32)
    want[filt, arg.flatten().long() % 3, arg.flatten().long() // 3] += 1
    assert torch.equal(l1.max_selection_count.cpu(), want)


def test_window_gather_operators():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 37, 5, 41, generator=g)
    for (k1, k2, s1, s2) in ((2, 3, 1, 2), (1, 4, 1, 1), (5, 1, 2, 3)):
        cols = mt.kernel.v4.im2col(x.to(DEV), k1, k2, s1, s2)
        assert torch.equal(cols.cpu(), torch.tensor(oracle.conv_windows(x.numpy(), k1, k2, s1, s2)))
        gg = torch.randn(cols.shape, generator=g)
        back = mt.kernel.v4.col2im(gg.to(DEV), x.shape, k1, k2, s1, s2)
        # adjoint: <im2col(x), g> = <x, col2im(g)>
        lhs = (cols.double().cpu() * gg.double()).sum().item()
        rhs = (x.double() * back.double().cpu()).sum().item()
        assert abs(lhs - rhs) <= 1e-9 * (cols.double().abs().cpu() * gg.double().abs()).sum().item()
    xs = torch.randn(1, 3, 4, 6, generator=g).to(DEV).requires_grad_(True)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.im2col, (xs, 2, 2, 1, 1))
    c = torch.randn(15, 12, generator=g).to(DEV).requires_grad_(True)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.col2im, (c, 1, 3, 4, 6, 2, 2, 1, 1))
    a = torch.randn(9, 5, generator=g).to(DEV).requires_grad_(True)
    b = torch.randn(9, 5, generator=g).to(DEV).requires_grad_(True)
    bias = torch.randn(5, generator=g).to(DEV).requires_grad_(True)
    torch.library.opcheck(torch.ops.mamtorch_kernel_v4.blend, (a, b, bias, 0.75, 0.25))
    assert torch.equal(mt.kernel.v4.blend(a, b, bias, 0.75, 0.25), (0.75 * a + 0.25 * b) + bias)
