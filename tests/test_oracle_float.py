"""Pins the float oracle's gradients (what backward_w / backward_x are checked against)."""
import numpy as np
import torch

from oracle import float_oracle as fo
from oracle.gates import TRUTH


def _case(seed, in_dim=12, out_dim=30, batch=9, dtype=torch.float64, force_equal=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(in_dim, batch, generator=g, dtype=dtype)
    a = torch.randint(0, in_dim, (out_dim,), generator=g)
    b = torch.randint(0, in_dim, (out_dim,), generator=g)
    if force_equal:
        b[3] = a[3]                      # a neuron wired twice to the same input
    w = torch.softmax(torch.randn(out_dim, 16, generator=g, dtype=dtype), -1)
    gy = torch.randn(out_dim, batch, generator=g, dtype=dtype)
    return x, a, b, w, gy


def test_gradcheck_fp64():
    x, a, b, w, _ = _case(0)
    xb = x.t().clone().requires_grad_(True)
    wl = w.clone().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda xx, ww: fo.layer_forward_sequential(xx, a, b, ww), (xb, wl),
                                    eps=1e-6, atol=1e-6)


def test_backward_w_closed_form():
    # grad_w[n,i] = sum_r gy[n,r] * f_i(a,b): four batch sums and the table's multilinear form
    x, a, b, w, gy = _case(1)
    got = fo.ext_backward_w(x, a, b, gy)
    xa, xb = x[a], x[b]
    S = {(0, 0): (gy * (1 - xa) * (1 - xb)).sum(1), (0, 1): (gy * (1 - xa) * xb).sum(1),
         (1, 0): (gy * xa * (1 - xb)).sum(1), (1, 1): (gy * xa * xb).sum(1)}
    want = torch.stack([sum(float(TRUTH[i, s, t]) * S[(s, t)] for s in (0, 1) for t in (0, 1))
                        for i in range(16)], 1)
    assert torch.allclose(got, want, atol=1e-12)
    assert (got[:, 0] == 0).all()
    assert torch.allclose(got[:, 15], gy.sum(1), atol=1e-12)


def test_backward_x_closed_form_including_a_equal_b():
    # dy/da = (P10-P00) + (P00-P01-P10+P11) b ; dy/db = (P01-P00) + (...) a ; scatter-add to inputs
    x, a, b, w, gy = _case(2)
    got = fo.ext_backward_x(x, a, b, w, gy)
    T = torch.as_tensor(TRUTH, dtype=w.dtype)
    P = torch.einsum("oi,ist->ost", w, T)
    cab = P[:, 0, 0] - P[:, 0, 1] - P[:, 1, 0] + P[:, 1, 1]
    da = (P[:, 1, 0] - P[:, 0, 0])[:, None] + cab[:, None] * x[b]
    db = (P[:, 0, 1] - P[:, 0, 0])[:, None] + cab[:, None] * x[a]
    want = torch.zeros_like(x)
    want.index_add_(0, a, gy * da)
    want.index_add_(0, b, gy * db)
    assert torch.allclose(got, want, atol=1e-12)


def test_group_sum_blocks_are_contiguous():
    x = torch.arange(24, dtype=torch.float32).reshape(2, 12)
    y = fo.group_sum(x, 3, 2.0)
    assert y.shape == (2, 3)
    assert torch.equal(y[0], torch.tensor([0 + 1 + 2 + 3, 4 + 5 + 6 + 7, 8 + 9 + 10 + 11.]) / 2)


def test_python_net_grad_factor_scales_input_grads():
    torch.manual_seed(0)
    layers = []
    d = 8
    for o in (16, 16, 20):
        layers.append((torch.randint(0, d, (o,)), torch.randint(0, d, (o,)),
                       torch.randn(o, 16, dtype=torch.float64, requires_grad=True)))
        d = o
    x = torch.rand(5, 8, dtype=torch.float64, requires_grad=True)
    y1 = fo.PythonNet(layers, 4, 3.0, 1.0)(x).square().sum()
    g1 = torch.autograd.grad(y1, [x] + [l[2] for l in layers])
    y2 = fo.PythonNet(layers, 4, 3.0, 2.0)(x).square().sum()
    g2 = torch.autograd.grad(y2, [x] + [l[2] for l in layers])
    assert torch.allclose(y1, y2)
    # the input passes 3 scalings, layer i's logits pass (L-1-i)
    assert torch.allclose(g2[0], g1[0] * 8)
    for i, (u, v) in enumerate(zip(g1[1:], g2[1:])):
        assert torch.allclose(v, u * 2.0 ** (2 - i))
