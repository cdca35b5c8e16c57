"""Float oracle: the reference's python implementation restated on CPU torch.
Test infrastructure (see oracle/__init__.py).

Two independent statements of the relaxed layer are kept:

* ``layer_forward_sequential``: the 16-term running sum ``r = r + w_i * f_i(a, b)`` over
  batch-major gathers, as difflogic/functional.py:65-70 + difflogic/difflogic.py:102-108.
* ``layer_forward_multilinear``: the multilinear extension of the truth table,
  ``y = sum_{s,t in {0,1}} P_st * a^s (1-a)^(1-s) * b^t (1-b)^(1-t)`` with
  ``P_st = sum_i w_i * TRUTH[i, s, t]``.  This is the closed form that pins the first.

Gradients come from torch autograd on either statement, which is how the reference's
python implementation obtains them.
"""
import torch

from .gates import NUM_GATES, TRUTH, real_gate


def gate_mixture(a, b, w):
    """sum_i w[..., i] * f_i(a, b), accumulated in gate order (functional.py:65-70)."""
    r = torch.zeros_like(a)
    for i in range(NUM_GATES):
        r = r + w[..., i] * real_gate(a, b, i)
    return r


def layer_weights(logits, training: bool, dtype=torch.float32):
    """Per-neuron gate distribution: softmax while training, one-hot argmax in eval
    (difflogic.py:103-107, 123, 128)."""
    if training:
        return torch.nn.functional.softmax(logits, dim=-1).to(dtype)
    return torch.nn.functional.one_hot(logits.argmax(-1), NUM_GATES).to(dtype)


def layer_forward_sequential(x, idx_a, idx_b, w):
    """x [..., in] batch-major, w [out,16] already softmaxed/one-hot -> [..., out]."""
    return gate_mixture(x[..., idx_a], x[..., idx_b], w)


def layer_forward_multilinear(x, idx_a, idx_b, w):
    a, b = x[..., idx_a], x[..., idx_b]
    T = torch.as_tensor(TRUTH, dtype=w.dtype)            # [16, 2, 2]
    P = torch.einsum("oi,ist->ost", w, T)                # [out, 2, 2]
    na, nb = 1 - a, 1 - b
    return P[:, 0, 0] * na * nb + P[:, 0, 1] * na * b + P[:, 1, 0] * a * nb + P[:, 1, 1] * a * b


def group_sum(x, k: int, tau: float):
    """difflogic.py:195-196: contiguous blocks of out/k neurons per class, divided by tau."""
    assert x.shape[-1] % k == 0, (x.shape, k)
    return x.reshape(*x.shape[:-1], k, x.shape[-1] // k).sum(-1) / tau


# --- feature-major entry points with the extension's signatures (difflogic.cpp:45-62) ---

def ext_forward(x_fm, idx_a, idx_b, w):
    """x_fm [in,B] -> y [out,B]."""
    return layer_forward_sequential(x_fm.t(), idx_a, idx_b, w).t().contiguous()


def ext_backward_w(x_fm, idx_a, idx_b, grad_y):
    """d(sum(y*grad_y))/dw, shape [out,16].  The forward is linear in w, so any w serves."""
    out = idx_a.shape[0]
    w = torch.zeros(out, NUM_GATES, dtype=x_fm.dtype, requires_grad=True)
    y = layer_forward_sequential(x_fm.t(), idx_a, idx_b, w)
    (g,) = torch.autograd.grad(y, w, grad_y.t())
    return g


def ext_backward_x(x_fm, idx_a, idx_b, w, grad_y):
    """d(sum(y*grad_y))/dx, shape [in,B] (autograd semantics, also for a[n]==b[n])."""
    xb = x_fm.t().detach().clone().requires_grad_(True)
    y = layer_forward_sequential(xb, idx_a, idx_b, w)
    (g,) = torch.autograd.grad(y, xb, grad_y.t())
    return g.t().contiguous()


class PythonNet:
    """Flatten -> LogicLayer x L -> GroupSum(k, tau) on CPU, python implementation.

    ``layers`` is a list of (idx_a, idx_b, logits) with logits a leaf tensor [out,16].
    ``grad_factor`` scales the gradient flowing into each layer's input
    (functional.py:130-138, applied at difflogic.py:82-83)."""

    def __init__(self, layers, k, tau, grad_factor=1.0):
        self.layers, self.k, self.tau, self.grad_factor = layers, k, tau, grad_factor

    def __call__(self, x, training=True):
        x = x.reshape(x.shape[0], -1)
        for idx_a, idx_b, logits in self.layers:
            if self.grad_factor != 1.0:
                x = _GradScale.apply(x, self.grad_factor)
            x = layer_forward_sequential(x, idx_a, idx_b, layer_weights(logits, training, x.dtype))
        return group_sum(x, self.k, self.tau)


class _GradScale(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, f):
        ctx.f = f
        return x.view_as(x)

    @staticmethod
    def backward(ctx, g):
        return g * ctx.f, None
