"""Host-side pieces of the LogicLayer API that are not kernels: the eager ("python")
implementation of the relaxed layer, the connectivity initialisers and GradFactor
(reference: difflogic/functional.py)."""
import numpy as np
import torch

# Gate i is true at (a, b) iff bit (3 - 2a - b) of i is set (difflogic/functional.py:7-24).
_CORNER_BITS = ((0, 0, 8), (0, 1, 4), (1, 0, 2), (1, 1, 1))


def bin_op(a, b, i):
    """Real-valued relaxation of gate ``i`` (difflogic/functional.py:26-62): the multilinear
    polynomial that agrees with the gate's truth table on {0,1}^2."""
    if not 0 <= i < 16:
        raise ValueError(i)
    r = torch.zeros_like(a)
    na, nb = 1 - a, 1 - b
    for s, t, bit in _CORNER_BITS:
        if i & bit:
            r = r + (a if s else na) * (b if t else nb)
    return r


def bin_op_s(a, b, i_s):
    """sum_i i_s[..., i] * bin_op(a, b, i) (difflogic/functional.py:65-70), evaluated through
    the four truth-table corners instead of sixteen polynomials."""
    na, nb = 1 - a, 1 - b
    r = torch.zeros_like(a)
    for s, t, bit in _CORNER_BITS:
        sel = [i for i in range(16) if i & bit]
        r = r + i_s[..., sel].sum(-1) * (a if s else na) * (b if t else nb)
    return r


def get_random_connections(in_dim, out_dim, device="cuda"):
    """Balanced random wiring (difflogic/difflogic.py:158-165); draws two permutations from the
    CPU default generator."""
    slots = torch.randperm(2 * out_dim) % in_dim
    c = torch.randperm(in_dim)[slots].reshape(2, out_dim).to(torch.int64)
    return c[0].contiguous().to(device), c[1].contiguous().to(device)


def get_unique_connections(in_dim, out_dim, device="cuda"):
    """Distinct input pairs (difflogic/functional.py:76-124): neighbours (0,1),(2,3).., then
    (1,2),(3,4).., then pairs at growing distance, cut to out_dim and shuffled by one
    permutation from the CPU default generator."""
    assert out_dim * 2 >= in_dim, (
        "The number of neurons ({}) must not be smaller than half of the number of inputs ({}) because otherwise "
        "not all inputs could be used or considered.".format(out_dim, in_dim))
    x = np.arange(in_dim, dtype=np.int64)
    first, second = [x[0::2]], [x[1::2]]

    def total(parts):
        return sum(len(p) for p in parts)

    def trim(parts, n):
        extra = total(parts) - n
        if extra > 0:
            parts[-1] = parts[-1][:len(parts[-1]) - extra]

    m = min(total(first), total(second))
    trim(first, m), trim(second, m)
    if m < out_dim:
        first.append(x[1::2]), second.append(x[2::2])
        m = min(total(first), total(second))
        trim(first, m), trim(second, m)
    offset = 2
    while out_dim > total(first) > offset:
        first.append(x[:-offset]), second.append(x[offset:])
        offset += 1
    if total(first) < out_dim:
        raise AssertionError((total(first), offset, out_dim))
    a = np.concatenate(first)[:out_dim]
    b = np.concatenate(second)[:out_dim]
    perm = torch.randperm(out_dim).numpy()
    return (torch.from_numpy(np.ascontiguousarray(a[perm])).to(device),
            torch.from_numpy(np.ascontiguousarray(b[perm])).to(device))


def build_reverse_index(idx_a, idx_b, in_dim):
    """For every input, the neurons that read it (difflogic/difflogic.py:60-69): CSR arrays
    ``start [in+1]`` and ``idx [2*out]``; within one input's list neurons ascend and a
    neuron's ``a`` slot precedes its ``b`` slot.  A stable sort of the interleaved slots."""
    a = idx_a.detach().cpu().numpy().astype(np.int64)
    b = idx_b.detach().cpu().numpy().astype(np.int64)
    slots = np.stack([a, b], axis=1).reshape(-1)             # a0 b0 a1 b1 ...
    order = np.argsort(slots, kind="stable")
    start = np.zeros(in_dim + 1, dtype=np.int64)
    np.cumsum(np.bincount(slots, minlength=in_dim), out=start[1:])
    return torch.from_numpy(start), torch.from_numpy(order // 2)


class GradFactor(torch.autograd.Function):
    """Identity whose gradient is multiplied by ``f`` (difflogic/functional.py:130-138)."""

    @staticmethod
    def forward(ctx, x, f):
        ctx.f = f
        return x.view_as(x)

    @staticmethod
    def backward(ctx, grad_y):
        return grad_y * ctx.f, None
