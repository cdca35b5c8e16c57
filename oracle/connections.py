"""Connectivity initialisers and the reverse index, restated.  Test infrastructure
(see oracle/__init__.py).

Both initialisers draw from torch's CPU default generator, in the same order and with the
same calls as the reference, so that after ``torch.manual_seed(s)`` they return the index
tensors the reference would (pinned by tests/golden/connections_*.npz).
"""
import numpy as np
import torch


def random_connections(in_dim: int, out_dim: int):
    """difflogic.py:158-165: a balanced random wiring.  Every input appears
    floor/ceil(2*out/in) times over the 2*out slots."""
    assert out_dim * 2 >= in_dim
    slots = torch.randperm(2 * out_dim) % in_dim
    relabel = torch.randperm(in_dim)
    c = relabel[slots].reshape(2, out_dim)
    return c[0].to(torch.int64), c[1].to(torch.int64)


def unique_connections(in_dim: int, out_dim: int):
    """functional.py:76-124: distinct unordered pairs, neighbours first, then growing
    offsets, truncated to out_dim and shuffled by one permutation."""
    assert out_dim * 2 >= in_dim
    x = np.arange(in_dim, dtype=np.int64)

    def clip(u, v):
        m = min(len(u), len(v))
        return u[:m], v[:m]

    a, b = clip(x[0::2], x[1::2])                       # (0,1), (2,3), ...
    if len(a) < out_dim:                                # (1,2), (3,4), ...
        a, b = clip(np.concatenate([a, x[1::2]]), np.concatenate([b, x[2::2]]))
    offset = 2
    while out_dim > len(a) > offset:                    # (i, i+offset)
        a = np.concatenate([a, x[:-offset]])
        b = np.concatenate([b, x[offset:]])
        offset += 1
    assert len(a) >= out_dim, (len(a), offset, out_dim)
    a, b = a[:out_dim], b[:out_dim]
    perm = torch.randperm(out_dim).numpy()
    return torch.from_numpy(a[perm].copy()), torch.from_numpy(b[perm].copy())


def reverse_index(idx_a, idx_b, in_dim: int):
    """difflogic.py:60-69: for every input c the list of neurons reading it, neurons in
    ascending order and, for one neuron, its ``a`` slot before its ``b`` slot.
    Returns (start [in+1], idx [2*out]) int64."""
    a = np.asarray(idx_a, dtype=np.int64)
    b = np.asarray(idx_b, dtype=np.int64)
    lists = [[] for _ in range(in_dim)]
    for y in range(len(a)):
        lists[a[y]].append(y)
        lists[b[y]].append(y)
    start = np.zeros(in_dim + 1, dtype=np.int64)
    start[1:] = np.cumsum([len(l) for l in lists])
    idx = np.array([y for l in lists for y in l], dtype=np.int64)
    return start, idx
