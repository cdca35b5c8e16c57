"""The allocation-free entry point dl_logic_eval_fused_groupbitsum_noalloc (static device scratch
inside the library) against the allocating dl_logic_eval_fused_groupbitsum and the CPU oracle,
through the C ABI.  Bit-exact: every comparison is equality."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import packed_oracle as po
from tests.helpers import random_layers

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda()


def _case(rng, in_dim, widths, W):
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, (in_dim, W), dtype=np.int64, endpoint=True)
    layers = random_layers(rng, in_dim, widths)
    dev_layers = [(_dev(a), _dev(b), _dev(op)) for a, b, op in layers]
    return x, layers, dev_layers


def _oracle(x, layers, pad, k):
    y = x
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    return po.groupbitsum(y, pad, k)


def test_noalloc_matches_allocating_entry_point_twice_in_a_row():
    """Two calls in a row share the GPU's static scratch; the second is smaller than the first, so
    stale contents of the first call's tables and counters lie behind everything it writes."""
    from difflogic_amd import difflogic_cuda as ext
    rng = np.random.default_rng(77)
    # (in_dim, widths, words, k, pad): a two-layer tail with 16-byte lanes, then a smaller one-layer
    # tail with 8-byte lanes and a ragged batch
    for in_dim, widths, W, k, pad in [(784, [8000, 8000], 130, 10, 5), (50, [640], 33, 10, 63)]:
        x, layers, dev_layers = _case(rng, in_dim, widths, W)
        xd = _dev(x)
        want = ext.eval_fused_groupbitsum(xd, dev_layers, pad, k)
        order = ext.count_order_for(dev_layers, in_dim, k)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        out = torch.full((W * 64 - pad, k), -1, dtype=torch.int32, device="cuda")
        mid = torch.cuda.memory_stats()["allocation.all.allocated"]
        got = ext.eval_fused_groupbitsum_noalloc(xd, dev_layers, pad, k, out)
        got2 = ext.eval_fused_groupbitsum_noalloc(xd, dev_layers, pad, k, torch.empty_like(out), order)
        after = torch.cuda.memory_stats()["allocation.all.allocated"]
        assert mid - before == 1 and after - mid == 1          # torch allocated only the two `out` tensors
        assert got is out and torch.equal(got, want) and torch.equal(got2, want)
        assert np.array_equal(got.cpu().numpy(), _oracle(x, layers, pad, k))


def test_noalloc_rejects_what_does_not_fit():
    from difflogic_amd import _lib
    from difflogic_amd import difflogic_cuda as ext
    rng = np.random.default_rng(5)
    lib = _lib.load()
    # 64000-wide tail on 2^20 samples needs ~0.5 GB of partial counters
    assert lib.dl_logic_eval_fused_groupbitsum_workspace_bytes(2, 64000, 16384, 64, 10) > _lib.DL_STATIC_SCRATCH_BYTES
    x, layers, dev_layers = _case(rng, 40, [64000], 4)
    big = torch.zeros((40, 16384), dtype=torch.int64, device="cuda")
    out = torch.empty((16384 * 64, 10), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="static scratch"):
        ext.eval_fused_groupbitsum_noalloc(big, dev_layers, 0, 10, out)
    # rows that are not whole 64-bit words: no per-layer fallback in this entry point
    x32 = torch.zeros((40, 5), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="size exceeds"):
        ext.eval_fused_groupbitsum_noalloc(x32, dev_layers, 0, 10, torch.empty((160, 10), dtype=torch.int32,
                                                                                device="cuda"))
    null = ctypes.c_void_p(0)
    assert lib.dl_logic_eval_fused_groupbitsum_noalloc(null, 3, null, null, null, null, null, 1, 64, 0, 10, null,
                                                       null) == _lib.DL_ERR_INVALID_ARGUMENT
