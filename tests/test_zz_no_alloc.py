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
        out = torch.full((W * 64 - pad, k), -1, dtype=torch.int32, device="cuda")
        out2 = torch.empty_like(out)
        # one call ahead of the measurement: the first call on a device looks the scratch array's address up
        ext.eval_fused_groupbitsum_noalloc(xd, dev_layers, pad, k, out2)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]              # the driver's view: sees a hipMalloc inside the library too
        got = ext.eval_fused_groupbitsum_noalloc(xd, dev_layers, pad, k, out)
        got2 = ext.eval_fused_groupbitsum_noalloc(xd, dev_layers, pad, k, out2, order)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before      # nothing through torch's allocator
        assert torch.cuda.mem_get_info()[0] == free_before                          # and nothing behind its back
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


def test_noalloc_first_call_on_a_device_is_refused_under_graph_capture():
    """The first call on a device looks the scratch array's address up with a runtime call, which must not happen
    while the stream is being captured: DL_ERR_CAPTURING then, and the same call works once one call was made
    outside a capture.  In a process of its own, where no call has been made yet."""
    import os
    import subprocess
    import sys
    code = r'''
import numpy as np, torch
from difflogic_amd import difflogic_cuda as ext
rng = np.random.default_rng(1)
dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
layers = [(dev(rng.integers(0, 50, 640)), dev(rng.integers(0, 50, 640)), dev(rng.integers(0, 16, 640).astype(np.uint8)))]
x = dev(rng.integers(0, 1 << 62, (50, 4), dtype=np.int64))
out = torch.empty((256, 10), dtype=torch.int32, device="cuda")
want = ext.eval_fused_groupbitsum(x, layers, 0, 10)
torch.cuda.synchronize()
stream = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
try:
    with torch.cuda.graph(graph, stream=stream):
        ext.eval_fused_groupbitsum_noalloc(x, layers, 0, 10, out)
    print("NOT REFUSED")
except RuntimeError as e:
    print("REFUSED:", e)
torch.cuda.synchronize()
ext.eval_fused_groupbitsum_noalloc(x, layers, 0, 10, out)          # outside a capture: looks the address up
graph = torch.cuda.CUDAGraph()
out.fill_(-1)
with torch.cuda.graph(graph, stream=stream):
    ext.eval_fused_groupbitsum_noalloc(x, layers, 0, 10, out)
graph.replay()
torch.cuda.synchronize()
print("REPLAY EQUAL:", bool(torch.equal(out, want)))
'''
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "REFUSED: " in proc.stdout and "graph capture" in proc.stdout, proc.stdout
    assert "REPLAY EQUAL: True" in proc.stdout, proc.stdout
