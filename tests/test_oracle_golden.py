"""The oracle against the fixtures that the reference itself produced
(tests/golden/make_golden.py): connectivity per seed and CompiledLogicNet outputs."""
import os

import numpy as np
import pytest
import torch

from oracle import cgen, connections, interp
from oracle import packed_oracle as po


@pytest.fixture(scope="module")
def conn(golden_dir):
    return np.load(os.path.join(golden_dir, "connections.npz"))


@pytest.fixture(scope="module")
def comp(golden_dir):
    return np.load(os.path.join(golden_dir, "compiled.npz"))


def test_connection_fixtures_reproduced_from_seed(conn):
    cases = [str(c) for c in conn["cases"]]
    assert len(cases) == 10
    for key in cases:
        kind, in_dim, out_dim, seed = key.split("_")
        in_dim, out_dim, seed = int(in_dim), int(out_dim), int(seed)
        torch.manual_seed(seed)
        if kind == "unique":
            a, b = connections.unique_connections(in_dim, out_dim)
        else:
            w = torch.randn(out_dim, 16)                 # the layer draws its logits first
            assert np.array_equal(w[0].numpy(), conn[key + "_w00"])
            a, b = connections.random_connections(in_dim, out_dim)
        assert a.dtype == torch.int64 and b.dtype == torch.int64
        assert np.array_equal(a.numpy(), conn[key + "_a"]), key
        assert np.array_equal(b.numpy(), conn[key + "_b"]), key


def test_unique_connections_are_distinct_pairs(conn):
    for key in (str(c) for c in conn["cases"]):
        if key.startswith("unique"):
            a, b = conn[key + "_a"], conn[key + "_b"]
            assert (a != b).all()
            pairs = set(zip(np.minimum(a, b).tolist(), np.maximum(a, b).tolist()))
            assert len(pairs) == len(a)


def test_random_connections_are_balanced():
    torch.manual_seed(0)
    a, b = connections.random_connections(10, 25)
    counts = np.bincount(np.concatenate([a.numpy(), b.numpy()]), minlength=10)
    assert counts.sum() == 50 and counts.min() == 5 and counts.max() == 5


def test_reverse_index_order():
    a = np.array([2, 0, 2, 1]); b = np.array([1, 2, 2, 0])
    start, idx = connections.reverse_index(a, b, 3)
    assert start.tolist() == [0, 2, 4, 8]
    assert idx.tolist() == [1, 3, 0, 3, 0, 1, 2, 2]      # neuron 2 reads input 2 twice: listed twice


def _layers(comp, name):
    F, k, bits, batch, L = (int(v) for v in comp[name + "_meta"])
    layers = [(comp[f"{name}_a{i}"], comp[f"{name}_b{i}"], comp[f"{name}_op{i}"]) for i in range(L)]
    return F, k, bits, batch, layers


def test_compiled_fixtures_all_oracles(comp):
    cases = [str(c) for c in comp["cases"]]
    assert len(cases) == 7
    for name in cases:
        F, k, bits, batch, layers = _layers(comp, name)
        x, want = comp[name + "_x"], comp[name + "_y"]
        assert x.shape == (batch, F) and want.shape == (batch, k) and want.dtype == np.int32
        assert (po.net_eval_bitwise(x, layers, k) == want).all(), name
        assert (po.net_eval_words(x, layers, k, bits) == want).all(), name
        assert (interp.net_eval(x, layers, k) == want).all(), name
        net = cgen.CompiledNet(layers, F, k, bits, opt_level=0)
        assert (net(x) == want).all(), name
