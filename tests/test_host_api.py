"""Host logic of the Python API on CPU: constructor semantics, wiring initialisers against the
reference's fixtures, the reverse index, the eager implementation, state_dict format."""
import os

import numpy as np
import pytest
import torch

import difflogic_amd as dl
from difflogic_amd import functional as F
from oracle import connections as oc
from oracle import float_oracle as fo


def test_constructor_defaults_and_rng_order():
    torch.manual_seed(0)
    layer = dl.LogicLayer(20, 16, device="cpu")
    assert layer.implementation == "python" and layer.connections == "random"
    assert layer.num_neurons == 16 and layer.num_weights == 16 and layer.grad_factor == 1.0
    assert layer.weights.shape == (16, 16) and list(layer.state_dict()) == ["weights"]
    assert repr(layer) == "LogicLayer(20, 16, train)"
    torch.manual_seed(0)
    w = torch.randn(16, 16)                                  # logits first, then the wiring
    a, b = oc.random_connections(20, 16)
    assert torch.equal(layer.weights.detach(), w)
    assert torch.equal(layer.indices[0], a) and torch.equal(layer.indices[1], b)
    with pytest.raises(AssertionError):
        dl.LogicLayer(100, 10, device="cpu")                 # fewer than in/2 neurons
    with pytest.raises(AssertionError):
        dl.LogicLayer(10, 10, device="cpu", connections="dense")
    with pytest.raises(AssertionError):
        dl.LogicLayer(10, 10, device="cpu", implementation="fast")
    assert repr(dl.GroupSum(10, 30.0)) == "GroupSum(k=10, tau=30.0)"


def test_wiring_matches_reference_fixtures(golden_dir):
    conn = np.load(os.path.join(golden_dir, "connections.npz"))
    for key in (str(c) for c in conn["cases"]):
        kind, in_dim, out_dim, seed = key.split("_")
        in_dim, out_dim, seed = int(in_dim), int(out_dim), int(seed)
        torch.manual_seed(seed)
        if kind == "unique":
            a, b = F.get_unique_connections(in_dim, out_dim, "cpu")
        else:
            layer = dl.LogicLayer(in_dim, out_dim, device="cpu", connections="random")
            a, b = layer.indices
        assert np.array_equal(a.numpy(), conn[key + "_a"]) and np.array_equal(b.numpy(), conn[key + "_b"]), key


def test_reverse_index_matches_loop_definition():
    g = torch.Generator().manual_seed(0)
    a = torch.randint(0, 13, (200,), generator=g)
    b = torch.randint(0, 13, (200,), generator=g)
    b[5] = a[5]
    start, idx = F.build_reverse_index(a, b, 13)
    s2, i2 = oc.reverse_index(a.numpy(), b.numpy(), 13)
    assert np.array_equal(start.numpy(), s2) and np.array_equal(idx.numpy(), i2)
    layer = dl.LogicLayer(13, 200, device="cpu", implementation="python")
    layer.set_connections(a, b)
    assert torch.equal(layer.indices[0], a)
    with pytest.raises(ValueError):
        layer.set_connections(a, b + 100)
    with pytest.raises(ValueError):
        layer.set_connections(a[:5], b[:5])


def test_eager_implementation_matches_oracle_and_autograd():
    torch.manual_seed(3)
    layer = dl.LogicLayer(12, 30, device="cpu", grad_factor=1.5).double()
    x = torch.rand(9, 12, dtype=torch.float64, requires_grad=True)
    y = layer(x)
    w = torch.softmax(layer.weights, -1)
    want = fo.layer_forward_sequential(x, layer.indices[0], layer.indices[1], w)
    assert torch.allclose(y, want, atol=1e-14)
    gy = torch.randn_like(y)
    gx, = torch.autograd.grad(y, x, gy, retain_graph=True)
    gx_want, = torch.autograd.grad(want, x, gy)
    assert torch.allclose(gx, 1.5 * gx_want, atol=1e-13)
    layer.eval()
    xb = (torch.rand(9, 12) < 0.5).double()
    hard = layer(xb)
    assert set(hard.unique().tolist()) <= {0.0, 1.0}
    for i in range(16):
        a, b = torch.rand(4, dtype=torch.float64), torch.rand(4, dtype=torch.float64)
        from oracle.gates import real_gate
        assert torch.allclose(F.bin_op(a, b, i), real_gate(a, b, i), atol=1e-15)


def test_group_sum_and_grad_factor():
    gs = dl.GroupSum(3, 2.0, device="cpu")
    x = torch.arange(12.).reshape(1, 12)
    assert torch.equal(gs(x), torch.tensor([[6., 22., 38.]]) / 2)
    with pytest.raises(AssertionError):
        gs(torch.zeros(1, 10))
    t = torch.ones(3, requires_grad=True)
    F.GradFactor.apply(t, 4.0).sum().backward()
    assert torch.equal(t.grad, torch.full((3,), 4.0))


def test_packbits_tensor_is_gpu_only():
    with pytest.raises(NotImplementedError):
        dl.PackBitsTensor(torch.zeros(4, 3, dtype=torch.bool), device="cpu")
    layer = dl.LogicLayer(3, 4, device="cpu").eval()

    class Fake(dl.PackBitsTensor):
        def __init__(self):
            pass
    with pytest.raises(AssertionError):
        layer(Fake())                                        # packed inference needs device='cuda'


def test_group_planner():
    from difflogic_amd.packbitstensor import plan_groups
    for dims, count in [([784] + [64000] * 6, True), ([784] + [8000] * 6, False), ([9216] + [256000] * 4, True),
                        ([100, 200], True), ([100, 200, 300, 400, 500, 600, 700, 800, 900], True), ([5, 5], False)]:
        groups = plan_groups(dims, count)
        assert sum(groups) == len(dims) - 1 and all(1 <= g <= 4 for g in groups)
        if count:
            assert groups[-1] <= 2
    assert plan_groups([7], True) == []
    # a wide net over few inputs: deep first group (its gathers hit in L2); square layers beyond the caches fuse deep as
    # well, since a quarter of the inputs of uniformly drawn gates is never fetched (measured on MI355X, 64000-wide,
    # 16384 words: four layers in one group 4.6 ms, as two pairs 6.5 ms)
    assert plan_groups([784] + [64000] * 6, True)[0] >= 3
    assert plan_groups([64000] * 5, False) == [4]


def test_gate_ids_follow_writes_through_data():
    """The packed path's gate ids are the argmax of the weights as they are now: writes through
    ``weights.data`` do not bump the tensor's version counter, so nothing may be cached on it."""
    torch.manual_seed(3)
    layer = dl.LogicLayer(12, 20, device="cpu")
    before = layer._gate_ids()
    assert before.dtype == torch.uint8 and torch.equal(before.long(), layer.weights.detach().argmax(-1))
    version = layer.weights._version
    new_ids = (before.long() + 5) % 16
    layer.weights.data.copy_(torch.nn.functional.one_hot(new_ids, 16).float())
    assert layer.weights._version == version                       # the write was invisible to autograd ...
    assert torch.equal(layer._gate_ids().long(), new_ids)          # ... and still shows
    layer.weights.data[0, :] = 0
    layer.weights.data[0, 9] = 1
    assert int(layer._gate_ids()[0]) == 9


def test_wiring_cache_lives_and_dies_with_its_tensors():
    import gc

    from difflogic_amd.difflogic_cuda import _WiringCache
    cache = _WiringCache()
    a, b = torch.arange(6), torch.arange(6)
    built = []

    def build():
        built.append(len(built))
        return object()

    v = cache.get((a, b), (7,), build)
    assert cache.get((a, b), (7,), build) is v and built == [0]
    assert cache.get((a, b), (8,), build) is not v and len(cache) == 2       # another in_dim: another entry
    a[0] = 3                                                                 # in-place edit: rebuilt, old entry gone
    v2 = cache.get((a, b), (7,), build)
    assert v2 is not v and len(cache) == 2
    c = a.clone()                                                            # equal values, other tensor
    assert cache.get((c, b), (7,), build) is not v2 and len(cache) == 3
    del a, c
    gc.collect()
    assert len(cache) == 0                                                   # nothing outlives the wiring
    # a new tensor that happens to reuse a freed address is never served a dead tensor's entry
    a = torch.arange(6)
    assert cache.get((a, b), (7,), build) is not v2
