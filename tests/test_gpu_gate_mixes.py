"""The packed path on nets whose gate mix is at an extreme of what the skipping machinery (constant folding,
ignored inputs not fetched, output rows nobody looks at not written, constant neurons left out of the count)
can meet: nothing to skip at all, pass-through gates only, layers that are constant as a whole.  Through
PackBitsTensor and GroupSum as a user runs them, on the streaming plan (layers too wide for the LDS-resident
kernel) and on the LDS-resident kernel, against the oracle's interpreter.  Bit-exact."""
import numpy as np
import pytest
import torch

from oracle import interp
from oracle import packed_oracle as po
from tests.helpers import build_model, random_layers

pytestmark = pytest.mark.gpu

TWO_INPUT = np.array([1, 2, 4, 6, 7, 8, 9, 11, 13, 14], np.uint8)     # the ten gates that look at both inputs
PASS_THROUGH = np.array([3, 5, 10, 12], np.uint8)                      # a, b, not b, not a
CONSTANT = np.array([0, 15], np.uint8)


def _draw(rng, n, kind):
    """Gate ids of one layer of `n` neurons."""
    if kind == "two-input":
        return rng.choice(TWO_INPUT, n)
    if kind == "pass-through":
        return rng.choice(PASS_THROUGH, n)
    if kind == "constant":
        return rng.choice(CONSTANT, n)
    if kind == "zeros":
        return np.zeros(n, np.uint8)
    if kind == "ones":
        return np.full(n, 15, np.uint8)
    if kind == "half pass-through":
        return np.where(rng.random(n) < 0.5, rng.choice(PASS_THROUGH, n), rng.integers(0, 16, n)).astype(np.uint8)
    if kind == "uniform":
        return rng.integers(0, 16, n).astype(np.uint8)
    raise ValueError(kind)


MIXES = {
    # name: the kind of every layer in turn (shorter lists repeat their last entry)
    "two-input gates only": ["two-input"],
    "pass-through gates only": ["pass-through"],
    "half pass-through": ["half pass-through"],
    "constant first layer": ["constant", "uniform"],
    "constant middle layer": ["uniform", "uniform", "constant", "uniform"],
    "all-zero middle layer": ["two-input", "two-input", "zeros", "two-input"],
    "all-ones layer below the top": ["uniform", "uniform", "uniform", "uniform", "ones", "uniform"],
    "constant top layer": ["uniform", "uniform", "uniform", "uniform", "uniform", "constant"],
    "pass-through below two-input": ["pass-through", "two-input", "pass-through", "two-input", "pass-through", "two-input"],
    "everything constant": ["constant"],
}


def _net(rng, F, widths, mix):
    kinds = MIXES[mix]
    layers = random_layers(rng, F, widths)
    return [(a, b, _draw(rng, len(a), kinds[min(i, len(kinds) - 1)]).astype(np.uint8)) for i, (a, b, _) in enumerate(layers)]


@pytest.mark.parametrize("mix", sorted(MIXES))
@pytest.mark.parametrize("shape", ["streaming", "streaming, narrow input", "lds"])
def test_gate_mix_extremes(mix, shape):
    import difflogic_amd as dl
    from difflogic_amd import packbitstensor as pbt
    rng = np.random.default_rng(sum(map(ord, mix + shape)))
    k = 10
    if shape == "lds":
        F, widths, B = 64, [500, 700, 640, 900, 500, 640], 1000
    elif shape == "streaming":
        F, widths, B = 96, [12000, 11000, 12000, 11500, 12000, 10500], 700
    else:
        F, widths, B = 16, [12000, 11000, 12000, 11500, 12000, 10500], 129
    layers = _net(rng, F, widths, mix)
    dims = [F] + widths
    if shape == "lds":
        assert pbt.lds_tail(dims, 16) == len(widths)
    else:
        assert pbt.lds_tail(dims, 16) == 0 and len(pbt.plan_groups(dims, True, 16)) >= 2
    x = rng.random((B, F)) < 0.5
    want = interp.net_eval(x, layers, k)
    model = build_model(F, layers, k).eval()
    for bits in (64, 32):
        with torch.no_grad():
            p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=bits)
            got = model(p)
        assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), want), (mix, shape, bits)
    # `.t` after the layers alone holds every row of the last layer, constant and unobserved ones included
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    with torch.no_grad():
        p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)
        for m in logic:
            p = m(p)
        words = p.t.cpu().numpy()
    y, _ = po.packbits(x.T, 64)
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    assert words.shape == y.shape
    assert np.array_equal(po.groupbitsum(words, words.shape[1] * 64 - B, k), want)
    assert np.array_equal(po.unpackbits(words, B), po.unpackbits(y, B)), (mix, shape)


@pytest.mark.parametrize("mix", sorted(MIXES))
@pytest.mark.parametrize("from_bool", [False, True])
def test_lds_resident_kernel_thinned_and_whole(mix, from_bool):
    """The LDS-resident kernel called directly, with the net thinned for the call (layers that shrink to nothing,
    classes without a neuron left, constants added to the counts) and whole (along the schedules and neuron by
    neuron), on the packed words and on the bool matrix."""
    from difflogic_amd import difflogic_cuda as ext
    rng = np.random.default_rng(sum(map(ord, mix)) + from_bool)
    F, widths, B, k = 48, [300, 1100, 640, 2100, 500, 1280], 64 * 5 + (17 if from_bool else 0), 10
    layers = _net(rng, F, widths, mix)
    x = rng.random((B, F)) < 0.5
    want = interp.net_eval(x, layers, k)
    dev = [tuple(torch.as_tensor(v).cuda() for v in l) for l in layers]
    for kw in (dict(thin=True), dict(), dict(scheduled=False)):
        if from_bool:
            got = ext.eval_net_lds_bool(torch.as_tensor(x).cuda(), dev, k, **kw)
        else:
            words, pad = po.packbits(x.T, 64)
            got = ext.eval_net_lds(torch.as_tensor(words).cuda(), dev, pad, k, **kw)
        assert got is not None and np.array_equal(got.cpu().numpy(), want), (mix, from_bool, kw)


def test_pack_tensor_thins_the_lds_net_by_the_measured_share(monkeypatch):
    """PackBitsTensor runs a net that is resident in LDS thinned when a good part of its gate inputs is ignored
    (uniformly drawn ids) and whole along the schedules when every gate looks at both inputs."""
    import difflogic_amd as dl
    from difflogic_amd import difflogic_cuda as ext
    rng = np.random.default_rng(5)
    F, widths, B, k = 64, [500, 700, 640], 300, 10
    seen = []
    real = ext.eval_net_lds_bool
    monkeypatch.setattr(ext, "eval_net_lds_bool", lambda *a, **kw: seen.append(kw.get("thin")) or real(*a, **kw))
    for mix, thin in (("half pass-through", True), ("two-input gates only", False)):
        layers = _net(rng, F, widths, mix)
        x = rng.random((B, F)) < 0.5
        model = build_model(F, layers, k).eval()
        with torch.no_grad():
            got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64))
        assert np.array_equal(got.cpu().numpy(), interp.net_eval(x, layers, k))
        assert seen and seen[-1] is thin, (mix, seen)


@pytest.mark.parametrize("seed", range(4))
def test_random_nets_with_a_gate_family_drawn_per_layer(seed):
    """Depth, widths (narrow: the LDS-resident kernel, wide: the streaming groups), class count, word width, batch
    AND every layer's gate family drawn at random, so that constant, pass-through and two-input layers meet in
    orders the fixed mixes above do not list."""
    import difflogic_amd as dl
    kinds = ["uniform", "two-input", "pass-through", "half pass-through", "constant", "uniform"]
    rng = np.random.default_rng(7000 + seed)
    for case in range(10):
        depth = int(rng.integers(1, 7))
        k = int(rng.choice([1, 2, 3, 5, 10, 16, 20]))
        F = int(rng.choice([16, 32, 48, 100, 784, 1000]))
        wide = case % 3 == 0
        widths, d = [], F
        for i in range(depth):
            lo = max(k, (d + 1) // 2)
            w = int(rng.integers(lo, max(lo + 1, 14000 if wide else 3000)))
            if i == depth - 1:
                w = max(k, -(-w // k) * k)
            widths.append(w)
            d = w
        B = int(rng.choice([1, 63, 64, 65, 127, 129, 1000, 4096, 8192 + 5]))
        layers = [(a, b, _draw(rng, len(a), kinds[int(rng.integers(0, len(kinds)))]).astype(np.uint8))
                  for a, b, _ in random_layers(rng, F, widths)]
        x = rng.random((B, F)) < 0.5
        want = interp.net_eval(x, layers, k)
        model = build_model(F, layers, k).eval()
        bits = int(rng.choice([8, 16, 32, 64]))
        with torch.no_grad():
            got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=bits)).cpu().numpy()
        assert got.shape == want.shape and np.array_equal(got, want), (seed, case, F, widths, k, bits, B)
