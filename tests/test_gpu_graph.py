"""A HIP-graph replay of the training step must reproduce the eager step on every replay,
with eager work and synchronisations between replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _model(dl, seed):
    torch.manual_seed(seed)
    mods, d = [torch.nn.Flatten()], 60
    for w in (400, 400, 300):
        mods.append(dl.LogicLayer(d, w, grad_factor=1.5))
        d = w
    return torch.nn.Sequential(*mods, dl.GroupSum(10, 10.0)).train()


def test_graphed_step_equals_eager_on_every_replay():
    import difflogic_amd as dl
    from difflogic_amd.graphs import GraphedTrainStep
    model = _model(dl, 0)
    loss_fn = torch.nn.CrossEntropyLoss()
    g = torch.Generator(device="cuda").manual_seed(0)
    xs = [(torch.rand(64, 60, device="cuda", generator=g) < 0.3).float() for _ in range(4)]
    ys = [torch.randint(0, 10, (64,), device="cuda", generator=g) for _ in range(4)]

    import copy
    eager = copy.deepcopy(model)                      # same logits and wiring, its own .grad tensors
    graphed = GraphedTrainStep(model, loss_fn, xs[0], ys[0])
    for rep in range(6):
        x, y = xs[rep % 4], ys[rep % 4]
        loss_g = graphed.step(x, y)
        torch.cuda.synchronize()
        # eager work between the replays
        eager.zero_grad(set_to_none=True)
        loss_e = loss_fn(eager(x), y)
        loss_e.backward()
        torch.cuda.synchronize()
        assert torch.equal(loss_g, loss_e.detach()), rep
        for pg, pe in zip(model.parameters(), eager.parameters()):
            assert pg.grad is not None and torch.equal(pg.grad, pe.grad), rep


def test_graphed_step_with_optimizer_tracks_eager_training():
    import copy

    import difflogic_amd as dl
    from difflogic_amd.graphs import GraphedTrainStep
    model = _model(dl, 1)
    eager = copy.deepcopy(model)
    loss_fn = torch.nn.CrossEntropyLoss()
    g = torch.Generator(device="cuda").manual_seed(1)
    x = (torch.rand(32, 60, device="cuda", generator=g) < 0.3).float()
    y = torch.randint(0, 10, (32,), device="cuda", generator=g)
    opt_g = torch.optim.Adam(model.parameters(), lr=0.01, capturable=True)
    opt_e = torch.optim.Adam(eager.parameters(), lr=0.01, capturable=True)
    # the constructor's warm-up steps train the model too: keep the eager copy in step
    graphed = GraphedTrainStep(model, loss_fn, x, y, optimizer=opt_g, warmup=2)
    for _ in range(3):                                # 2 warm-ups + the captured (not executed) step is not run
        pass
    losses_g, losses_e = [], []
    for _ in range(2):
        opt_e.zero_grad(set_to_none=True)
        loss_fn(eager(x), y).backward()
        opt_e.step()
    for rep in range(5):
        losses_g.append(graphed.step().item())
        opt_e.zero_grad(set_to_none=True)
        le = loss_fn(eager(x), y)
        le.backward()
        opt_e.step()
        losses_e.append(le.item())
        torch.cuda.synchronize()
    assert losses_g == losses_e, (losses_g, losses_e)
    assert losses_g[-1] < losses_g[0]


def test_graphed_step_of_the_fused_model_equals_its_eager_step(monkeypatch):
    """fuse_for_training (first two layers with the inner activation recomputed, last layer with
    GroupSum) captured and replayed: every replay reproduces the eager step of the same fused
    model bit for bit, on changing inputs."""
    import copy

    import difflogic_amd as dl
    from difflogic_amd.graphs import GraphedTrainStep
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)        # layers this narrow walk their schedules too
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    monkeypatch.setattr(dl.difflogic_cuda, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)
    base = _model(dl, 2)
    model = dl.fuse_for_training(base).train()
    eager = dl.fuse_for_training(copy.deepcopy(base)).train()
    assert isinstance(model[1], dl.FusedLogicLayerPair) and isinstance(model[-2], dl.FusedLogicLayerGroupSum)
    loss_fn = torch.nn.CrossEntropyLoss()
    g = torch.Generator(device="cuda").manual_seed(0)
    xs = [(torch.rand(64, 60, device="cuda", generator=g) < 0.3).float() for _ in range(3)]
    ys = [torch.randint(0, 10, (64,), device="cuda", generator=g) for _ in range(3)]
    graphed = GraphedTrainStep(model, loss_fn, xs[0], ys[0])
    for rep in range(5):
        x, y = xs[rep % 3], ys[rep % 3]
        loss_g = graphed.step(x, y)
        torch.cuda.synchronize()
        eager.zero_grad(set_to_none=True)
        loss_e = loss_fn(eager(x), y)
        loss_e.backward()
        torch.cuda.synchronize()
        assert torch.equal(loss_g, loss_e.detach()), rep
        for pg, pe in zip(model.parameters(), eager.parameters()):
            assert pg.grad is not None and torch.equal(pg.grad, pe.grad), rep


@pytest.mark.parametrize("F,widths,k,B", [(64, [512, 512, 320], 10, 1000), (784, [12000, 12000, 12000], 10, 4096),
                                          (48, [96, 48], 4, 77), (784, [40000, 40000], 10, 1024)])
def test_graphed_packed_inference_equals_eager_on_every_replay(F, widths, k, B):
    """Packing, gate layers and count captured once (the narrow nets run resident in LDS, the wide ones
    stream) and replayed on new batches, with eager work and synchronisation between the replays; every
    replay equals the eager result and the bitwise oracle.  Gate weights changed in place are picked up."""
    import numpy as np
    import difflogic_amd as dl
    from difflogic_amd.graphs import GraphedPackedInference
    from oracle import interp
    from tests.helpers import build_model, random_layers
    rng = np.random.default_rng(F + B)
    layers = random_layers(rng, F, widths)
    model = build_model(F, layers, k).eval()
    xs = [torch.as_tensor(rng.random((B, F)) < p).cuda() for p in (0.2, 0.5, 0.8, 0.35)]
    graphed = GraphedPackedInference(model, xs[0], bit_count=32)
    for i, x in enumerate(xs):
        got = graphed(x).clone()
        with torch.no_grad():
            eager = model(dl.PackBitsTensor(x, bit_count=32))
        torch.cuda.synchronize()
        assert torch.equal(got, eager), i
        if B <= 1024 or i == 0:
            assert np.array_equal(got.cpu().numpy(), interp.net_eval(x.cpu().numpy(), layers, k)), i
    # another gate table in the same storage: the graph reads the weights at replay time
    last = [m for m in model if isinstance(m, dl.LogicLayer)][-1]
    with torch.no_grad():
        last.weights.copy_(torch.randn_like(last.weights))
    got = graphed(xs[1]).clone()
    with torch.no_grad():
        eager = model(dl.PackBitsTensor(xs[1], bit_count=32))
    assert torch.equal(got, eager)
