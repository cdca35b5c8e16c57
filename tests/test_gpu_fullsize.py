"""The packed path at BASELINE.json's full sizes.  The CPU oracle cannot evaluate 2^20 samples
of a 384 000-gate net in seconds, so these tests check (1) the oracle on slices of the batch
(first, middle, last word columns), (2) that the fused pipeline equals the per-layer kernels
(an independent code path: six `eval` launches + `groupbitsum`) on the whole batch, and (3)
size-independent properties: batch-permutation equivariance, bounds, a ragged tail."""
import numpy as np
import pytest
import torch

from oracle import interp

pytestmark = pytest.mark.gpu


def _build(dl, F, widths, seed, connections="random"):
    torch.manual_seed(seed)
    mods, d = [torch.nn.Flatten()], F
    for w in widths:
        mods.append(dl.LogicLayer(d, w, connections=connections))
        d = w
    return torch.nn.Sequential(*mods, dl.GroupSum(10, 30.0)).eval()


def _tables(dl, model):
    return [(m.indices[0].cpu().numpy(), m.indices[1].cpu().numpy(),
             m.weights.argmax(-1).cpu().numpy().astype(np.uint8)) for m in model if isinstance(m, dl.LogicLayer)]


def _per_layer(dl, model, x):
    """Reference call sequence of packbits_eval: one eval per layer, then groupbitsum."""
    ext = dl.difflogic_cuda
    t, pad = ext.tensor_packbits_cuda(x.T.contiguous(), 64)
    for m in model:
        if isinstance(m, dl.LogicLayer):
            t = ext.eval(t, m.indices[0], m.indices[1], m.weights.argmax(-1).to(torch.uint8))
    return ext.groupbitsum(t, pad, 10)


@pytest.mark.parametrize("name,F,widths,log2b,thresholds", [
    ("headline 784->6x64000", 784, [64000] * 6, 20, False),
    ("C2 784->6x8000", 784, [8000] * 6, 20, False),
    ("C4 9216->4x256000", 9216, [256000] * 4, 18, True),
])
def test_full_size_packed_inference(name, F, widths, log2b, thresholds):
    import difflogic_amd as dl
    B = 1 << log2b
    model = _build(dl, F, widths, 0)
    g = torch.Generator(device="cuda").manual_seed(1)
    if thresholds:      # 3 thresholds of a uniform image, concatenated on the channel axis
        u = torch.rand(B, F // 3, device="cuda", generator=g)
        x = torch.cat([u > (i + 1) / 4 for i in range(3)], dim=1).contiguous()
    else:
        x = torch.rand(B, F, device="cuda", generator=g) < 0.2
    with torch.no_grad():
        out = model(dl.PackBitsTensor(x, bit_count=64))
    assert out.shape == (B, 10) and out.dtype == torch.int32
    assert int(out.min()) >= 0 and int(out.max()) <= widths[-1] // 10

    # (1) oracle on three slices of the batch
    idx = torch.cat([torch.arange(0, 128), torch.arange(B // 2 - 64, B // 2 + 64), torch.arange(B - 128, B)]).cuda()
    want = interp.net_eval(x[idx].cpu().numpy(), _tables(dl, model), 10, threads=16)
    assert np.array_equal(out[idx].cpu().numpy(), want), name

    # (2) the per-layer kernels on the whole batch
    with torch.no_grad():
        ref = _per_layer(dl, model, x)
    assert torch.equal(out, ref), name
    del ref

    # (3) permuting the batch permutes the result; a ragged prefix equals the prefix of the result
    perm = torch.randperm(B, device="cuda", generator=g)
    with torch.no_grad():
        out_p = model(dl.PackBitsTensor(x[perm].contiguous(), bit_count=64))
        out_r = model(dl.PackBitsTensor(x[:B - 37], bit_count=64))
    assert torch.equal(out_p, out[perm]), name
    assert torch.equal(out_r, out[:B - 37]), name


def _set_gate_ids(dl, model, rng, kinds):
    """Overwrites the model's gate logits with one-hot rows: layer i draws its gate ids from kinds[i]."""
    pools = {"two-input": [1, 2, 4, 6, 7, 8, 9, 11, 13, 14], "pass-through": [3, 5, 10, 12], "constant": [0, 15],
             "uniform": list(range(16)), "half pass-through": [3, 5, 10, 12] * 4 + list(range(16))}
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    with torch.no_grad():
        for m, kind in zip(logic, kinds):
            ids = torch.as_tensor(rng.choice(np.array(pools[kind]), m.out_dim)).cuda()
            m.weights.copy_(torch.nn.functional.one_hot(ids.long(), 16).float())


@pytest.mark.parametrize("mix,kinds", [
    ("two-input gates only", ["two-input"] * 6),                 # nothing to skip anywhere
    ("pass-through gates only", ["pass-through"] * 6),           # one live leaf per tree
    ("half pass-through", ["half pass-through"] * 6),
    ("constant middle layer", ["uniform", "uniform", "constant", "uniform", "uniform", "uniform"]),
    ("constant first layer", ["constant"] + ["uniform"] * 5),
    ("constant layer below the top", ["two-input"] * 4 + ["constant", "two-input"]),
])
def test_full_size_gate_mixes(mix, kinds):
    """The headline net (784 -> 6 x 64000, batch 2^20) with gate mixes at the extremes of what the packed kernels
    skip, through PackBitsTensor on the streaming plan: the oracle on slices of the batch and the per-layer
    kernels (which skip nothing but ignored rows) on the whole batch."""
    import difflogic_amd as dl
    B, F, widths = 1 << 20, 784, [64000] * 6
    model = _build(dl, F, widths, 0)
    _set_gate_ids(dl, model, np.random.default_rng(len(mix)), kinds)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.rand(B, F, device="cuda", generator=g) < 0.2
    with torch.no_grad():
        out = model(dl.PackBitsTensor(x, bit_count=64))
    assert out.shape == (B, 10) and out.dtype == torch.int32
    idx = torch.cat([torch.arange(0, 128), torch.arange(B // 2 - 64, B // 2 + 64), torch.arange(B - 128, B)]).cuda()
    want = interp.net_eval(x[idx].cpu().numpy(), _tables(dl, model), 10, threads=16)
    assert np.array_equal(out[idx].cpu().numpy(), want), mix
    with torch.no_grad():
        ref = _per_layer(dl, model, x)
    assert torch.equal(out, ref), mix
    del ref
    with torch.no_grad():                                        # a second call reuses the cached schedules and plans
        again = model(dl.PackBitsTensor(x[:B - 37], bit_count=64))
    assert torch.equal(again, out[:B - 37]), mix


# ------------------------------------------------------------------------------------------
# fp32 training at BASELINE.json's full sizes (C3: 64000-wide, B = 512, 'unique';
# C5: 128000-wide, B = 1024, 'random', grad_factor 2; C1: 784 -> 4 x 8000, B = 128, 'random', with
# Adam).  Tolerance as everywhere for fp32: |got - want| <= 1e-5 * max|want| + 1e-5 * |want| against
# the fp64 python formulation; parameter gradients (long fp32 sums) are held to the error budget
# of tests.helpers.within_budget: that bound, or the fp32 python formulation's own distance from
# the fp64 value on the same case, whichever is larger.
# ------------------------------------------------------------------------------------------
from oracle import connections as oc          # noqa: E402
from oracle import float_oracle as fo         # noqa: E402
from tests.helpers import within_budget       # noqa: E402

RTOL = 1e-5


def _close(got, want, rtol=RTOL):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    scale = want.abs().max().item()
    return bool(((got - want).abs() <= rtol * scale + rtol * want.abs()).all())


@pytest.mark.parametrize("name,width,B,connections,grad_factor", [
    ("C3 layer", 64000, 512, "unique", 1.0),
    ("C5 layer", 128000, 1024, "random", 2.0),
])
def test_full_size_training_layer(name, width, B, connections, grad_factor, monkeypatch):
    """One square layer at full size, dense gradient: the oracle on slices (sampled neurons for y
    and grad_w, sampled inputs with all their consumers for grad_x), and the layer's chained /
    one-pass kernels against its plain kernels on everything."""
    import difflogic_amd as dl
    torch.manual_seed(3)
    layer = dl.LogicLayer(width, width, connections=connections, grad_factor=grad_factor)
    assert layer._train_schedule() is not None
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.rand(B, width, device="cuda", generator=g).requires_grad_()
    gy = torch.randn(B, width, device="cuda", generator=g)
    y = layer(x)
    (y * gy).sum().backward()
    gw, gx = layer.weights.grad.clone(), x.grad.clone()

    a, b = layer.indices[0].cpu(), layer.indices[1].cpu()
    logits = layer.weights.detach().cpu().double()
    xc, gyc = x.detach().cpu().double(), gy.cpu().double()
    pick = torch.Generator().manual_seed(5)
    S = torch.cat([torch.tensor([0, 1, width - 1]), torch.randint(0, width, (61,), generator=pick)])
    lw = logits[S].clone().requires_grad_()
    want_y = fo.layer_forward_sequential(xc, a[S], b[S], torch.softmax(lw, -1))
    assert _close(y[:, S.cuda()], want_y), name
    want_gw, = torch.autograd.grad(want_y, lw, gyc[:, S])
    lw32 = logits[S].float().requires_grad_()
    y32 = fo.layer_forward_sequential(xc.float(), a[S], b[S], torch.softmax(lw32, -1))
    ref_gw, = torch.autograd.grad(y32, lw32, gyc[:, S].float())
    ok, rep = within_budget(gw[S.cuda()], want_gw, ref_gw)
    assert ok, (name, rep)

    start, idx = oc.reverse_index(a.numpy(), b.numpy(), width)
    C = torch.cat([torch.tensor([0, width - 1]), torch.randint(0, width, (30,), generator=pick)])
    N = torch.as_tensor(np.unique(np.concatenate([idx[start[c]:start[c + 1]] for c in C.tolist()])))
    xr = xc.clone().requires_grad_()
    sub = fo.layer_forward_sequential(xr, a[N], b[N], torch.softmax(logits[N], -1))
    want_gx, = torch.autograd.grad(sub, xr, gyc[:, N])
    assert _close(gx[:, C.cuda()], grad_factor * want_gx[:, C]), name

    # the same layer through the plain kernels (no schedule)
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 1 << 40)
    assert layer._train_schedule() is None
    layer.weights.grad = None
    x.grad = None
    y_plain = layer(x)
    (y_plain * gy).sum().backward()
    assert torch.equal(y, y_plain), name                       # same arithmetic per element
    assert torch.equal(gw, layer.weights.grad), name           # same summation order
    assert _close(gx, x.grad), name                            # same terms, another order


@pytest.mark.parametrize("name,F,width,L,B,tau,connections,grad_factor,n_oracle", [
    ("C3 784->6x64000", 784, 64000, 6, 512, 30.0, "unique", 1.0, 32),
    ("C5 9216->12x128000", 9216, 128000, 12, 1024, 100.0, "random", 2.0, 16),
])
def test_full_size_training_step(name, F, width, L, B, tau, connections, grad_factor, n_oracle, monkeypatch):
    """Whole net, forward + CrossEntropy + backward.  (1) The loss is restricted to a few samples,
    so the fp64 python formulation of the whole net on just those samples gives the expected
    logits and parameter gradients, while every kernel still runs at the full batch.  (2) With the
    loss on all samples: chained / one-pass kernels against the plain ones, and bitwise
    repeatability."""
    import difflogic_amd as dl
    torch.manual_seed(6)
    mods, d = [torch.nn.Flatten()], F
    for _ in range(L):
        mods.append(dl.LogicLayer(d, width, connections=connections, grad_factor=grad_factor))
        d = width
    model = torch.nn.Sequential(*mods, dl.GroupSum(10, tau)).train()
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    g = torch.Generator(device="cuda").manual_seed(7)
    x = (torch.rand(B, F, device="cuda", generator=g) < 0.3).float()
    labels = torch.randint(0, 10, (B,), device="cuda", generator=g)
    rows = torch.cat([torch.arange(n_oracle // 2), torch.arange(B - n_oracle // 2, B)]).cuda()

    def run(select):
        model.zero_grad(set_to_none=True)
        out = model(x)
        loss = torch.nn.functional.cross_entropy(out[select], labels[select], reduction="sum")
        loss.backward()
        return out.detach(), loss.detach(), [m.weights.grad.clone() for m in layers]

    def python_impl(dtype):
        ref = [(m.indices[0].cpu(), m.indices[1].cpu(), m.weights.detach().cpu().to(dtype).requires_grad_())
               for m in layers]
        o = fo.PythonNet(ref, 10, tau, grad_factor)(x[rows].cpu().to(dtype))
        l = torch.nn.functional.cross_entropy(o, labels[rows].cpu(), reduction="sum")
        l.backward()
        return o.detach(), l.detach(), [r[2].grad for r in ref]

    want_out, want_loss, want_grads = python_impl(torch.float64)
    _, _, ref_grads = python_impl(torch.float32)

    def check_against_python(out, loss, grads, what):
        assert _close(out[rows], want_out), (name, what)
        assert abs(float(loss) - float(want_loss)) <= 1e-5 * abs(float(want_loss)), (name, what)
        for i, (got, w64, w32) in enumerate(zip(grads, want_grads, ref_grads)):
            ok, rep = within_budget(got, w64, w32)
            assert ok, (name, what, i, rep)

    check_against_python(*run(rows), "chained / one-pass kernels")

    everything = torch.arange(B, device="cuda")
    out, loss, grads = run(everything)
    out2, loss2, grads2 = run(everything)
    assert torch.equal(out, out2) and torch.equal(loss, loss2), name
    assert all(torch.equal(u, v) for u, v in zip(grads, grads2)), name
    # fuse_for_training: first two layers as one node (C3: the activation between them recomputed), last layer with
    # GroupSum.  Same parameters; the same sums in another order (the fused tail hands a slightly different gradient
    # down to every layer below it).
    plain_model, model = model, dl.fuse_for_training(model).train()
    assert isinstance(model[1], dl.FusedLogicLayerPair) and isinstance(model[-2], dl.FusedLogicLayerGroupSum)
    check_against_python(*run(rows), "fused for training")
    outf, lossf, gradsf = run(everything)
    assert _close(outf, out), name
    # (the gradients are not compared with the unfused run's: the fused tail adds 6400 / 12800 terms per class in
    # another order, and that difference is carried through every layer below; each layer is held to the python
    # formulation's error budget above instead)
    out2f, loss2f, grads2f = run(everything)
    assert torch.equal(outf, out2f) and all(torch.equal(u, v) for u, v in zip(gradsf, grads2f)), name
    model = plain_model
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 1 << 40)
    check_against_python(*run(rows), "plain kernels")
    out3, loss3, grads3 = run(everything)
    assert torch.equal(out, out3), name
    for i, (u, v) in enumerate(zip(grads, grads3)):
        # two fp32 evaluations of the same sums in different orders: each within 1e-5 of the exact
        # value, hence within 2e-5 of each other
        assert _close(u, v, 2 * RTOL), (name, i)


@pytest.mark.parametrize("fused", [False, True], ids=["as written", "fuse_for_training"])
def test_c1_training_steps_with_adam(fused):
    """BASELINE config C1 in full on the HIP path: 784 -> 4 x 8000 -> GroupSum(10, tau 10), B = 128,
    'random' wiring, CrossEntropy, three Adam(lr 0.01) steps (experiments/main.py:169,174-181).
    8000-wide layers run the unchained forward / backward_w / backward_x kernels.  Per step: class
    scores, loss and every layer's gradient against the CPU python implementation in fp64, with the
    fp32 python implementation (what the reference computes) setting the error budget."""
    import difflogic_amd as dl
    torch.manual_seed(0)
    F, width, L, B, k, tau = 784, 8000, 4, 128, 10, 10.0
    mods, d = [torch.nn.Flatten()], F
    for _ in range(L):
        mods.append(dl.LogicLayer(d, width, connections="random"))
        d = width
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    assert all(m._train_schedule() is None for m in layers)
    if fused:                     # head and tail fused (the head only where layers walk their schedules); same parameters
        model = dl.fuse_for_training(model).train()
    g = torch.Generator().manual_seed(1)
    x = (torch.rand(B, F, generator=g) < 0.2).float()
    labels = torch.randint(0, k, (B,), generator=g)

    def python_impl(dtype):
        ws = [m.weights.detach().cpu().to(dtype).requires_grad_() for m in layers]
        net = fo.PythonNet([(m.indices[0].cpu(), m.indices[1].cpu(), w) for m, w in zip(layers, ws)], k, tau)
        return net, ws, torch.optim.Adam(ws, lr=0.01), x.to(dtype)

    refs = {dt: python_impl(dt) for dt in (torch.float64, torch.float32)}
    opt = dl.FusedAdam(model.parameters(), lr=0.01) if fused else torch.optim.Adam(model.parameters(), lr=0.01)
    xd, ld = x.cuda(), labels.cuda()
    for step in range(3):
        res = {}
        for dt, (net, ws, o, xin) in refs.items():
            o.zero_grad()
            out = net(xin)
            loss = torch.nn.functional.cross_entropy(out, labels)
            loss.backward()
            res[dt] = (out.detach(), loss.detach(), [w.grad.clone() for w in ws])
            o.step()
        opt.zero_grad()
        out = model(xd)
        loss = torch.nn.functional.cross_entropy(out, ld)
        loss.backward()
        (o64, l64, g64), (o32, l32, g32) = res[torch.float64], res[torch.float32]
        ok, rep = within_budget(out, o64, o32)
        assert ok, (step, "class scores", rep)
        assert abs(loss.item() - l64.item()) <= max(1e-5 * abs(l64.item()), abs(l32.item() - l64.item())), step
        for i, (m, w64, w32) in enumerate(zip(layers, g64, g32)):
            ok, rep = within_budget(m.weights.grad, w64, w32)
            assert ok, (step, i, rep)
        opt.step()
