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


# ------------------------------------------------------------------------------------------
# fp32 training at BASELINE.json's full sizes (C3: 64000-wide, B = 512, 'unique';
# C5: 128000-wide, B = 1024, 'random', grad_factor 2).  Tolerance as everywhere for fp32:
# |got - want| <= 1e-5 * max|want| + 1e-5 * |want| against the fp64 python formulation.
# ------------------------------------------------------------------------------------------
from oracle import connections as oc          # noqa: E402
from oracle import float_oracle as fo         # noqa: E402

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
    assert _close(gw[S.cuda()], want_gw, 2 * RTOL), name

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

    out, loss, grads = run(rows)
    ref_layers = [(m.indices[0].cpu(), m.indices[1].cpu(), m.weights.detach().cpu().double().requires_grad_())
                  for m in layers]
    net = fo.PythonNet(ref_layers, 10, tau, grad_factor)
    want_out = net(x[rows].cpu().double())
    want_loss = torch.nn.functional.cross_entropy(want_out, labels[rows].cpu(), reduction="sum")
    want_loss.backward()
    assert _close(out[rows], want_out), name
    assert abs(float(loss) - float(want_loss.detach())) <= 1e-5 * abs(float(want_loss.detach())), name
    for i, (got, ref) in enumerate(zip(grads, ref_layers)):
        assert _close(got, ref[2].grad, 4 * RTOL), (name, i)    # through up to 12 layers
    del net, want_out, want_loss, ref_layers

    everything = torch.arange(B, device="cuda")
    out, loss, grads = run(everything)
    out2, loss2, grads2 = run(everything)
    assert torch.equal(out, out2) and torch.equal(loss, loss2), name
    assert all(torch.equal(u, v) for u, v in zip(grads, grads2)), name
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 1 << 40)
    out3, loss3, grads3 = run(everything)
    assert torch.equal(out, out3), name
    for i, (u, v) in enumerate(zip(grads, grads3)):
        assert _close(u, v, 4 * RTOL), (name, i)
