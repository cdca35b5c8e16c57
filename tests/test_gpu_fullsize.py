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
