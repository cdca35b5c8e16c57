"""FusedAdam (dl_adam_step through the C ABI) against torch.optim.Adam, which is what the
reference trains with (experiments/main.py:169,179)."""
import copy

import pytest
import torch

pytestmark = pytest.mark.gpu


def _params(seed, shapes):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return [torch.randn(s, device="cuda", generator=g).requires_grad_() for s in shapes]


def _close(a, b, tol):
    if b.numel() == 0:
        return a.numel() == 0
    scale = b.abs().max().clamp_min(1e-30)
    return bool(((a - b).abs() <= tol * scale + tol * b.abs()).all())


@pytest.mark.parametrize("weight_decay", [0.0, 0.05])
def test_fused_adam_matches_torch_adam(weight_decay):
    import difflogic_amd as dl
    # sizes around the 4-element vectors and the 4096-element blocks; an empty tensor; a misaligned view
    shapes = [(8000, 16), (1,), (3,), (4097,), (0,), (4096,), (5, 7, 3)]
    ours = _params(0, shapes)
    base = torch.randn(10001, device="cuda")
    ours.append(base[1:].detach().requires_grad_())            # storage offset 4 bytes: not 16-byte aligned
    ref = [p.detach().clone().requires_grad_() for p in ours]
    kw = dict(lr=0.01, betas=(0.9, 0.999), eps=1e-8, weight_decay=weight_decay)
    opt_o, opt_r = dl.FusedAdam(ours, **kw), torch.optim.Adam(ref, **kw)
    g = torch.Generator(device="cuda").manual_seed(7)
    for step in range(12):
        for po, pr in zip(ours, ref):
            grad = torch.randn(po.shape, device="cuda", generator=g) * (10.0 ** (step % 3 - 1))
            po.grad, pr.grad = grad.clone(), grad.clone()
        opt_o.step()
        opt_r.step()
        for i, (po, pr) in enumerate(zip(ours, ref)):
            # fp32 rounding of two differently ordered evaluations of the same formula
            assert _close(po.detach(), pr.detach(), 2e-6), (step, i)
    for po, pr in zip(ours, ref):
        if po.numel():
            assert _close(opt_o.state[po]["exp_avg"], opt_r.state[pr]["exp_avg"], 2e-6)
            assert _close(opt_o.state[po]["exp_avg_sq"], opt_r.state[pr]["exp_avg_sq"], 2e-6)
    assert float(opt_o.state[ours[0]]["step"]) == 12.0


def test_fused_adam_skips_parameters_without_gradient_and_rejects_other_dtypes():
    import difflogic_amd as dl
    a, b = _params(1, [(10,), (10,)])
    opt = dl.FusedAdam([a, b], lr=0.1)
    a.grad = torch.ones_like(a)
    before = b.detach().clone()
    opt.step()
    assert torch.equal(b.detach(), before) and not torch.equal(a.detach(), before)
    h = torch.zeros(4, device="cuda", dtype=torch.float64, requires_grad=True)
    h.grad = torch.ones_like(h)
    with pytest.raises(RuntimeError):
        dl.FusedAdam([h]).step()
    with pytest.raises(ValueError):
        dl.FusedAdam([a], lr=-1.0)


def test_fused_adam_more_tensors_than_one_launch_takes():
    import difflogic_amd as dl
    n = dl._lib.load().dl_adam_max_tensors() + 5
    ours = _params(2, [(33,)] * n)
    ref = [p.detach().clone().requires_grad_() for p in ours]
    opt_o, opt_r = dl.FusedAdam(ours, lr=0.01), torch.optim.Adam(ref, lr=0.01)
    for _ in range(3):
        for po, pr in zip(ours, ref):
            po.grad = torch.full_like(po, 0.5)
            pr.grad = torch.full_like(pr, 0.5)
        opt_o.step()
        opt_r.step()
    for po, pr in zip(ours, ref):
        assert _close(po.detach(), pr.detach(), 2e-6)


def test_graphed_training_step_with_fused_adam_tracks_eager_torch_adam():
    """Forward + loss + backward + FusedAdam captured as one HIP graph and replayed (the step
    counter advances on the device) against eager steps with torch.optim.Adam."""
    import difflogic_amd as dl
    from difflogic_amd.graphs import GraphedTrainStep
    torch.manual_seed(3)
    model = torch.nn.Sequential(dl.LogicLayer(60, 400, device="cuda"), dl.LogicLayer(400, 400, device="cuda"),
                                dl.GroupSum(10, tau=4.0))
    eager = copy.deepcopy(model)
    loss_fn = torch.nn.CrossEntropyLoss()
    g = torch.Generator(device="cuda").manual_seed(1)
    x = (torch.rand(32, 60, device="cuda", generator=g) < 0.3).float()
    y = torch.randint(0, 10, (32,), device="cuda", generator=g)
    opt_e = torch.optim.Adam(eager.parameters(), lr=0.01)
    graphed = GraphedTrainStep(model, loss_fn, x, y, optimizer=dl.FusedAdam(model.parameters(), lr=0.01), warmup=2)
    for _ in range(2):                                          # the constructor's warm-up steps trained the model
        opt_e.zero_grad(set_to_none=True)
        loss_fn(eager(x), y).backward()
        opt_e.step()
    for rep in range(6):
        lg = graphed.step().item()
        opt_e.zero_grad(set_to_none=True)
        le = loss_fn(eager(x), y)
        le.backward()
        opt_e.step()
        torch.cuda.synchronize()
        assert abs(lg - le.item()) <= 1e-5 * abs(le.item()), (rep, lg, le.item())
    for pg, pe in zip(model.parameters(), eager.parameters()):
        assert _close(pg.detach(), pe.detach(), 1e-5)
