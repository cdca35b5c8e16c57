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


def test_fused_adam_counter_steps_for_all_of_its_members_or_none():
    """Parameters updated by one launch share a step counter.  A step on which only some of them have a gradient
    would advance the count of the others as well (torch keeps a step per parameter): that raises; a step on which
    none of them has one is skipped as in torch."""
    import difflogic_amd as dl
    a, b = _params(1, [(10,), (10,)])
    opt = dl.FusedAdam([a, b], lr=0.1)
    a.grad, b.grad = torch.ones_like(a), torch.ones_like(b)
    opt.step()
    b.grad = None
    with pytest.raises(RuntimeError, match="step counter"):
        opt.step()
    a.grad = None
    before = (a.detach().clone(), b.detach().clone())
    opt.step()                                                  # nothing to do
    assert torch.equal(a.detach(), before[0]) and torch.equal(b.detach(), before[1])
    assert float(opt.state[a]["step"]) == 1.0


@pytest.mark.parametrize("saved_by", ["torch.optim.Adam", "FusedAdam"])
def test_fused_adam_resumes_from_a_saved_state(saved_by):
    """load_state_dict of a state saved by torch.optim.Adam (a step per parameter, no shared counter) or by
    FusedAdam itself: training goes on as torch.optim.Adam's does (bias correction from the restored count)."""
    import difflogic_amd as dl
    shapes = [(300, 16), (7,), (4100,)]
    ref = _params(5, shapes)
    first = [p.detach().clone().requires_grad_() for p in ref]
    opt_r = torch.optim.Adam(ref, lr=0.01)
    opt_f = (torch.optim.Adam if saved_by == "torch.optim.Adam" else dl.FusedAdam)(first, lr=0.01)
    g = torch.Generator(device="cuda").manual_seed(9)
    grads = [[torch.randn(s, device="cuda", generator=g) for s in shapes] for _ in range(7)]
    for step in range(3):
        for pr, pf, gr in zip(ref, first, grads[step]):
            pr.grad, pf.grad = gr.clone(), gr.clone()
        opt_r.step()
        opt_f.step()
    ours = [p.detach().clone().requires_grad_() for p in first]
    opt_o = dl.FusedAdam(ours, lr=0.01)
    opt_o.load_state_dict(copy.deepcopy(opt_f.state_dict()))
    for step in range(3, 7):
        for pr, po, gr in zip(ref, ours, grads[step]):
            pr.grad, po.grad = gr.clone(), gr.clone()
        opt_r.step()
        opt_o.step()
        for i, (po, pr) in enumerate(zip(ours, ref)):
            assert _close(po.detach(), pr.detach(), 4e-6), (step, i)
    assert float(opt_o.state[ours[0]]["step"]) == 7.0
    # the three tensors share one rebuilt counter again: one launch
    assert len({opt_o.state[p]["_counter"].data_ptr() for p in ours}) == 1


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
