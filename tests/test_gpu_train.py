"""Parity of the training-mode HIP kernels with the float oracle (the python implementation
restated on CPU).

Tolerance: fp32 results must satisfy |got - want| <= 1e-5 * max|want| + 1e-5 * |want|
(1e-5 relative, with the tensor's scale as the floor for entries that cancel to ~0) against the
python implementation evaluated in fp64.  Gradients that are long fp32 sums are held to the
error budget of tests.helpers.within_budget instead: the same bound, or the distance of the
fp32 python implementation itself from the fp64 value on the same case, whichever is larger.
No test widens the 1e-5 beyond that."""
import numpy as np
import pytest
import torch

from oracle import float_oracle as fo
from tests.helpers import build_model, random_layers, within_budget

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def close(got, want, rtol=RTOL):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    scale = want.abs().max().item() if want.numel() else 0.0
    err = (got - want).abs()
    ok = bool((err <= rtol * scale + rtol * want.abs()).all())
    return ok, float(err.max()) / (scale + 1e-300) if want.numel() else 0.0


@pytest.fixture(scope="module")
def ext():
    import difflogic_amd
    return difflogic_amd.difflogic_cuda


def _case(seed, in_dim, out_dim, batch, dtype=torch.float32, equal_pairs=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(in_dim, batch, generator=g, dtype=dtype)
    a = torch.randint(0, in_dim, (out_dim,), generator=g)
    b = torch.randint(0, in_dim, (out_dim,), generator=g)
    if equal_pairs and out_dim > 3:
        b[1] = a[1]
        b[out_dim // 2] = a[out_dim // 2]
    w = torch.softmax(torch.randn(out_dim, 16, generator=g, dtype=dtype), -1)
    gy = torch.randn(out_dim, batch, generator=g, dtype=dtype)
    return x, a, b, w, gy


def _csr(a, b, in_dim):
    from difflogic_amd.functional import build_reverse_index
    return build_reverse_index(a, b, in_dim)


SHAPES = [(5, 9, 1), (12, 30, 7), (20, 40, 64), (33, 100, 256), (64, 130, 260), (50, 77, 513), (16, 40, 2048),
          (8, 6, 5000)]


@pytest.mark.parametrize("in_dim,out_dim,batch", SHAPES)
def test_forward_fp32(ext, in_dim, out_dim, batch):
    x, a, b, w, _ = _case(batch, in_dim, out_dim, batch)
    want = fo.ext_forward(x, a, b, w)
    got = ext.forward(x.cuda(), a.cuda(), b.cuda(), w.cuda())
    ok, err = close(got, want)
    assert ok, err
    want64 = fo.ext_forward(x.double(), a, b, w.double())
    assert close(got, want64)[0]


@pytest.mark.parametrize("in_dim,out_dim,batch", SHAPES)
def test_backward_w_fp32(ext, in_dim, out_dim, batch):
    x, a, b, w, gy = _case(batch + 1, in_dim, out_dim, batch)
    want = fo.ext_backward_w(x, a, b, gy)
    got = ext.backward_w(x.cuda(), a.cuda(), b.cuda(), gy.cuda())
    assert got.shape == (out_dim, 16)
    # the batch sum of B products carries ~sqrt(B) * eps of rounding in either implementation:
    # compare both fp32 results with the fp64 value
    want64 = fo.ext_backward_w(x.double(), a, b, gy.double())
    ok, err = close(got, want64)
    assert ok, (err, close(want, want64)[1])
    assert bool((got[:, 0] == 0).all())


@pytest.mark.parametrize("in_dim,out_dim,batch", SHAPES)
def test_backward_x_fp32(ext, in_dim, out_dim, batch):
    x, a, b, w, gy = _case(batch + 2, in_dim, out_dim, batch)
    start, idx = _csr(a, b, in_dim)
    want64 = fo.ext_backward_x(x.double(), a, b, w.double(), gy.double())
    got = ext.backward_x(x.cuda(), a.cuda(), b.cuda(), w.cuda(), gy.cuda(), start.cuda(), idx.cuda())
    ok, err = close(got, want64)
    assert ok, err
    got2 = ext.backward_x(x.cuda(), a.cuda(), b.cuda(), w.cuda(), gy.cuda(), start.cuda(), idx.cuda(), 2.5)
    assert close(got2, want64 * 2.5)[0]


def test_backward_x_unused_inputs_get_zero(ext):
    x, a, b, w, gy = _case(0, 10, 12, 64, equal_pairs=False)
    a = a.clamp(max=4)
    b = b.clamp(max=4)
    start, idx = _csr(a, b, 10)
    got = ext.backward_x(x.cuda(), a.cuda(), b.cuda(), w.cuda(), gy.cuda(), start.cuda(), idx.cuda())
    assert bool((got[5:] == 0).all())
    assert close(got, fo.ext_backward_x(x.double(), a, b, w.double(), gy.double()))[0]


@pytest.mark.parametrize("dtype,rtol", [(torch.float64, 1e-12), (torch.float16, 4e-3)])
def test_other_dtypes(ext, dtype, rtol):
    in_dim, out_dim, batch = 24, 50, 264
    x, a, b, w, gy = _case(3, in_dim, out_dim, batch, torch.float64)
    start, idx = _csr(a, b, in_dim)
    xq, wq, gq = x.to(dtype), w.to(dtype), gy.to(dtype)
    xr, wr, gr = xq.double(), wq.double(), gq.double()       # the oracle sees the rounded inputs
    y = ext.forward(xq.cuda(), a.cuda(), b.cuda(), wq.cuda())
    assert y.dtype == dtype and close(y, fo.ext_forward(xr, a, b, wr), rtol)[0]
    gw = ext.backward_w(xq.cuda(), a.cuda(), b.cuda(), gq.cuda())
    assert gw.dtype == dtype and close(gw, fo.ext_backward_w(xr, a, b, gr), rtol)[0]
    gx = ext.backward_x(xq.cuda(), a.cuda(), b.cuda(), wq.cuda(), gq.cuda(), start.cuda(), idx.cuda())
    assert gx.dtype == dtype and close(gx, fo.ext_backward_x(xr, a, b, wr, gr), rtol)[0]


def test_backward_is_deterministic(ext):
    x, a, b, w, gy = _case(9, 100, 3000, 512)
    start, idx = _csr(a, b, 100)
    dev = [t.cuda() for t in (x, a, b, w, gy, start, idx)]
    w1 = ext.backward_w(dev[0], dev[1], dev[2], dev[4])
    x1 = ext.backward_x(*dev)
    for _ in range(3):
        assert torch.equal(w1, ext.backward_w(dev[0], dev[1], dev[2], dev[4]))
        assert torch.equal(x1, ext.backward_x(*dev))


def test_one_hot_binary_forward_is_exact(ext):
    rng = np.random.default_rng(4)
    x = torch.as_tensor((rng.random((40, 300)) < 0.5).astype(np.float32))
    (a, b, op), = random_layers(rng, 40, [160])
    w = torch.nn.functional.one_hot(torch.as_tensor(op).long(), 16).float()
    got = ext.forward(x.cuda(), torch.as_tensor(a).cuda(), torch.as_tensor(b).cuda(), w.cuda())
    want = fo.ext_forward(x, torch.as_tensor(a), torch.as_tensor(b), w)
    assert torch.equal(got.cpu(), want)


def test_input_checks(ext):
    x, a, b, w, gy = _case(0, 8, 10, 16)
    with pytest.raises(RuntimeError):
        ext.forward(x, a, b, w)                                     # CPU tensors
    with pytest.raises(RuntimeError):
        ext.forward(x.cuda().t().contiguous().t(), a.cuda(), b.cuda(), w.cuda())   # not contiguous
    with pytest.raises(RuntimeError):
        ext.forward(x.cuda().int(), a.cuda(), b.cuda(), w.cuda())   # dtype
    with pytest.raises(RuntimeError):
        ext.forward(x.cuda(), a.cuda()[:5], b.cuda(), w.cuda())     # table length


@pytest.mark.parametrize("conn,grad_factor,batch", [("random", 1.0, 128), ("unique", 1.0, 100), ("random", 2.0, 36)])
def test_train_step_matches_python_implementation(conn, grad_factor, batch):
    """Flatten -> 4 x LogicLayer -> GroupSum -> CrossEntropy: loss and every gradient against
    the CPU python implementation with the same wiring and logits."""
    import difflogic_amd as dl
    torch.manual_seed(0)
    F, widths, k, tau = 60, [400, 400, 400, 300], 10, 10.0
    mods, d = [torch.nn.Flatten()], F
    for wd in widths:
        mods.append(dl.LogicLayer(d, wd, grad_factor=grad_factor, connections=conn))
        d = wd
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = (torch.rand(batch, F) < 0.2).float()
    labels = torch.randint(0, k, (batch,))

    def python_impl(dtype):
        """(logits, loss, [grad per layer], grad_x) of the CPU python implementation in ``dtype``."""
        lg = [l.weights.detach().cpu().to(dtype).requires_grad_(True) for l in layers]
        net = fo.PythonNet([(l.indices[0].cpu(), l.indices[1].cpu(), w) for l, w in zip(layers, lg)], k, tau, grad_factor)
        xo = x.detach().clone().to(dtype).requires_grad_(True)
        out = net(xo, training=True)
        loss = torch.nn.functional.cross_entropy(out, labels)
        loss.backward()
        return out.detach(), loss.detach(), [w.grad for w in lg], xo.grad

    out32, loss32, gw32, gx32 = python_impl(torch.float32)
    out64, loss64, gw64, gx64 = python_impl(torch.float64)

    xg = x.detach().cuda().requires_grad_(True)
    got_out = model(xg)
    got_loss = torch.nn.functional.cross_entropy(got_out, labels.cuda())
    got_loss.backward()

    assert close(got_out, out64)[0] and close(got_out, out32)[0]
    assert abs(got_loss.item() - loss64.item()) <= RTOL * abs(loss64.item())
    for l, w64, w32 in zip(layers, gw64, gw32):
        ok, rep = within_budget(l.weights.grad, w64, w32)
        assert ok, rep
    ok, rep = within_budget(xg.grad, gx64, gx32)
    assert ok, rep


@pytest.mark.parametrize("seed", range(8))
def test_random_models_train_like_the_python_implementation(seed, monkeypatch):
    """Depth, widths, wiring kind, batch, tau, grad_factor, the kernels' route (plain or along the schedules) and the
    model's form (as written or fuse_for_training) drawn at random: loss and every gradient of one step against the
    CPU python implementation in fp64, with the fp32 python implementation's own distance as the budget."""
    import difflogic_amd as dl
    rng = np.random.default_rng(4200 + seed)
    torch.manual_seed(seed)
    if seed % 2:
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    depth = int(rng.integers(1, 6))
    k = int(rng.choice([2, 5, 10]))
    F = int(rng.choice([20, 64, 200]))
    tau = float(rng.choice([1.0, 10.0, 30.0]))
    grad_factor = float(rng.choice([1.0, 1.5, 2.0]))
    batch = int(rng.choice([1, 7, 32, 100, 128, 260]))
    mods, d, widths = [torch.nn.Flatten()], F, []
    for i in range(depth):
        w = int(rng.integers((d + 1) // 2 + 1, max((d + 1) // 2 + 2, 500)))
        if i == depth - 1:
            w = -(-w // k) * k
        conn = str(rng.choice(["random", "unique"])) if d * (d - 1) // 2 >= w else "random"
        mods.append(dl.LogicLayer(d, w, grad_factor=grad_factor, connections=conn))
        widths.append(w)
        d = w
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = (torch.rand(batch, F) < 0.3).float()
    labels = torch.randint(0, k, (batch,))
    want_gx = bool(rng.random() < 0.5)
    net_gpu = dl.fuse_for_training(model).train() if seed % 4 >= 2 else model

    def python_impl(dtype):
        lg = [l.weights.detach().cpu().to(dtype).requires_grad_(True) for l in layers]
        net = fo.PythonNet([(l.indices[0].cpu(), l.indices[1].cpu(), w) for l, w in zip(layers, lg)], k, tau, grad_factor)
        xo = x.detach().clone().to(dtype).requires_grad_(True)
        out = net(xo, training=True)
        loss = torch.nn.functional.cross_entropy(out, labels)
        loss.backward()
        return out.detach(), loss.detach(), [w.grad for w in lg], xo.grad

    out32, loss32, gw32, gx32 = python_impl(torch.float32)
    out64, loss64, gw64, gx64 = python_impl(torch.float64)
    xg = x.detach().cuda().requires_grad_(want_gx)
    got_out = net_gpu(xg)
    got_loss = torch.nn.functional.cross_entropy(got_out, labels.cuda())
    got_loss.backward()
    what = (seed, F, widths, k, tau, grad_factor, batch)
    ok, rep = within_budget(got_out, out64, out32)
    assert ok, (what, rep)
    assert abs(got_loss.item() - loss64.item()) <= RTOL * abs(loss64.item()) + 1e-7, what
    for l, w64, w32 in zip(layers, gw64, gw32):
        ok, rep = within_budget(l.weights.grad, w64, w32)
        assert ok, (what, rep)
    if want_gx:
        ok, rep = within_budget(xg.grad, gx64, gx32)
        assert ok, (what, rep)


def test_eval_mode_and_state_dict_round_trip():
    import difflogic_amd as dl
    torch.manual_seed(1)
    m1 = torch.nn.Sequential(torch.nn.Flatten(), dl.LogicLayer(30, 64), dl.LogicLayer(64, 40), dl.GroupSum(4, 2.0))
    assert list(m1.state_dict().keys()) == ["1.weights", "2.weights"]
    torch.manual_seed(2)
    m2 = torch.nn.Sequential(torch.nn.Flatten(), dl.LogicLayer(30, 64), dl.LogicLayer(64, 40), dl.GroupSum(4, 2.0))
    m2.load_state_dict(m1.state_dict())
    for l1, l2 in ((m1[1], m2[1]), (m1[2], m2[2])):
        l2.set_connections(*l1.indices)
    x = (torch.rand(17, 30) < 0.5).float().cuda()
    m1.eval(), m2.eval()
    with torch.no_grad():
        y1, y2 = m1(x), m2(x)
    assert torch.equal(y1, y2)
    layers = [(l.indices[0].cpu(), l.indices[1].cpu(), l.weights.detach().cpu()) for l in (m1[1], m1[2])]
    want = fo.PythonNet(layers, 4, 2.0)(x.cpu(), training=False)
    assert torch.equal(y1.cpu(), want)


@pytest.mark.parametrize("out_dim,batch,k", [(30, 1, 3), (640, 100, 10), (64000, 512, 10), (8000, 128, 10), (77, 260, 7),
                                             (1200, 2048, 2), (40, 5000, 1)])
def test_group_sum_feature_major(ext, out_dim, batch, k):
    g = torch.Generator().manual_seed(out_dim + batch)
    x = torch.rand(out_dim, batch, generator=g)
    tau = 3.5
    want = fo.group_sum(x.double().t(), k, tau)
    got = ext.group_sum_forward(x.cuda(), k, tau)
    assert got.shape == (batch, k)
    ok, err = close(got, want)
    assert ok, err
    assert torch.equal(got, ext.group_sum_forward(x.cuda(), k, tau))           # deterministic
    gy = torch.randn(batch, k, generator=g)
    gx = ext.group_sum_backward(gy.cuda(), out_dim, tau)
    want_gx = (gy.double() / tau).t().repeat_interleave(out_dim // k, dim=0)
    assert gx.shape == (out_dim, batch) and close(gx, want_gx)[0]


def test_group_sum_module_uses_feature_major_path_and_matches_torch():
    import difflogic_amd as dl
    gs = dl.GroupSum(10, 30.0)
    y_fm = torch.rand(640, 96, device="cuda", requires_grad=True)
    out = gs(y_fm.transpose(0, 1))
    ref = y_fm.detach().t().reshape(96, 10, 64).sum(-1) / 30.0
    assert close(out, ref)[0]
    out.square().sum().backward()
    want = (2 * ref / 30.0).t().repeat_interleave(64, dim=0)
    assert close(y_fm.grad, want)[0]
    # a plain [B, out] tensor still takes the generic path
    z = torch.rand(96, 640, device="cuda")
    assert close(gs(z), z.reshape(96, 10, 64).sum(-1) / 30.0)[0]
    with pytest.raises(ValueError):
        dl.difflogic_cuda.group_sum_forward(torch.rand(7, 4, device="cuda"), 2, 1.0)


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-5), (torch.float64, 1e-12)])
@pytest.mark.parametrize("in_dim,out_dim,batch", [(12, 30, 7), (33, 100, 256), (50, 77, 513), (16, 40, 2048)])
def test_logits_entry_points(ext, dtype, rtol, in_dim, out_dim, batch):
    """forward_logits / backward_logits = softmax + forward / backward_w + softmax backward."""
    g = torch.Generator().manual_seed(batch)
    x = torch.rand(in_dim, batch, generator=g, dtype=torch.float64)
    a = torch.randint(0, in_dim, (out_dim,), generator=g)
    b = torch.randint(0, in_dim, (out_dim,), generator=g)
    logits = (3 * torch.randn(out_dim, 16, generator=g, dtype=torch.float64)).requires_grad_(True)
    gy = torch.randn(out_dim, batch, generator=g, dtype=torch.float64)
    xq, lq, gq = x.to(dtype), logits.detach().to(dtype), gy.to(dtype)
    want_p = torch.softmax(lq.double(), -1)
    want_y = fo.ext_forward(xq.double(), a, b, want_p)
    y, probs = ext.forward_logits(xq.cuda(), a.cuda(), b.cuda(), lq.cuda())
    assert y.dtype == dtype and probs.shape == (out_dim, 16)
    assert close(probs, want_p, rtol)[0] and close(y, want_y, rtol)[0]
    lw = lq.double().clone().requires_grad_(True)
    yy = fo.layer_forward_sequential(xq.double().t(), a, b, torch.softmax(lw, -1))
    want_g, = torch.autograd.grad(yy, lw, gq.double().t())
    got_g = ext.backward_logits(xq.cuda(), a.cuda(), b.cuda(), gq.cuda(), probs)
    if dtype == torch.float32:            # the python formulation in fp32 sets the budget
        l32 = lq.clone().requires_grad_(True)
        y32 = fo.layer_forward_sequential(xq.t(), a, b, torch.softmax(l32, -1))
        ref_g, = torch.autograd.grad(y32, l32, gq.t())
        ok, rep = within_budget(got_g, want_g, ref_g)
        assert ok, rep
    else:
        ok, err = close(got_g, want_g, rtol)
        assert ok, err
    assert torch.equal(got_g, ext.backward_logits(xq.cuda(), a.cuda(), b.cuda(), gq.cuda(), probs))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
@pytest.mark.parametrize("in_dim,out_dim,batch,kind", [(64, 64, 256, "random"), (100, 300, 512, "random"),
                                                       (50, 60, 1024, "unique"), (30, 47, 260, "any"),
                                                       (5, 3, 64, "self"), (40, 90, 4096, "any"), (20, 40, 6, "any")])
def test_chained_training_kernels_are_bit_identical(ext, dtype, in_dim, out_dim, batch, kind):
    from oracle import connections as oc
    g = torch.Generator().manual_seed(in_dim + batch)
    torch.manual_seed(in_dim)
    if kind == "random":
        a, b = oc.random_connections(in_dim, out_dim)
    elif kind == "unique":
        a, b = oc.unique_connections(in_dim, out_dim)
    elif kind == "self":
        a, b = torch.tensor([1, 1, 2]), torch.tensor([1, 1, 2])
    else:
        a, b = torch.randint(0, in_dim, (out_dim,), generator=g), torch.randint(0, in_dim, (out_dim,), generator=g)
    x = torch.rand(in_dim, batch, generator=g).to(dtype).cuda()
    logits = torch.randn(out_dim, 16, generator=g).to(dtype).cuda()
    gy = torch.randn(out_dim, batch, generator=g).to(dtype).cuda()
    a, b = a.cuda(), b.cuda()
    sched = ext.schedule_for(a, b, in_dim)
    y0, p0 = ext.forward_logits(x, a, b, logits)
    y1, p1 = ext.forward_logits(x, a, b, logits, sched)
    g0 = ext.backward_logits(x, a, b, gy, p0)
    g1 = ext.backward_logits(x, a, b, gy, p0, sched)
    if dtype == torch.float16:
        # the fp32 arithmetic is the same, but the compiler may round the final fp32 -> fp16
        # conversion in one step (fused multiply-add with fp16 result) in one kernel and in two in
        # the other: rare last-bit differences are allowed
        for u, v in ((y0, y1), (p0, p1), (g0, g1)):
            diff = (u.float() - v.float()).abs()
            assert float((diff > 0).float().mean()) < 0.01
            assert bool((diff <= 2.0 ** -10 * u.float().abs().clamp(min=2.0 ** -14)).all())
    else:
        assert torch.equal(y0, y1) and torch.equal(p0, p1) and torch.equal(g0, g1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
@pytest.mark.parametrize("in_dim,out_dim,batch,kind", [(64, 64, 256, "random"), (300, 300, 512, "random"),
                                                       (50, 60, 1024, "unique"), (200, 200, 64, "unique"),
                                                       (30, 47, 260, "any"), (5, 3, 64, "self"),
                                                       (40, 20, 16, "sparse"), (20, 40, 8, "any"),
                                                       (40, 90, 4096, "any"), (64, 64, 2052, "random")])
@pytest.mark.parametrize("softmax_backward", [False, True])
def test_fused_chained_backward_matches_separate_kernels(ext, monkeypatch, dtype, in_dim, out_dim, batch, kind,
                                                         softmax_backward):
    from oracle import connections as oc
    monkeypatch.setattr(ext, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)     # exercise the overflow rows on any wiring
    g = torch.Generator().manual_seed(in_dim + batch)
    torch.manual_seed(in_dim)
    if kind == "random":
        a, b = oc.random_connections(in_dim, out_dim)
    elif kind == "unique":
        a, b = oc.unique_connections(in_dim, out_dim)
    elif kind == "self":
        a, b = torch.tensor([1, 1, 2]), torch.tensor([1, 1, 2])
    elif kind == "sparse":                                           # half of the inputs feed no neuron
        a, b = torch.randint(0, in_dim // 2, (out_dim,), generator=g), torch.randint(0, in_dim // 2, (out_dim,),
                                                                                    generator=g)
    else:
        a, b = torch.randint(0, in_dim, (out_dim,), generator=g), torch.randint(0, in_dim, (out_dim,), generator=g)
    x = torch.rand(in_dim, batch, generator=g).to(dtype).cuda()
    w = torch.softmax(torch.randn(out_dim, 16, generator=g), -1).to(dtype).cuda()
    gy = torch.randn(out_dim, batch, generator=g).to(dtype).cuda()
    start, idx = oc.reverse_index(a, b, in_dim)
    a, b = a.cuda(), b.cuda()
    start, idx = torch.as_tensor(start).cuda(), torch.as_tensor(idx).cuda()
    sched = ext.schedule_for(a, b, in_dim)
    scale = 1.5
    both = ext.backward_chained(x, w, gy, sched, scale, softmax_backward=softmax_backward)
    if batch * x.element_size() % 16:                               # rows must be whole 16-byte vectors
        assert both is None
        return
    # rows of 33..256 16-byte vectors are summed in the order of the unfused kernel; shorter rows use
    # 8-byte vectors and longer ones are cut into segments (same terms, another order)
    one_segment = 32 * 16 < batch * x.element_size() <= 256 * 16
    assert both is not None
    gw, gx = both
    want_gx = ext.backward_x(x, a, b, w, gy, start, idx, scale)
    want_gw = ext.backward_logits(x, a, b, gy, w) if softmax_backward else ext.backward_w(x, a, b, gy)
    # grad_w: same arithmetic and, for rows of one segment, the same summation order as the unfused kernels
    if dtype == torch.float16:
        assert close(gw, want_gw.double(), 2e-3)[0]
    elif one_segment:
        assert torch.equal(gw, want_gw)
    else:
        assert close(gw, want_gw.double(), 1e-5 if dtype == torch.float32 else 1e-12)[0]
    # grad_x: the same terms summed in another order
    rtol = {torch.float16: 4e-3, torch.float32: 1e-5, torch.float64: 1e-12}[dtype]
    ok, err = close(gx, want_gx.double(), rtol)
    assert ok, err
    again = ext.backward_chained(x, w, gy, sched, scale, softmax_backward=softmax_backward)
    assert torch.equal(again[0], gw) and torch.equal(again[1], gx)   # deterministic


def test_fused_chained_backward_declines_where_it_does_not_apply(ext):
    from oracle import connections as oc
    torch.manual_seed(3)
    a, b = oc.random_connections(16, 400)                            # degree 50: nearly every row would overflow
    a, b = a.cuda(), b.cuda()
    sched = ext.schedule_for(a, b, 16)
    x, w, gy = torch.rand(16, 64).cuda(), torch.rand(400, 16).cuda(), torch.rand(400, 64).cuda()
    assert ext.backward_chained(x, w, gy, sched) is None
    a, b = oc.random_connections(64, 64)
    a, b = a.cuda(), b.cuda()
    sched = ext.schedule_for(a, b, 64)
    x, w, gy = torch.rand(64, 6).cuda(), torch.rand(64, 16).cuda(), torch.rand(64, 6).cuda()
    assert ext.backward_chained(x, w, gy, sched) is None             # rows are not whole 16-byte vectors
    x, w, gy = torch.rand(64, 16388).cuda(), torch.rand(64, 16).cuda(), torch.rand(64, 16388).cuda()
    assert ext.backward_chained(x, w, gy, sched) is None             # rows longer than 64 KB


def test_layer_uses_schedule_for_wide_inputs():
    import difflogic_amd as dl
    torch.manual_seed(0)
    wide, narrow = dl.LogicLayer(5000, 40000), dl.LogicLayer(100, 40000)
    assert wide._train_schedule() is not None and narrow._train_schedule() is None
    assert dl.LogicLayer(5000, 5000)._train_schedule() is None
    x = torch.rand(64, 5000, device="cuda", requires_grad=True)
    y = wide(x)
    y.square().sum().backward()
    ref = fo.layer_forward_sequential(x.detach().cpu().double(), wide.indices[0].cpu(), wide.indices[1].cpu(),
                                      torch.softmax(wide.weights.detach().cpu().double(), -1))
    assert close(y, ref)[0]
    # the backward pass took the fused chained kernel; compare with autograd through the python formulation
    xr = x.detach().cpu().double().requires_grad_()
    wr = wide.weights.detach().cpu().double().requires_grad_()
    fo.layer_forward_sequential(xr, wide.indices[0].cpu(), wide.indices[1].cpu(),
                                torch.softmax(wr, -1)).square().sum().backward()
    x32 = x.detach().cpu().requires_grad_()
    w32 = wide.weights.detach().cpu().requires_grad_()
    fo.layer_forward_sequential(x32, wide.indices[0].cpu(), wide.indices[1].cpu(),
                                torch.softmax(w32, -1)).square().sum().backward()
    ok, rep = within_budget(x.grad, xr.grad, x32.grad)
    assert ok, rep
    ok, rep = within_budget(wide.weights.grad, wr.grad, w32.grad)
    assert ok, rep
    # eval mode on float inputs takes the chained forward too: exact 0/1 results of the discretised gates
    wide.eval()
    xb = (torch.rand(64, 5000, device="cuda") < 0.5).float()
    ye = wide(xb)
    onehot = torch.nn.functional.one_hot(wide.weights.argmax(-1), 16).double().cpu()
    want = fo.layer_forward_sequential(xb.cpu().double(), wide.indices[0].cpu(), wide.indices[1].cpu(), onehot)
    assert torch.equal(ye.cpu().double(), want) and not ye.requires_grad


def test_chained_layer_matches_the_python_formulation_on_random_wirings(monkeypatch):
    """LogicLayer with its schedule forced on (chained forward, one-pass backward), against the
    fp64 python formulation with autograd, over random wirings of every awkward kind: inputs
    that feed no neuron, many neurons on one input, neurons wired twice to one input, one
    neuron, rows shorter and longer than a wave."""
    import difflogic_amd as dl
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    monkeypatch.setattr(dl.difflogic_cuda, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)
    pick = torch.Generator().manual_seed(99)
    for case in range(40):
        in_dim = int(torch.randint(1, 60, (1,), generator=pick))
        out_dim = int(torch.randint(max(1, (in_dim + 1) // 2), 130, (1,), generator=pick))
        batch = [4, 8, 20, 64, 100, 128, 256, 260, 512, 1024, 1028, 2048][case % 12]
        grad_factor = [1.0, 2.0, 0.5][case % 3]
        layer = dl.LogicLayer(in_dim, out_dim, grad_factor=grad_factor)
        kind = case % 4
        a = torch.randint(0, in_dim, (out_dim,), generator=pick)
        b = torch.randint(0, in_dim, (out_dim,), generator=pick)
        if kind == 1:                                   # a few inputs carry everything
            a, b = a % max(1, in_dim // 4), b % max(1, in_dim // 4)
        elif kind == 2:                                 # self loops
            b = torch.where(torch.rand(out_dim, generator=pick) < 0.3, a, b)
        layer.set_connections(a, b)
        assert layer._train_schedule() is not None
        x = torch.rand(batch, in_dim, generator=pick).cuda().requires_grad_()
        gy = torch.randn(batch, out_dim, generator=pick)
        y = layer(x)
        (y * gy.cuda()).sum().backward()
        xr = x.detach().cpu().double().requires_grad_()
        wr = layer.weights.detach().cpu().double().requires_grad_()
        yr = fo.layer_forward_sequential(xr, a, b, torch.softmax(wr, -1))
        (yr * gy.double()).sum().backward()
        x32 = x.detach().cpu().requires_grad_()
        w32 = layer.weights.detach().cpu().requires_grad_()
        (fo.layer_forward_sequential(x32, a, b, torch.softmax(w32, -1)) * gy).sum().backward()
        tag = (case, in_dim, out_dim, batch, kind)
        assert close(y, yr)[0], tag
        ok, rep = within_budget(layer.weights.grad, wr.grad, w32.grad)
        assert ok, (tag, rep)
        ok, rep = within_budget(x.grad, grad_factor * xr.grad, grad_factor * x32.grad)
        assert ok, (tag, rep)


@pytest.mark.parametrize("along_schedule", [False, True])
@pytest.mark.parametrize("dtype,rtol", [(torch.float16, 4e-3), (torch.float64, 1e-5)])
def test_layer_module_with_half_and_double_activations(dtype, rtol, along_schedule, monkeypatch):
    """The reference's --training-bit-count 16 / 64 (experiments/main.py:19-23,286): the input is
    cast to half / double while the weights stay fp32, so LogicLayer takes the
    softmax-in-torch + LogicLayerCudaFunction route (difflogic/difflogic.py:123-126,205-221).
    Outputs and both gradients against the same formulation on CPU (fp64 arithmetic on the
    values as rounded to ``dtype``, the fp32 softmax and the casts as autograd sees them).
    ``along_schedule``: the layer counts as wide, so the same route runs the kernels that walk the
    wiring along its trails (forward, and both gradients in one pass)."""
    import difflogic_amd as dl
    if along_schedule:
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    torch.manual_seed(5)
    in_dim, out_dim, batch = 48, 120, 264
    layer = dl.LogicLayer(in_dim, out_dim, grad_factor=1.5).train()
    assert (layer._train_schedule() is not None) == along_schedule
    a, b = layer.indices[0].cpu(), layer.indices[1].cpu()
    g = torch.Generator().manual_seed(6)
    x = torch.rand(batch, in_dim, generator=g).to(dtype)
    gy = torch.randn(batch, out_dim, generator=g).to(dtype)

    xg = x.cuda().requires_grad_()
    y = layer(xg)
    assert y.dtype == dtype and y.shape == (batch, out_dim)
    (y * gy.cuda()).sum().backward()
    assert layer.weights.grad.dtype == torch.float32 and xg.grad.dtype == dtype

    w32 = layer.weights.detach().cpu().requires_grad_()
    xr = x.double().requires_grad_()
    wq = torch.softmax(w32, -1).to(dtype).double()
    yr = fo.layer_forward_sequential(xr, a, b, wq)
    (yr * gy.double()).sum().backward()
    assert close(y, yr.to(dtype), rtol)[0]
    ok, err = close(xg.grad, 1.5 * xr.grad, rtol)
    assert ok, err
    ok, err = close(layer.weights.grad, w32.grad, rtol)
    assert ok, err


@pytest.mark.parametrize("dtype,rtol", [(torch.float16, 4e-3), (torch.float64, 1e-5)])
@pytest.mark.parametrize("in_dim,out_dim,batch", [(20, 50, 37), (48, 120, 264), (64, 200, 1040), (30, 64, 4104), (16, 24, 8)])
def test_kernels_take_fp32_weights_beside_half_and_double_activations(ext, dtype, rtol, in_dim, out_dim, batch):
    """DL_F16_W32 / DL_F64_W32 through the bindings: half / double activations and gradients, fp32 logits,
    probabilities and logit gradients, with the softmax and its backward inside the kernels (the reference casts
    the fp32 softmax to the activations' dtype in torch, difflogic/difflogic.py:123-126).  Plain kernels, the kernels
    along the schedule and the one-pass backward, against fp64 arithmetic on the values as rounded to ``dtype``."""
    x, a, b, _, gy = _case(in_dim + batch, in_dim, out_dim, batch, dtype=dtype)
    g = torch.Generator().manual_seed(batch)
    logits = torch.randn(out_dim, 16, generator=g)
    xd, ad, bd, ld, gd = x.cuda(), a.cuda(), b.cuda(), logits.cuda(), gy.cuda()
    sched = ext.schedule_for(ad, bd, in_dim)
    start, idx = _csr(a, b, in_dim)

    l64 = logits.double().requires_grad_()
    x64 = x.double().t().contiguous().requires_grad_()
    y64 = fo.layer_forward_sequential(x64, a, b, torch.softmax(l64, -1))           # [B, out]
    (y64 * gy.double().t()).sum().backward()

    for schedule in (None, sched):
        y, probs = ext.forward_logits(xd, ad, bd, ld, schedule)
        assert y.dtype == dtype and probs.dtype == torch.float32
        assert close(probs, torch.softmax(logits.double(), -1), 2e-6)[0]
        ok, err = close(y, y64.t().to(dtype), rtol)
        assert ok, (schedule is not None, err)
        gl = ext.backward_logits(xd, ad, bd, gd, probs, schedule)
        assert gl.dtype == torch.float32
        ok, err = close(gl, l64.grad, rtol)
        assert ok, (schedule is not None, err)
    gx = ext.backward_x(xd, ad, bd, probs, gd, start.cuda(), idx.cuda(), 1.5)
    assert gx.dtype == dtype
    ok, err = close(gx, 1.5 * x64.grad.t(), rtol)
    assert ok, err
    both = ext.backward_chained(xd, probs, gd, sched, 1.5, softmax_backward=True)
    if both is not None:
        assert both[0].dtype == torch.float32 and both[1].dtype == dtype
        ok, err = close(both[0], l64.grad, rtol)
        assert ok, err
        ok, err = close(both[1], 1.5 * x64.grad.t(), rtol)
        assert ok, err
    # probabilities given instead of logits (the reference's forward), fp32 beside the activations
    ok, err = close(ext.forward(xd, ad, bd, probs), y64.t().to(dtype), rtol)
    assert ok, err
    with pytest.raises(RuntimeError):
        ext.forward(xd.float(), ad, bd, probs.double())           # only fp32 weights may differ from the activations


@pytest.mark.parametrize("in_dim,out_dim,batch,k", [(12, 30, 7, 3), (33, 100, 256, 10), (50, 77, 513, 7), (16, 40, 2048, 2),
                                                    (64, 1300, 260, 10), (20, 64, 64, 1)])
def test_forward_and_backward_fused_with_group_sum(ext, in_dim, out_dim, batch, k):
    """dl_logic_forward_group_sum / dl_logic_backward_*_grouped against the separate kernels (same
    terms, the class sums in another order) and the fp64 python formulation."""
    g = torch.Generator().manual_seed(in_dim + batch)
    x = torch.rand(in_dim, batch, generator=g)
    a = torch.randint(0, in_dim, (out_dim,), generator=g)
    b = torch.randint(0, in_dim, (out_dim,), generator=g)
    b[1] = a[1]
    logits = 2 * torch.randn(out_dim, 16, generator=g)
    gs = torch.randn(batch, k, generator=g)
    tau = 3.5
    xd, ad, bd, ld = x.cuda(), a.cuda(), b.cuda(), logits.cuda()
    start, idx = (t.cuda() for t in _csr(a, b, in_dim))

    sums, probs = ext.forward_group_sum(xd, ad, bd, ld, k, tau)
    y0, p0 = ext.forward_logits(xd, ad, bd, ld)
    assert torch.equal(probs, p0) and sums.shape == (batch, k)
    assert close(sums, ext.group_sum_forward(y0, k, tau))[0]
    lw = logits.double().requires_grad_()
    xr = x.double().t().contiguous().requires_grad_()
    want = fo.group_sum(fo.layer_forward_sequential(xr, a, b, torch.softmax(lw, -1)), k, tau)
    assert close(sums, want)[0]
    assert torch.equal(sums, ext.forward_group_sum(xd, ad, bd, ld, k, tau)[0])           # deterministic

    (want * gs.double()).sum().backward()
    grad_cls = (gs.cuda() / tau).t().contiguous()
    gw, gx = ext.backward_group_sum(xd, ad, bd, probs, grad_cls, start, idx, None, 1.5, True, True)
    gy_full = ext.group_sum_backward(gs.cuda(), out_dim, tau)
    assert close(gw, ext.backward_logits(xd, ad, bd, gy_full, probs))[0]
    assert close(gx, ext.backward_x(xd, ad, bd, probs, gy_full, start, idx, 1.5))[0]
    l32 = logits.clone().requires_grad_()
    x32 = x.t().contiguous().requires_grad_()
    (fo.group_sum(fo.layer_forward_sequential(x32, a, b, torch.softmax(l32, -1)), k, tau) * gs).sum().backward()
    ok, rep = within_budget(gw, lw.grad, l32.grad)
    assert ok, rep
    ok, rep = within_budget(gx, 1.5 * xr.grad.t(), 1.5 * x32.grad.t())
    assert ok, rep
    # along the schedule (one pass): the same gradients
    sched = ext.schedule_for(ad, bd, in_dim)
    if batch % 4 == 0:
        gw2, gx2 = ext.backward_group_sum(xd, ad, bd, probs, grad_cls, start, idx, sched, 1.5, True, True)
        assert close(gw2, gw)[0] and close(gx2, gx)[0]
    only_w, none_x = ext.backward_group_sum(xd, ad, bd, probs, grad_cls, start, idx, sched, 1.5, False, True)
    assert none_x is None and torch.equal(only_w, gw)


@pytest.mark.parametrize("widths,batch,conn,grad_factor,wide", [([400, 400, 300], 128, "random", 1.0, False),
                                                                ([300, 600, 600], 100, "unique", 2.0, False),
                                                                ([500, 500], 64, "random", 1.0, True)])
def test_fuse_group_sum_trains_like_the_unfused_model(widths, batch, conn, grad_factor, wide, monkeypatch):
    """fuse_group_sum(model): same positions, parameters and state_dict keys; in training the same
    class scores, loss and gradients as the unfused model (up to summation order) and as the CPU
    python implementation; eval mode and packed inference unchanged."""
    import difflogic_amd as dl
    if wide:          # the last layer takes the kernels that walk the schedule
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    torch.manual_seed(3)
    F, k, tau = 60, 10, 10.0
    mods, d = [torch.nn.Flatten()], F
    for wd in widths:
        mods.append(dl.LogicLayer(d, wd, grad_factor=grad_factor, connections=conn))
        d = wd
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    fused = dl.fuse_group_sum(model).train()
    assert list(fused.state_dict()) == list(model.state_dict()) and len(fused) == len(model)
    assert isinstance(fused[-2], dl.FusedLogicLayerGroupSum) and fused[-2].weights is model[-2].weights
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = (torch.rand(batch, F) < 0.3).float()
    labels = torch.randint(0, k, (batch,))

    def run(net):
        net.zero_grad(set_to_none=True)
        xg = x.cuda().requires_grad_()
        out = net(xg)
        loss = torch.nn.functional.cross_entropy(out, labels.cuda())
        loss.backward()
        return out.detach(), loss.detach(), [l.weights.grad.clone() for l in layers], xg.grad.clone()

    out0, loss0, gw0, gx0 = run(model)
    out1, loss1, gw1, gx1 = run(fused)
    assert close(out1, out0)[0] and abs(float(loss1) - float(loss0)) <= RTOL * abs(float(loss0))

    def python_impl(dtype):
        lg = [l.weights.detach().cpu().to(dtype).requires_grad_() for l in layers]
        net = fo.PythonNet([(l.indices[0].cpu(), l.indices[1].cpu(), w) for l, w in zip(layers, lg)], k, tau, grad_factor)
        xo = x.detach().clone().to(dtype).requires_grad_()
        o = net(xo)
        torch.nn.functional.cross_entropy(o, labels).backward()
        return o.detach(), [w.grad for w in lg], xo.grad

    o64, w64, x64 = python_impl(torch.float64)
    o32, w32, x32 = python_impl(torch.float32)
    assert close(out1, o64)[0]
    for got, r64, r32 in zip(gw1, w64, w32):
        ok, rep = within_budget(got, r64, r32)
        assert ok, rep
    ok, rep = within_budget(gx1, x64, x32)
    assert ok, rep
    out2, loss2, gw2, gx2 = run(fused)
    assert torch.equal(out1, out2) and all(torch.equal(u, v) for u, v in zip(gw1, gw2)) and torch.equal(gx1, gx2)

    # eval mode: float and packed inference go through the two original modules
    model.eval(), fused.eval()
    with torch.no_grad():
        assert torch.equal(fused(x.cuda()), model(x.cuda()))
        assert torch.equal(fused(dl.PackBitsTensor(x.bool().cuda(), bit_count=64)),
                           model(dl.PackBitsTensor(x.bool().cuda(), bit_count=64)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
@pytest.mark.parametrize("in0,in_dim,out_dim,batch,kind", [(40, 64, 64, 256, "random"), (100, 300, 300, 512, "random"),
                                                           (30, 50, 60, 1024, "unique"), (150, 200, 200, 64, "unique"),
                                                           (20, 30, 47, 260, "any"), (9, 5, 3, 64, "self"),
                                                           (25, 40, 20, 16, "sparse"), (15, 20, 40, 8, "any"),
                                                           (784, 1000, 1200, 128, "random")])
@pytest.mark.parametrize("softmax_lower", [False, True])
def test_chained_backward_with_the_lower_layers_backward_w(ext, monkeypatch, dtype, in0, in_dim, out_dim, batch, kind,
                                                           softmax_lower):
    """dl_logic_backward_chained_lower: grad_w of the layer as the plain one-pass backward gives it,
    and grad_w of the layer below as backward_w / backward_logits give it on the grad_x rows the
    plain pass stores (which this one never writes)."""
    from oracle import connections as oc
    monkeypatch.setattr(ext, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)     # exercise the fix-up rows on any wiring
    g = torch.Generator().manual_seed(in_dim + batch + in0)
    torch.manual_seed(in_dim)
    if kind == "random":
        a, b = oc.random_connections(in_dim, out_dim)
    elif kind == "unique":
        a, b = oc.unique_connections(in_dim, out_dim)
    elif kind == "self":
        a, b = torch.tensor([1, 1, 2]), torch.tensor([1, 1, 2])
    elif kind == "sparse":                                           # half of the inputs feed no neuron
        a, b = torch.randint(0, in_dim // 2, (out_dim,), generator=g), torch.randint(0, in_dim // 2, (out_dim,),
                                                                                    generator=g)
    else:
        a, b = torch.randint(0, in_dim, (out_dim,), generator=g), torch.randint(0, in_dim, (out_dim,), generator=g)
    a0 = torch.randint(0, in0, (in_dim,), generator=g).cuda()
    b0 = torch.randint(0, in0, (in_dim,), generator=g).cuda()
    x0 = torch.rand(in0, batch, generator=g).to(dtype).cuda()
    p0 = torch.softmax(torch.randn(in_dim, 16, generator=g), -1).to(dtype).cuda()
    x = torch.rand(in_dim, batch, generator=g).to(dtype).cuda()
    w = torch.softmax(torch.randn(out_dim, 16, generator=g), -1).to(dtype).cuda()
    gy = torch.randn(out_dim, batch, generator=g).to(dtype).cuda()
    a, b = a.cuda(), b.cuda()
    sched = ext.schedule_for(a, b, in_dim)
    scale = 1.5
    got = ext.backward_chained_lower(x, w, gy, sched, x0, a0, b0, p0, scale, softmax_backward=True,
                                     softmax_backward_lower=softmax_lower)
    plain = ext.backward_chained(x, w, gy, sched, scale, softmax_backward=True)
    if batch * x.element_size() % 16 or batch * x.element_size() > 256 * 16:
        assert got is None                                          # whole 16-byte vectors, rows of at most 4 KB
        return
    assert got is not None and plain is not None
    gw, gw0 = got
    assert torch.equal(gw, plain[0])
    want0 = ext.backward_logits(x0, a0, b0, plain[1], p0) if softmax_lower else ext.backward_w(x0, a0, b0, plain[1])
    # the same terms; the same order of additions too for rows of 33..256 vectors (shorter rows: 8-byte vectors)
    if dtype != torch.float16 and 32 * 16 < batch * x.element_size():
        assert torch.equal(gw0, want0)
    else:
        rtol = {torch.float16: 4e-3, torch.float32: 1e-5, torch.float64: 1e-12}[dtype]
        ok, err = close(gw0, want0.double(), rtol)
        assert ok, err
    again = ext.backward_chained_lower(x, w, gy, sched, x0, a0, b0, p0, scale, softmax_backward=True,
                                       softmax_backward_lower=softmax_lower)
    assert torch.equal(again[0], gw) and torch.equal(again[1], gw0)  # deterministic
    # x left out: its rows are recomputed from the layer below (fp32 / fp64); the same gradients bit for bit when x
    # is what that layer's forward pass gives
    x1 = ext.forward(x0, a0, b0, p0)
    ref = ext.backward_chained_lower(x1, w, gy, sched, x0, a0, b0, p0, scale, softmax_backward=True,
                                     softmax_backward_lower=softmax_lower)
    rec = ext.backward_chained_lower(None, w, gy, sched, x0, a0, b0, p0, scale, softmax_backward=True,
                                     softmax_backward_lower=softmax_lower)
    if dtype == torch.float16:
        assert rec is None
    else:
        assert torch.equal(rec[0], ref[0]) and torch.equal(rec[1], ref[1])


@pytest.mark.parametrize("widths,batch,conn,grad_factor", [([400, 400, 300], 128, "random", 1.0),
                                                           ([300, 600, 600], 100, "unique", 2.0),
                                                           ([500, 500, 500, 250], 64, "random", 1.5),
                                                           ([200, 400], 32, "random", 1.0)])
def test_fuse_first_layers_trains_like_the_unfused_model(widths, batch, conn, grad_factor, monkeypatch):
    """fuse_first_layers / fuse_for_training: same positions, parameters and state_dict keys; in
    training the same scores and gradients as the unfused model and as the CPU python
    implementation; inputs that want a gradient, eval mode and packed inference take the two
    original layers."""
    import difflogic_amd as dl
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)        # layers this narrow walk their schedules too
    monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
    monkeypatch.setattr(dl.difflogic_cuda, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)
    torch.manual_seed(5)
    F, k, tau = 60, 10, 10.0
    mods, d = [torch.nn.Flatten()], F
    for wd in widths:
        mods.append(dl.LogicLayer(d, wd, grad_factor=grad_factor, connections=conn))
        d = wd
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    fused = dl.fuse_for_training(model).train()
    assert list(fused.state_dict()) == list(model.state_dict()) and len(fused) == len(model)
    assert isinstance(fused[-2], dl.FusedLogicLayerGroupSum)
    if len(widths) > 2:
        assert isinstance(fused[1], dl.FusedLogicLayerPair) and fused[1].weights is model[1].weights
        assert fused[2].weights is model[2].weights
    else:
        assert isinstance(fused[1], dl.LogicLayer)                  # two layers: the second belongs to the tail
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = (torch.rand(batch, F) < 0.3).float()
    labels = torch.randint(0, k, (batch,))

    def run(net, want_gx=False):
        net.zero_grad(set_to_none=True)
        xg = x.cuda()
        if want_gx:
            xg.requires_grad_()
        out = net(xg)
        torch.nn.functional.cross_entropy(out, labels.cuda()).backward()
        return out.detach(), [l.weights.grad.clone() for l in layers], xg.grad

    calls = []
    real = dl.difflogic_cuda.backward_chained_lower
    monkeypatch.setattr(dl.difflogic_cuda, "backward_chained_lower",
                        lambda *a, **kw: calls.append(a[0] is None) or real(*a, **kw))
    out0, gw0, _ = run(model)
    assert not calls
    out1, gw1, _ = run(fused)
    assert calls == ([True] if len(widths) > 2 else [])           # the pair recomputes its inner activation
    assert close(out1, out0)[0]
    for u, v in zip(gw1, gw0):
        assert close(u, v.double())[0]

    def python_impl(dtype):
        lg = [l.weights.detach().cpu().to(dtype).requires_grad_() for l in layers]
        net = fo.PythonNet([(l.indices[0].cpu(), l.indices[1].cpu(), w) for l, w in zip(layers, lg)], k, tau, grad_factor)
        o = net(x.detach().clone().to(dtype))
        torch.nn.functional.cross_entropy(o, labels).backward()
        return o.detach(), [w.grad for w in lg]

    o64, w64 = python_impl(torch.float64)
    o32, w32 = python_impl(torch.float32)
    assert close(out1, o64)[0]
    for got, r64, r32 in zip(gw1, w64, w32):
        ok, rep = within_budget(got, r64, r32)
        assert ok, rep
    out2, gw2, _ = run(fused)
    assert torch.equal(out1, out2) and all(torch.equal(u, v) for u, v in zip(gw1, gw2))

    # an input that wants its gradient: the two layers run one after the other
    n = len(calls)
    _, gw3, gx3 = run(fused, want_gx=True)
    _, gw4, gx4 = run(model, want_gx=True)
    assert len(calls) == n and gx3 is not None and close(gx3, gx4.double())[0]
    for u, v in zip(gw3, gw4):
        assert close(u, v.double())[0]

    # a frozen first layer: only the second layer's gradient, by the separate kernels
    model[1].weights.requires_grad_(False)
    fused.zero_grad(set_to_none=True)
    torch.nn.functional.cross_entropy(fused(x.cuda()), labels.cuda()).backward()
    assert model[1].weights.grad is None and close(model[2].weights.grad, gw0[1].double())[0]
    model[1].weights.requires_grad_(True)

    model.eval(), fused.eval()
    with torch.no_grad():
        assert torch.equal(fused(x.cuda()), model(x.cuda()))
        assert torch.equal(fused(dl.PackBitsTensor(x.bool().cuda(), bit_count=64)),
                           model(dl.PackBitsTensor(x.bool().cuda(), bit_count=64)))


@pytest.mark.parametrize("widths,wide", [([400, 400, 300], False), ([300, 600, 600, 300], True), ([200, 400], False)])
def test_fused_sequential_runs_the_logic_layers_as_one_autograd_node(widths, wide, monkeypatch):
    """fuse_for_training's Sequential: one autograd node from the first logic layer to the class scores, with the
    scores and every gradient bit for bit those of the same modules run one after the other; inputs that want a
    gradient are served too, and so are half / double inputs under float weights; a module the node does not know in
    between and eval mode fall back to (or are) the modules one by one."""
    import difflogic_amd as dl
    if wide:                                                     # layers this narrow walk their schedules too
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_IN_DIM", 0)
        monkeypatch.setattr(dl.LogicLayer, "_CHAIN_MIN_OUT_DIM", 0)
        monkeypatch.setattr(dl.difflogic_cuda, "BACKWARD_CHAIN_MAX_OVERFLOW", 1e9)
    torch.manual_seed(9)
    F, k, B = 60, 10, 96
    mods, d = [torch.nn.Flatten()], F
    for wd in widths:
        mods.append(dl.LogicLayer(d, wd, grad_factor=1.5))
        d = wd
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, 5.0)).train()
    fused = dl.fuse_for_training(model).train()
    assert isinstance(fused, dl.difflogic.FusedSequential) and list(fused.state_dict()) == list(model.state_dict())
    one_by_one = torch.nn.Sequential(*fused)                   # the same modules without the node
    layers = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = (torch.rand(B, F) < 0.4).float().cuda()
    labels = torch.randint(0, k, (B,)).cuda()

    def run(net, inp):
        net.zero_grad(set_to_none=True)
        out = net(inp)
        torch.nn.functional.cross_entropy(out, labels).backward()
        return out, [l.weights.grad.clone() for l in layers]

    out, gw = run(fused, x)
    assert type(out.grad_fn).__name__ == "LogicNetFunctionBackward"
    ref, gref = run(one_by_one, x)
    assert type(ref.grad_fn).__name__ != "LogicNetFunctionBackward"
    assert torch.equal(out, ref) and all(torch.equal(u, v) for u, v in zip(gw, gref))
    xg = x.clone().requires_grad_()
    out, gw = run(fused, xg)
    gx = xg.grad.clone()
    xg.grad = None
    ref, gref = run(one_by_one, xg)
    assert type(out.grad_fn).__name__ == "LogicNetFunctionBackward"
    assert torch.equal(out, ref) and torch.equal(gx, xg.grad) and all(torch.equal(u, v) for u, v in zip(gw, gref))
    # the activations are freed with the graph's buffers, as for any node; a retained graph can be walked twice
    fused.zero_grad(set_to_none=True)
    loss = torch.nn.functional.cross_entropy(fused(x), labels)
    loss.backward(retain_graph=True)
    first = [l.weights.grad.clone() for l in layers]
    fused.zero_grad(set_to_none=True)
    loss.backward()
    assert all(torch.equal(u, l.weights.grad) for u, l in zip(first, layers))
    with pytest.raises(RuntimeError):
        loss.backward()
    # double / half inputs under float weights: the layers take them (fp32 logits beside the activations), the fused
    # layer + GroupSum kernels do not: those two run as stages of their own inside the node
    for dt in (torch.float64, torch.float16):
        out, gw = run(fused, x.to(dt))
        assert out.dtype == dt and type(out.grad_fn).__name__ == "LogicNetFunctionBackward"
        ref, gref = run(one_by_one, x.to(dt))
        assert torch.equal(out, ref) and all(torch.equal(u, v) for u, v in zip(gw, gref))
    ref, gref = run(one_by_one, x)
    # a module the node does not know
    odd = dl.difflogic.FusedSequential(*list(fused)[:2], torch.nn.Identity(), *list(fused)[2:]).train()
    out = odd(x)
    assert type(out.grad_fn).__name__ != "LogicNetFunctionBackward" and torch.equal(out, ref)
    fused.eval()
    with torch.no_grad():
        assert torch.equal(fused(x), one_by_one.eval()(x))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
@pytest.mark.parametrize("in0,in_dim,out_dim,batch,kind", [(40, 64, 64, 256, "random"), (100, 300, 300, 512, "random"),
                                                           (30, 50, 60, 128, "unique"), (20, 30, 47, 260, "any"),
                                                           (15, 20, 40, 8, "any"), (25, 40, 24, 16, "sparse"),
                                                           (784, 1000, 1200, 128, "random"), (30, 50, 60, 1024, "unique")])
def test_two_layer_forward_recomputes_the_inner_activation(ext, dtype, in0, in_dim, out_dim, batch, kind):
    """dl_logic_forward_chained_lower: the output and both layers' probabilities of two forward_logits
    calls in a row, bit for bit, without the activation between them."""
    from oracle import connections as oc
    g = torch.Generator().manual_seed(in_dim + batch + in0)
    torch.manual_seed(in_dim)
    if kind == "random":
        a, b = oc.random_connections(in_dim, out_dim)
    elif kind == "unique":
        a, b = oc.unique_connections(in_dim, out_dim)
    elif kind == "sparse":                                           # half of the lower neurons feed nothing
        a, b = torch.randint(0, in_dim // 2, (out_dim,), generator=g), torch.randint(0, in_dim // 2, (out_dim,),
                                                                                    generator=g)
    else:
        a, b = torch.randint(0, in_dim, (out_dim,), generator=g), torch.randint(0, in_dim, (out_dim,), generator=g)
    a0 = torch.randint(0, in0, (in_dim,), generator=g).cuda()
    b0 = torch.randint(0, in0, (in_dim,), generator=g).cuda()
    x0 = torch.rand(in0, batch, generator=g).to(dtype).cuda()
    l0 = torch.randn(in_dim, 16, generator=g).to(dtype).cuda()
    l1 = torch.randn(out_dim, 16, generator=g).to(dtype).cuda()
    a, b = a.cuda(), b.cuda()
    sched = ext.schedule_for(a, b, in_dim)
    got = ext.forward_logits_lower(x0, a0, b0, l0, l1, sched)
    if batch * x0.element_size() % 16 or batch * x0.element_size() > 128 * 16:
        assert got is None                                          # whole 16-byte vectors, rows of at most 2 KB
        return
    y1, p0 = ext.forward_logits(x0, a0, b0, l0)
    y2, p1 = ext.forward_logits(y1, a, b, l1, sched)
    used = torch.zeros(in_dim, dtype=torch.bool, device="cuda")
    used[a] = True
    used[b] = True
    if dtype == torch.float16:
        # same fp32 arithmetic; the compiler may fold the final fp32 -> fp16 rounding into a fused multiply-add in
        # one kernel and not in the other: rare last-bit differences (which the second layer then carries on)
        for u, v in ((got[0], y2), (got[2], p1), (got[1][used], p0[used])):
            diff = (u.float() - v.float()).abs()
            assert float((diff > 0).float().mean()) < 0.05
            assert bool((diff <= 2.0 ** -9 * u.float().abs().clamp(min=2.0 ** -14)).all())
    else:
        assert torch.equal(got[0], y2) and torch.equal(got[2], p1) and torch.equal(got[1][used], p0[used])
    assert bool((got[1][~used] == 0).all())
