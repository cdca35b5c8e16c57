"""Parity of the packed-inference HIP kernels (through the C ABI and the Python API) with the
CPU oracle.  Bit-exact: every comparison is equality."""
import os

import numpy as np
import pytest
import torch

from oracle import connections as oc
from oracle import interp
from oracle import packed_oracle as po
from tests.helpers import build_model, random_layers

pytestmark = pytest.mark.gpu

NP_WORD = {8: np.int8, 16: np.int16, 32: np.int32, 64: np.int64}


@pytest.fixture(scope="module")
def ext():
    import difflogic_amd
    return difflogic_amd.difflogic_cuda


def _dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("F,B", [(1, 1), (3, 7), (5, 64), (5, 65), (7, 1000), (4, 1024), (9, 4112), (2, 70000),
                                 (784, 256)])
def test_packbits(ext, bits, F, B):
    rng = np.random.default_rng(F * 131 + B + bits)
    t = rng.random((F, B)) < 0.3
    want, pad = po.packbits(t, bits)
    got, got_pad = ext.tensor_packbits_cuda(_dev(t), bits)
    assert got_pad == pad and got.dtype == torch.as_tensor(want).dtype and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


def test_packbits_nonzero_bytes_count_as_true(ext):
    raw = torch.tensor([[0, 1, 2, 128, 255, 0, 7, 0] * 4], dtype=torch.uint8).cuda()
    got, _ = ext.tensor_packbits_cuda(raw.view(torch.bool), 32)
    want, _ = po.packbits(raw.cpu().numpy() != 0, 32)
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("B,F", [(1, 1), (7, 3), (64, 8), (65, 12), (1000, 7), (1024, 256), (4112, 260), (70000, 2),
                                 (3000, 784), (130, 1028), (200, 816), (333, 832), (129, 1648), (700, 9216),
                                 (513, 16), (8200, 48), (1100, 2368), (600, 2352), (9000, 128)])
def test_packbits_batch_major(ext, bits, B, F):
    rng = np.random.default_rng(F * 131 + B + bits)
    x = rng.random((B, F)) < 0.3
    want, pad = po.packbits(x.T, bits)
    got, got_pad = ext.tensor_packbits_batch_major(_dev(x), bits)
    assert got_pad == pad and got.dtype == torch.as_tensor(want).dtype and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
    # and it agrees with the two-step path of the reference
    two, _ = ext.tensor_packbits_cuda(_dev(x).T.contiguous(), bits)
    assert torch.equal(got, two)


@pytest.mark.parametrize("B,F,row_bytes", [(1, 1, 16), (7, 3, 8), (64, 8, 16), (65, 12, 16), (1000, 7, 128), (1000, 16, 144),
                                            (1000, 784, 128), (4112, 260, 528), (130, 1028, 32), (700, 9216, 96),
                                            (513, 16, 80), (0, 5, 16), (8200, 48, 1040), (129, 1648, 2064)])
def test_packbits_batch_major_rows(ext, B, F, row_bytes):
    """Rows longer than the batch needs: the bits are where tensor_packbits_cuda puts them, the rest is zero
    (the output buffer starts out as ones)."""
    rng = np.random.default_rng(F * 131 + B + row_bytes)
    x = rng.random((B, F)) < 0.3
    want = np.zeros((F, row_bytes), np.uint8)
    want[:, :-(-B // 8)] = np.packbits(x.T, axis=1, bitorder="little")
    got = ext.tensor_packbits_batch_major_rows(_dev(x), row_bytes)
    assert got.dtype == torch.int64 and tuple(got.shape) == (F, row_bytes // 8)
    assert np.array_equal(got.cpu().numpy().view(np.uint8), want)
    with pytest.raises(RuntimeError):
        ext.tensor_packbits_batch_major_rows(_dev(x), 8 * ((B - 1) // 64))  # too short


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("B", [1, 37, 64, 100, 128, 200, 1000, 1024 + 96, 16384, 16384 + 128, 3 * 8192 + 100])
def test_pack_tensor_every_width_and_batch(bits, B):
    """PackBitsTensor keeps padded rows inside (whole 16-byte vectors, from 2 KB on whole 128-byte lines); `.t`,
    `.pad_len` and the counts are the reference's for every word width and batch size, before, between and after
    layers, and writes into `.t` are seen."""
    import difflogic_amd as dl
    rng = np.random.default_rng(B * 4 + bits)
    layers = random_layers(rng, 24, [48, 48, 30])
    x = rng.random((B, 24)) < 0.5
    model = build_model(24, layers, 3).eval()
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    want_t, want_pad = po.packbits(x.T, bits)
    p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=bits)
    assert p.pad_len == want_pad and p.features == 24
    assert p.t.dtype == torch.as_tensor(want_t).dtype and np.array_equal(p.t.cpu().numpy(), want_t)
    assert p.t.is_contiguous() and p.t is p.t
    assert np.array_equal(p.group_sum(3).cpu().numpy(), po.groupbitsum(want_t, want_pad, 3))
    with torch.no_grad():
        p = logic[0](p)
    t1 = po.eval_layer(want_t, *layers[0])
    assert np.array_equal(p.t.cpu().numpy(), t1)
    with torch.no_grad():
        p = logic[2](logic[1](p))
    t3 = po.eval_layer(po.eval_layer(t1, *layers[1]), *layers[2])
    assert np.array_equal(p.group_sum(3).cpu().numpy(), po.groupbitsum(t3, want_pad, 3))     # last layers still deferred
    assert np.array_equal(p.t.cpu().numpy(), t3) and p.features == 30
    assert np.array_equal(p.group_sum(3).cpu().numpy(), po.groupbitsum(t3, want_pad, 3))
    p.t.zero_()                                                                              # in place, through `.t`
    assert int(p.group_sum(3).sum()) == 0
    p.t = torch.as_tensor(t1).cuda()                                                         # assigned
    with torch.no_grad():
        got = logic[2](logic[1](p)).group_sum(3)
    assert np.array_equal(got.cpu().numpy(), po.groupbitsum(t3, want_pad, 3))
    # the whole model at once (no `.t` read in between) against the bitwise oracle
    with torch.no_grad():
        got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=bits))
    assert np.array_equal(got.cpu().numpy(), po.net_eval_bitwise(x, layers, 3))


def test_packbits_batch_major_nonzero_bytes(ext):
    raw = torch.tensor([[0, 1, 2, 128], [255, 0, 7, 0], [3, 3, 0, 0]], dtype=torch.uint8).cuda()
    got, _ = ext.tensor_packbits_batch_major(raw.view(torch.bool), 8)
    want, _ = po.packbits((raw.cpu().numpy() != 0).T, 8)
    assert np.array_equal(got.cpu().numpy(), want)
    # rows of whole 16-byte chunks take the kernel that folds in registers: every byte value, every position
    rng = np.random.default_rng(5)
    raw = torch.as_tensor(rng.integers(0, 256, (777, 32), dtype=np.uint8) * (rng.random((777, 32)) < 0.5)).cuda()
    got, _ = ext.tensor_packbits_batch_major(raw.view(torch.bool), 64)
    want, _ = po.packbits((raw.cpu().numpy() != 0).T, 64)
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("W", [1, 2, 3, 5, 64, 127, 128, 129, 300])
def test_eval_layer_random(ext, bits, W):
    rng = np.random.default_rng(W * 7 + bits)
    in_dim, out_dim = 37, 203
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    (a, b, op), = random_layers(rng, in_dim, [out_dim])
    want = po.eval_layer(x, a, b, op)
    got = ext.eval(_dev(x), _dev(a), _dev(b), _dev(op))
    assert got.dtype == torch.as_tensor(want).dtype
    assert np.array_equal(got.cpu().numpy(), want)


def test_eval_every_gate_on_every_input_pair(ext):
    t = np.array([[0, 0, 1, 1], [0, 1, 0, 1]], dtype=bool)
    x, _ = po.packbits(t, 64)
    ops = np.arange(16, dtype=np.uint8)
    got = ext.eval(_dev(x), _dev(np.zeros(16, np.int64)), _dev(np.ones(16, np.int64)), _dev(ops)).cpu().numpy()
    assert np.array_equal(got, po.eval_layer(x, np.zeros(16, int), np.ones(16, int), ops))
    bits = po.unpackbits(got, 4)
    for i in range(16):
        assert bits[i].astype(int).tolist() == [int(c) for c in format(i, "04b")]


def test_eval_unaligned_views(ext):
    # a row length that is a multiple of 8 but not 16 bytes, and an odd int8 row length
    rng = np.random.default_rng(5)
    for bits, W in ((64, 3), (8, 13), (16, 5), (32, 3)):
        x = rng.integers(-100, 100, (9, W)).astype(NP_WORD[bits])
        (a, b, op), = random_layers(rng, 9, [40])
        got = ext.eval(_dev(x), _dev(a), _dev(b), _dev(op)).cpu().numpy()
        assert np.array_equal(got, po.eval_layer(x, a, b, op))


@pytest.mark.parametrize("bits,in_dim,W,k,pad", [
    (64, 30, 1, 3, 0), (64, 30, 3, 5, 17), (64, 640, 70, 10, 63), (64, 130, 129, 2, 1), (64, 7, 5, 7, 0),
    (64, 51, 2, 1, 5), (32, 64, 6, 4, 3), (32, 64, 5, 4, 3), (16, 40, 12, 5, 0), (16, 40, 7, 5, 9),
    (8, 24, 16, 3, 2), (8, 24, 9, 3, 7), (64, 40000, 2, 2, 11), (64, 70000, 1, 1, 0),
])
def test_groupbitsum(ext, bits, in_dim, W, k, pad):
    rng = np.random.default_rng(in_dim + W + k)
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    want = po.groupbitsum(x, pad, k)
    got = ext.groupbitsum(_dev(x), pad, k)
    assert got.dtype == torch.int32 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


def test_groupbitsum_saturated_counts(ext):
    # all bits set: every count equals the class size, for sizes around the counter-plane limits
    for per_class in (15, 16, 17, 4095 * 4, 4096 * 4, 4096 * 4 + 1):
        x = torch.full((per_class * 2, 3), -1, dtype=torch.int64).cuda()
        got = ext.groupbitsum(x, 5, 2)
        assert got.shape == (3 * 64 - 5, 2) and bool((got == per_class).all())


def test_errors(ext):
    x = torch.zeros(6, 2, dtype=torch.int64).cuda()
    with pytest.raises(ValueError):
        ext.groupbitsum(x, 0, 4)
    with pytest.raises(ValueError):
        ext.tensor_packbits_cuda(torch.zeros(2, 8, dtype=torch.bool).cuda(), 12)
    with pytest.raises(RuntimeError):
        ext.tensor_packbits_cuda(torch.zeros(2, 8, dtype=torch.bool), 8)            # CPU tensor
    with pytest.raises(RuntimeError):
        ext.groupbitsum(torch.zeros(6, 4, dtype=torch.int64).cuda()[:, ::2], 0, 3)  # not contiguous
    with pytest.raises(RuntimeError):
        ext.eval(x, torch.zeros(3, dtype=torch.int64).cuda(), torch.zeros(4, dtype=torch.int64).cuda(),
                 torch.zeros(3, dtype=torch.uint8).cuda())                          # a/b/w lengths differ
    # empty batch
    out, pad = ext.tensor_packbits_cuda(torch.zeros(3, 0, dtype=torch.bool).cuda(), 64)
    assert out.shape == (3, 0) and pad == 0
    assert ext.groupbitsum(out, 0, 3).shape == (0, 3)


def test_compiled_fixtures_through_the_api(golden_dir):
    """The reference's own CompiledLogicNet outputs, reproduced by PackBitsTensor -> LogicLayer
    (eval) -> GroupSum on the GPU."""
    import difflogic_amd as dl
    comp = np.load(os.path.join(golden_dir, "compiled.npz"))
    for name in (str(c) for c in comp["cases"]):
        F, k, bits, batch, L = (int(v) for v in comp[name + "_meta"])
        layers = [(comp[f"{name}_a{i}"], comp[f"{name}_b{i}"], comp[f"{name}_op{i}"]) for i in range(L)]
        model = build_model(F, layers, k).eval()
        x = torch.as_tensor(comp[name + "_x"])
        for bc in (bits, 64):
            with torch.no_grad():
                got = model(dl.PackBitsTensor(x.cuda(), bit_count=bc))
            assert got.dtype == torch.int32
            assert np.array_equal(got.cpu().numpy(), comp[name + "_y"]), (name, bc)


@pytest.mark.parametrize("F,widths,k,B", [(784, [8000] * 6, 10, 4096 + 37), (100, [1000, 3000, 2000], 5, 777),
                                          (9216, [25600, 25600], 10, 1024)])
def test_net_against_c_interpreter(F, widths, k, B):
    import difflogic_amd as dl
    rng = np.random.default_rng(F + B)
    layers = random_layers(rng, F, widths)
    x = rng.random((B, F)) < 0.2
    want = interp.net_eval(x, layers, k, threads=8)
    model = build_model(F, layers, k).eval()
    with torch.no_grad():
        got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64))
    assert np.array_equal(got.cpu().numpy(), want)


def test_packed_equals_float_eval():
    """On {0,1} inputs the float eval path (one-hot gates) times tau equals the packed counts."""
    import difflogic_amd as dl
    rng = np.random.default_rng(11)
    layers = random_layers(rng, 50, [200, 200, 120])
    x = rng.random((300, 50)) < 0.4
    model = build_model(50, layers, 4, tau=7.0).eval()
    with torch.no_grad():
        packed = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=32))
        flt = model(torch.as_tensor(x).float().cuda())
    assert np.array_equal(packed.cpu().numpy(), np.rint(flt.cpu().numpy() * 7.0).astype(np.int32))
    assert np.array_equal(packed.cpu().numpy(), po.net_eval_bitwise(x, layers, 4))


def test_pack_tensor_repr_and_modes():
    import difflogic_amd as dl
    t = torch.tensor([[1, 0], [0, 0], [1, 1]], dtype=torch.bool)          # [B=3, F=2]
    p = dl.PackBitsTensor(t.cuda(), bit_count=8)
    assert p.pad_len == 5 and p.t.shape == (2, 1) and p.flatten() is p
    assert repr(p) == "10100000\n00100000"
    layer = dl.LogicLayer(2, 4)
    with pytest.raises(AssertionError):
        layer(p)                                                          # training mode
    with pytest.raises(NotImplementedError):
        dl.PackBitsTensor(t, device="cpu")


def _chain(rng, in_dim, widths):
    layers = random_layers(rng, in_dim, widths)
    return layers, [tuple(_dev(t) for t in l) for l in layers]


@pytest.mark.parametrize("bits,in_dim,widths,W", [
    (64, 30, [60], 3), (64, 30, [60, 50], 1), (64, 50, [64, 70, 40], 70), (64, 33, [130, 90, 100, 77], 129),
    (32, 20, [64, 64], 6), (32, 20, [64, 64, 64], 5), (16, 20, [40, 30], 12), (8, 12, [24, 24, 24, 24], 16),
    (8, 12, [24, 30], 9), (64, 784, [4000, 4000, 4000, 4000], 40), (64, 3000, [3000, 3000], 64),
])
def test_eval_fused_equals_layer_by_layer(ext, bits, in_dim, widths, W):
    rng = np.random.default_rng(in_dim + W + len(widths))
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    layers, dev_layers = _chain(rng, in_dim, widths)
    want = x
    for a, b, op in layers:
        want = po.eval_layer(want, a, b, op)
    got = ext.eval_fused(_dev(x), dev_layers)
    assert got.dtype == torch.as_tensor(want).dtype and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


def test_eval_fused_every_gate_combination(ext):
    # depth 2 over the four input pairs: 16^3 gate triples, one output neuron each
    t = np.array([[0, 0, 1, 1], [0, 1, 0, 1]], dtype=bool)
    x, _ = po.packbits(t, 64)
    g1, g2, g3 = np.meshgrid(np.arange(16), np.arange(16), np.arange(16), indexing="ij")
    l1 = (np.zeros(256, np.int64), np.ones(256, np.int64), np.arange(256) // 16 % 16)          # 256 first-layer gates
    l1 = (np.zeros(32, np.int64), np.ones(32, np.int64), (np.arange(32) % 16).astype(np.uint8))
    a2 = g1.reshape(-1).astype(np.int64)
    b2 = (16 + g2.reshape(-1)).astype(np.int64)
    l2 = (a2, b2, g3.reshape(-1).astype(np.uint8))
    want = po.eval_layer(po.eval_layer(x, *l1), *l2)
    got = ext.eval_fused(_dev(x), [tuple(_dev(v) for v in l1), tuple(_dev(v) for v in l2)])
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("bits,in_dim,widths,W,k,pad", [
    (64, 30, [60], 1, 3, 0), (64, 50, [640], 70, 10, 63), (64, 33, [130], 129, 2, 1), (32, 20, [64], 6, 4, 3),
    (16, 20, [40], 12, 5, 0), (8, 12, [24], 16, 3, 2), (8, 12, [24], 9, 3, 7), (64, 100, [40000], 2, 2, 11),
    (64, 64, [70000], 1, 1, 0), (32, 20, [64], 5, 4, 3),
    (64, 30, [60, 90], 1, 3, 0), (64, 50, [100, 640], 70, 10, 63), (64, 33, [66, 130], 129, 2, 1),
    (32, 20, [40, 64], 6, 4, 3), (8, 12, [24, 24], 9, 3, 7), (64, 100, [200, 40000], 2, 2, 11),
    (64, 784, [8000, 8000], 33, 10, 5),
])
def test_fused_eval_groupbitsum(ext, bits, in_dim, widths, W, k, pad):
    rng = np.random.default_rng(in_dim + W + k + widths[-1])
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    layers, dev_layers = _chain(rng, in_dim, widths)
    y = x
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    want = po.groupbitsum(y, pad, k)
    got = ext.eval_fused_groupbitsum(_dev(x), dev_layers, pad, k)
    assert got.dtype == torch.int32 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
    assert torch.equal(got, ext.groupbitsum(ext.eval_fused(_dev(x), dev_layers), pad, k))
    # walking the neurons in the cache-friendly order changes nothing
    order = ext.count_order_for(dev_layers, in_dim, k)
    assert order.dtype == torch.int32 and sorted(order.tolist()) == list(range(widths[-1]))
    assert torch.equal(got, ext.eval_fused_groupbitsum(_dev(x), dev_layers, pad, k, order))
    assert ext.count_order_for(dev_layers, in_dim, k) is order          # cached per wiring


def test_lazy_pack_tensor_keeps_t_current():
    """``.t`` read between layers and after the last layer equals the eager per-layer result."""
    import difflogic_amd as dl
    rng = np.random.default_rng(21)
    layers = random_layers(rng, 20, [64, 64, 33])
    x = rng.random((200, 20)) < 0.5
    model = build_model(20, layers, 3).eval()
    p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)
    t = p.t.cpu().numpy()
    for layer, (a, b, op) in zip([m for m in model if isinstance(m, dl.LogicLayer)], layers):
        with torch.no_grad():
            p = layer(p)
        t = po.eval_layer(t, a, b, op)
        assert np.array_equal(p.t.cpu().numpy(), t)
    assert np.array_equal(p.group_sum(3).cpu().numpy(), po.groupbitsum(t, p.pad_len, 3))
    with pytest.raises(ValueError):
        p.group_sum(7)
    # deferred last layer + group_sum (fused) and a user assigning .t
    p2 = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)
    with torch.no_grad():
        got = model(p2)
    assert np.array_equal(got.cpu().numpy(), po.groupbitsum(t, p.pad_len, 3))
    p2.t = torch.zeros_like(p2.t)
    assert int(p2.group_sum(3).sum()) == 0


@pytest.mark.parametrize("bits,in_dim,widths,W,kind", [
    (64, 64, [64], 130, "random"), (64, 100, [100, 100], 3, "random"), (64, 30, [200, 200, 200], 64, "random"),
    (32, 50, [60, 70], 7, "unique"), (8, 7, [20, 20], 16, "any"), (64, 5, [3, 3], 5, "self"),
    (64, 784, [6000, 6000, 6000, 6000], 64, "random"), (64, 3000, [3000, 3000], 128, "random"),
    (64, 40, [80, 80, 80, 80], 9, "any"), (64, 500, [64000], 16, "random"),
    # 8, 9 and 65 column tiles of 128 words: each XCD sweeps whole column tiles (a whole number each; not with 9;
    # with 65 the grid is padded to 72 and the tiles past the last column do nothing)
    (64, 784, [2000, 2000], 1024, "random"), (64, 784, [2000, 2000], 1100, "random"), (64, 100, [300, 300], 8197, "random"),
    (64, 784, [1500, 1500, 1500, 1500], 1024, "random"), (64, 200, [600, 600, 600], 2048, "unique"),
])
def test_eval_chained_equals_eval_fused(ext, bits, in_dim, widths, W, kind):
    from oracle import connections as oc
    rng = np.random.default_rng(in_dim + len(widths) + W)
    torch.manual_seed(in_dim)
    layers, d = [], in_dim
    for o in widths:
        if kind == "random":
            a, b = (t.numpy() for t in oc.random_connections(d, o))
        elif kind == "unique":
            a, b = (t.numpy() for t in oc.unique_connections(d, o))
        elif kind == "self":
            a, b = np.array([1, 1, 2]), np.array([1, 1, 2])
        else:
            a, b = rng.integers(0, d, o), rng.integers(0, d, o)
        layers.append((a.astype(np.int64), b.astype(np.int64), rng.integers(0, 16, o).astype(np.uint8)))
        d = o
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    want = x
    for a, b, op in layers:
        want = po.eval_layer(want, a, b, op)
    dev_layers = [tuple(_dev(t) for t in l) for l in layers]
    got = ext.eval_chained(_dev(x), dev_layers)
    assert got.dtype == torch.as_tensor(want).dtype and np.array_equal(got.cpu().numpy(), want)
    sched = ext.schedule_for(dev_layers[-1][0], dev_layers[-1][1], (in_dim if len(widths) == 1 else widths[-2]))
    assert sched.steps % sched.chunk == 0 and sched.steps >= widths[-1]
    assert ext.schedule_for(dev_layers[-1][0], dev_layers[-1][1], sched.in_dim) is sched         # cached


def test_fold_gate_constants(ext):
    """Constants folded through the gate ids: the folded net is the same function of the rows that vary (checked
    against the per-layer oracle on the ORIGINAL gate ids), constant neurons are found (their folded id is 0 or
    15), and a gate that reads one ignores that input afterwards."""
    rng = np.random.default_rng(11)
    in_dim, widths, W = 40, [300, 300, 300, 200], 5
    layers = random_layers(rng, in_dim, widths)
    for l in layers:                                         # plenty of constant and one-input gates
        l[2][rng.random(len(l[2])) < 0.3] = rng.choice([0, 15, 3, 5, 10, 12])
    dev_layers = [tuple(_dev(t) for t in l) for l in layers]
    folded = ext.fold_gate_constants(dev_layers)
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, (in_dim, W), dtype=np.int64, endpoint=True)
    want, got = x, x
    consts = np.zeros(in_dim, bool)
    for (a, b, op), (_, _, fop) in zip(layers, folded):
        fop = fop.cpu().numpy()
        want = po.eval_layer(want, a, b, op)
        got = po.eval_layer(got, a, b, fop)
        assert np.array_equal(got, want)
        is_const = (fop == 0) | (fop == 15)
        # every row that is constant for ALL inputs it can see is found when it follows from the gates alone:
        # a folded constant really is one, and a gate reading a constant row no longer looks at it
        assert np.all((want[is_const] == 0) | (want[is_const] == -1))
        uses_a = (((fop >> 3) ^ (fop >> 1)) & 1) | (((fop >> 2) ^ fop) & 1)
        uses_b = (((fop >> 3) ^ (fop >> 2)) & 1) | (((fop >> 1) ^ fop) & 1)
        assert not np.any(uses_a.astype(bool) & consts[a]) and not np.any(uses_b.astype(bool) & consts[b])
        consts = is_const
    assert consts.sum() > 20
    # folding is idempotent
    again = ext.fold_gate_constants(folded)
    assert all(torch.equal(u[2], v[2]) for u, v in zip(folded, again))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
def test_gate_ids_folded_is_gate_ids_then_fold(ext, dtype):
    """dl_gate_ids_folded against dl_gate_ids followed by dl_fold_gate_constants, layer by layer (ties, NaNs and
    constant gates included), and LogicLayer in eval mode hands PackBitsTensor exactly those ids."""
    import difflogic_amd as dl
    rng = np.random.default_rng(23)
    torch.manual_seed(23)
    in_dim, widths = 50, [400, 300, 500]
    layers = random_layers(rng, in_dim, widths)
    state, plain = None, []
    for a, b, _ in layers:
        w = torch.randn(len(a), 16, dtype=dtype)
        w[rng.random(len(a)) < 0.2, 0] = 30.0                     # constant-zero gates
        w[rng.random(len(a)) < 0.1, 15] = 40.0                    # constant-one gates
        w[rng.random(len(a)) < 0.1, :] = 1.0                      # ties: the first wins
        w[rng.random(len(a)) < 0.05, 7] = float("nan")            # a NaN counts as maximal
        w = w.cuda()
        ids = ext.gate_ids(w)
        assert torch.equal(ids.cpu(), w.cpu().argmax(-1).to(torch.uint8))
        plain.append((_dev(a), _dev(b), ids))
        got_ids, state = ext.gate_ids_folded(w, _dev(a), _dev(b), state)
        want = ext.fold_gate_constants(plain)[-1][2]
        assert torch.equal(got_ids, want)
        assert torch.equal(state, torch.where(want == 0, 1, torch.where(want == 15, 2, 0)).to(torch.uint8))
    assert int((state != 0).sum()) > 100
    # through the modules: the deferred layers hold the folded ids, and nothing is folded again before they run
    model = build_model(in_dim, [(a, b, w.cpu().numpy()) for a, b, w in plain], 10).eval()
    p = dl.PackBitsTensor(torch.as_tensor(rng.random((70, in_dim)) < 0.5).cuda(), bit_count=64)
    with torch.no_grad():
        for m in model:
            if isinstance(m, dl.LogicLayer):
                p = m(p)
    assert p._folded and len(p._pending) == 3
    want = ext.fold_gate_constants([(a, b, m.weights.argmax(-1).to(torch.uint8)) for (a, b, _), m in
                                    zip(plain, [m for m in model if isinstance(m, dl.LogicLayer)])])
    assert all(torch.equal(u[2], v[2]) for u, v in zip(p._pending, want))


def test_rows_written_through_t_are_not_taken_for_constants():
    """A layer of constant gates makes constant rows, which the next layer's gate ids fold in; once `.t` has been
    handed out the caller may have written into those rows, and the folding must not rely on them any more."""
    import difflogic_amd as dl
    rng = np.random.default_rng(29)
    F, B = 40, 200
    layers = random_layers(rng, F, [128, 256])
    layers[0][2][:] = rng.choice([0, 15], 128)                 # every row of the first layer is constant
    model = build_model(F, layers, 2).eval()
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    x = rng.random((B, F)) < 0.5
    p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)
    with torch.no_grad():
        p = logic[0](p)
        assert p.row_state(torch.device("cuda", 0)) is not None
        words = p.t                                            # a view of the rows where their length allows it
        fresh = torch.as_tensor(rng.integers(-2**62, 2**62, tuple(words.shape), dtype=np.int64)).cuda()
        words.copy_(fresh)                                     # the rows vary now
        mid = p.t.cpu().numpy().copy()
        p = logic[1](p)
        got = p.t.cpu().numpy()
    assert np.array_equal(got, po.eval_layer(mid, *layers[1]))


def test_pack_tensor_after_counting_with_rows_left_unwritten():
    """A net too wide for the LDS kernel streams in several groups; group_sum leaves rows of the inner groups unwritten
    that no gate above looks at.  The object stays usable: counting again, reading `.t` (every row of the last layer)
    and applying one more layer give what the oracle gives."""
    import difflogic_amd as dl
    from difflogic_amd import packbitstensor as pbt
    rng = np.random.default_rng(17)
    F, widths, k, B = 100, [12000, 11000, 12000, 10500], 10, 200
    layers = random_layers(rng, F, widths)
    x = rng.random((B, F)) < 0.5
    assert len(pbt.plan_groups([F] + widths, True, 4)) >= 2 and pbt.lds_tail([F] + widths, 4) == 0
    model = build_model(F, layers, k).eval()
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    want = po.net_eval_bitwise(x, layers, k)
    p = dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=32)
    with torch.no_grad():
        for m in logic:
            p = m(p)
    assert np.array_equal(p.group_sum(k).cpu().numpy(), want)
    assert np.array_equal(p.group_sum(k).cpu().numpy(), want)                   # again, from the rows kept
    t = po.packbits(x.T, 32)[0]
    for a, b, op in layers:
        t = po.eval_layer(t, a, b, op)
    assert np.array_equal(p.t.cpu().numpy(), t)                                 # every row of the last layer
    assert np.array_equal(p.group_sum(k).cpu().numpy(), want)
    extra = random_layers(rng, widths[-1], [6000])[0]
    more = dl.LogicLayer(widths[-1], 6000)
    more.set_connections(torch.as_tensor(extra[0]), torch.as_tensor(extra[1]))
    with torch.no_grad():
        more.weights.copy_(torch.nn.functional.one_hot(torch.as_tensor(extra[2]).long(), 16).float())
        p = more.eval()(p)
    assert np.array_equal(p.group_sum(k).cpu().numpy(), po.groupbitsum(po.eval_layer(t, *extra), p.pad_len, k))


def test_live_inputs_and_rows_left_unwritten(ext):
    """live_inputs marks exactly the rows some needed neuron looks at (numpy restatement); eval_chained with that
    vector writes every marked row as the oracle has it, and the layers above give the same result whatever the
    other rows hold."""
    rng = np.random.default_rng(12)
    in_dim, widths, W = 60, [500, 480, 520, 400, 300], 6
    layers = random_layers(rng, in_dim, widths)
    dev_layers = ext.fold_gate_constants([tuple(_dev(t) for t in l) for l in layers])
    host = [(a, b, w.cpu().numpy()) for (a, b, _), (_, _, w) in zip(layers, dev_layers)]
    live = ext.live_inputs(dev_layers)
    assert live[0] is None
    need = np.ones(widths[-1], bool)
    for i in range(len(layers) - 1, 0, -1):
        a, b, w = host[i]
        uses_a = ((((w >> 3) ^ (w >> 1)) & 1) | (((w >> 2) ^ w) & 1)).astype(bool)
        uses_b = ((((w >> 3) ^ (w >> 2)) & 1) | (((w >> 1) ^ w) & 1)).astype(bool)
        want = np.zeros(widths[i - 1], bool)
        want[a[need & uses_a]] = True
        want[b[need & uses_b]] = True
        assert np.array_equal(live[i].cpu().numpy().astype(bool), want), i
        need = want
    assert 0.2 < live[3].float().mean().item() < 0.95          # something to skip, something to keep
    # the first three layers as one group whose output feeds layers 4 and 5
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, (in_dim, W), dtype=np.int64, endpoint=True)
    want = x
    for a, b, op in layers[:3]:
        want = po.eval_layer(want, a, b, op)
    got = ext.eval_chained(_dev(x), dev_layers[:3], out_live=live[3])
    keep = live[3].cpu().numpy().astype(bool)
    assert np.array_equal(got.cpu().numpy()[keep], want[keep])
    full = want
    for a, b, op in layers[3:]:
        full = po.eval_layer(full, a, b, op)
    rest = ext.eval_chained(got, dev_layers[3:])
    assert np.array_equal(rest.cpu().numpy(), full)
    with pytest.raises(RuntimeError):
        ext.eval_chained(_dev(x), dev_layers[:3], out_live=live[2])


def test_eval_schedule_rejects_bad_wiring(ext):
    with pytest.raises(RuntimeError):
        ext.EvalSchedule(torch.tensor([0, 5]).cuda(), torch.tensor([1, 1]).cuda(), 3)


def test_schedule_follows_in_place_wiring_changes():
    import difflogic_amd as dl
    rng = np.random.default_rng(8)
    F = 300
    layers = random_layers(rng, F, [600, 600, 600])
    x = rng.random((130, F)) < 0.5
    model = build_model(F, layers, 10).eval()
    with torch.no_grad():
        got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)).cpu().numpy()
    assert np.array_equal(got, interp.net_eval(x, layers, 10, threads=4))
    layers2 = random_layers(rng, F, [600, 600, 600])
    for m, (a, b, op) in zip([model[1], model[2], model[3]], layers2):
        m.indices[0].copy_(torch.as_tensor(a))              # in place: same storage, new version
        m.indices[1].copy_(torch.as_tensor(b))
        with torch.no_grad():
            m.weights.copy_(torch.nn.functional.one_hot(torch.as_tensor(op).long(), 16).float())
    with torch.no_grad():
        got2 = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)).cpu().numpy()
    assert np.array_equal(got2, interp.net_eval(x, layers2, 10, threads=4))


def test_packed_inference_follows_weight_writes_through_data():
    """``layer.weights.data.copy_(...)`` (no version bump) between two packed evaluations: the second
    one uses the new gates."""
    import difflogic_amd as dl
    rng = np.random.default_rng(12)
    F = 40
    layers = random_layers(rng, F, [80, 80, 60])
    x = rng.random((200, F)) < 0.5
    model = build_model(F, layers, 10).eval()
    xd = torch.as_tensor(x).cuda()
    with torch.no_grad():
        got = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got, interp.net_eval(x, layers, 10))
    layers2 = [(a, b, ((op.astype(np.int64) * 7 + 3) % 16).astype(np.uint8)) for a, b, op in layers]
    for m, (_, _, op) in zip([model[1], model[2], model[3]], layers2):
        m.weights.data.copy_(torch.nn.functional.one_hot(torch.as_tensor(op).long(), 16).float())
    with torch.no_grad():
        got2 = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got2, interp.net_eval(x, layers2, 10))


@pytest.mark.parametrize("shape", ["streaming", "lds"])
def test_packed_inference_follows_wiring_writes_after_invalidate_wiring(shape):
    """The schedules and plans cached per wiring follow the index tensors' version counters.  A write through
    ``indices[i].data`` leaves the counter alone: LogicLayer.invalidate_wiring() after it makes the next packed
    evaluation (and the training kernels' schedules, and the reverse index) use the new wiring.  In-place
    operations that do bump the version are noticed by the schedule caches themselves; set_connections needs no call."""
    import difflogic_amd as dl
    rng = np.random.default_rng(31)
    F, widths, B = (64, [12000, 11000, 10500], 300) if shape == "streaming" else (48, [600, 700, 640], 300)
    layers = random_layers(rng, F, widths)
    x = rng.random((B, F)) < 0.5
    model = build_model(F, layers, 10).eval()
    xd = torch.as_tensor(x).cuda()
    with torch.no_grad():
        got = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got, interp.net_eval(x, layers, 10))
    logic = [m for m in model if isinstance(m, dl.LogicLayer)]
    # (1) through .data, then invalidate_wiring
    layers2 = [(np.roll(a, 3), b[::-1].copy(), op) for a, b, op in layers]
    for m, (a, b, _) in zip(logic, layers2):
        m.indices[0].data.copy_(torch.as_tensor(a))
        m.indices[1].data.copy_(torch.as_tensor(b))
        m.invalidate_wiring()
    with torch.no_grad():
        got2 = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got2, interp.net_eval(x, layers2, 10))
    start, idx = oc.reverse_index(layers2[1][0], layers2[1][1], widths[0])
    assert np.array_equal(logic[1].given_x_indices_of_y_start.cpu().numpy(), start)
    assert np.array_equal(logic[1].given_x_indices_of_y.cpu().numpy(), idx)
    # (2) an in-place operation (version bump): nothing to call
    layers3 = [(b, a, op) for a, b, op in layers2]
    for m, (a, b, _) in zip(logic, layers3):
        m.indices[0].copy_(torch.as_tensor(a))
        m.indices[1].copy_(torch.as_tensor(b))
    with torch.no_grad():
        got3 = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got3, interp.net_eval(x, layers3, 10))
    # (3) set_connections
    for m, (a, b, _) in zip(logic, layers):
        m.set_connections(torch.as_tensor(a), torch.as_tensor(b))
    with torch.no_grad():
        got4 = model(dl.PackBitsTensor(xd, bit_count=64)).cpu().numpy()
    assert np.array_equal(got4, got)


@pytest.mark.parametrize("bits,in_dim,widths,W,k,pad", [
    (64, 30, [60], 1, 3, 0),                              # a single layer: straight into the class phase
    (64, 30, [60, 90], 1, 3, 0), (64, 50, [100, 640], 7, 10, 63), (64, 33, [66, 130, 77, 130], 129, 2, 1),
    (32, 20, [40, 64], 6, 4, 3), (8, 12, [24, 24, 24], 16, 3, 2), (16, 20, [40, 40], 12, 5, 0),
    (64, 784, [8000] * 6, 9, 10, 5),                      # C2's net: 2 columns per workgroup, odd column count
    (64, 784, [4000] * 3, 11, 10, 0),                     # 4 columns per workgroup, 3 columns left over
    (64, 6000, [3000, 10240, 3000], 3, 3, 7),             # widest supported layer; input wider than the last layer
    (64, 100, [300, 4096], 5, 2, 0),                      # 2048 neurons per class: 8 counter planes per lane
    (64, 64, [128, 1920], 2, 2, 11),                      # 960 per class: the most 4 planes per lane hold
    (64, 64, [128, 2048], 2, 2, 11),                      # 1024 per class: 16 per lane, needs the fifth plane
    (64, 40, [80, 400], 4, 40, 9),                        # more classes than waves
    (64, 5, [3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 3, 4], 2, 2, 0),     # 16 layers
    (64, 200, [8100, 8100, 300], 2, 10, 0),               # more than 1024 chunks: the steps past them go one per thread
    (64, 4000, [2000, 5000, 5000, 40], 5, 4, 0),          # 4 columns: some schedules fit its buffer, some do not
    (64, 3000, [8190, 8250, 9000, 20], 3, 4, 0),          # schedules around 8192 steps and over 9216
])
def test_net_lds_groupbitsum(ext, bits, in_dim, widths, W, k, pad):
    """The LDS-resident whole-net kernel against the oracle (eval per layer, then groupbitsum) and
    against the streaming kernels."""
    rng = np.random.default_rng(in_dim + W + k + widths[-1] + len(widths))
    x = rng.integers(np.iinfo(NP_WORD[bits]).min, np.iinfo(NP_WORD[bits]).max, (in_dim, W), dtype=NP_WORD[bits],
                     endpoint=True)
    layers, dev_layers = _chain(rng, in_dim, widths)
    y = x
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    want = po.groupbitsum(y, pad, k)
    got = ext.eval_net_lds(_dev(x), dev_layers, pad, k)
    if W * bits % 64:
        assert got is None                                # rows are not whole 64-bit words
        return
    assert got is not None and got.dtype == torch.int32 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
    # hidden layers evaluated neuron by neuron instead of along their schedules: the same counts
    assert torch.equal(got, ext.eval_net_lds(_dev(x), dev_layers, pad, k, scheduled=False))
    # the net thinned for the call (constants folded, neurons that nothing looks at left out): the same counts
    assert torch.equal(got, ext.eval_net_lds(_dev(x), dev_layers, pad, k, thin=True))
    t = _dev(x)
    for lay in dev_layers:
        t = ext.eval(t, *lay)
    assert torch.equal(got, ext.groupbitsum(t, pad, k))


def test_net_lds_every_gate_and_saturated_counts(ext):
    """All 16 gates on all four input pairs through the per-lane mask path, and a class whose
    every neuron is true for every sample (the count reaches the class size in every lane)."""
    t = np.array([[0, 0, 1, 1], [0, 1, 0, 1]], dtype=bool)
    x, pad = po.packbits(t, 64)
    l1 = (np.zeros(16, np.int64), np.ones(16, np.int64), np.arange(16).astype(np.uint8))
    want = po.groupbitsum(po.eval_layer(x, *l1), pad, 16)
    l0 = (np.array([0, 1]), np.array([1, 0]), np.array([3, 3], dtype=np.uint8))        # gate 3 = a: rows stay as they are
    got = ext.eval_net_lds(_dev(x), [tuple(_dev(v) for v in l0), tuple(_dev(v) for v in l1)], pad, 16)
    assert np.array_equal(got.cpu().numpy(), want)
    ones = (np.zeros(5000, np.int64), np.zeros(5000, np.int64), np.full(5000, 15, np.uint8))
    xs = np.zeros((3, 5), dtype=np.int64)
    got = ext.eval_net_lds(_dev(xs), [tuple(_dev(v) for v in ones), tuple(_dev(v) for v in ones)], 3, 2)
    assert got.shape == (317, 2) and bool((got == 2500).all())


def test_net_lds_declines_what_does_not_fit(ext):
    rng = np.random.default_rng(2)
    layers, dev_layers = _chain(rng, 30, [60, 10241])
    assert ext.eval_net_lds(_dev(np.zeros((30, 2), np.int64)), dev_layers, 0, 1) is None        # too wide
    layers, dev_layers = _chain(rng, 30, [40] * 17)
    assert ext.eval_net_lds(_dev(np.zeros((30, 2), np.int64)), dev_layers, 0, 1) is None        # too deep
    with pytest.raises(ValueError):
        ext.eval_net_lds(_dev(np.zeros((30, 2), np.int64)), dev_layers, 0, 3)                   # 40 % 3


def test_pack_tensor_runs_narrow_tail_in_lds(monkeypatch):
    """PackBitsTensor.group_sum hands the narrow end of a net to the LDS kernel (the wide head
    streams), and the result equals the oracle's."""
    import difflogic_amd as dl
    from difflogic_amd import packbitstensor as pbt
    assert pbt.lds_tail([784, 8000, 8000, 8000]) == 3 and pbt.lds_tail([784, 64000, 64000]) == 0
    assert pbt.lds_tail([20000, 12000, 12000]) == 0 and pbt.lds_tail([784, 8000]) == 1
    # at full batch the narrow end of a wide net streams (staging thousands of packed rows in 16-byte pieces costs
    # more than it saves); on a short batch, where launches count, it goes to the LDS kernel
    taper = [784, 64000, 32000, 16000, 8000, 8000]
    assert pbt.lds_tail(taper, 16384) == 0 and pbt.lds_tail(taper, 4) == 1
    rng = np.random.default_rng(31)
    F, widths = 40, [12000, 6000, 3000, 1500]
    layers = random_layers(rng, F, widths)
    x = rng.random((300, F)) < 0.4
    model = build_model(F, layers, 10).eval()
    calls = []
    real = dl.difflogic_cuda.eval_net_lds
    monkeypatch.setattr(dl.difflogic_cuda, "eval_net_lds", lambda *a, **kw: calls.append(len(a[1])) or real(*a, **kw))
    with torch.no_grad():
        got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=64)).cpu().numpy()
    assert calls == [2]                                   # 6000 -> 3000 -> 1500 in LDS; what reads the 12000 rows streams
    assert np.array_equal(got, interp.net_eval(x, layers, 10))


@pytest.mark.parametrize("in_dim,widths,W,k,pad,kind", [
    (30, [60], 1, 3, 0, "any"), (50, [640], 70, 10, 63, "any"), (33, [130], 129, 2, 1, "any"),
    (64, [64], 3, 16, 0, "random"), (100, [40000], 2, 2, 11, "any"),
    (30, [60, 90], 1, 3, 0, "any"), (50, [100, 640], 70, 10, 63, "any"), (33, [66, 130], 129, 2, 1, "any"),
    (784, [8000, 8000], 33, 10, 5, "random"), (784, [8000, 8000], 32, 10, 0, "unique"),
    (300, [3000, 3000], 16, 1, 0, "random"),               # one class: every output lands in one counter
    (20, [40, 64], 4, 16, 3, "self"), (40, [80, 2400], 2, 12, 0, "any"),
    # more classes than a workgroup has waves: two sets of counters per wave
    (50, [100, 640], 70, 20, 63, "any"), (784, [8000, 8000], 32, 32, 0, "random"), (40, [96], 5, 24, 7, "any"),
    (30, [60, 3200], 3, 25, 0, "any"), (300, [6800], 16, 17, 0, "random"),
    # 8 and 16 column tiles: the workgroups of a column tile share an XCD (count and finishing kernels)
    (784, [2000, 2000], 1024, 10, 3, "random"), (100, [2560], 2048, 10, 0, "any"),
])
def test_chained_groupbitsum(ext, in_dim, widths, W, k, pad, kind):
    """The count walked along the evaluation schedule against the oracle and the unchained
    fused count, for 16-byte and 8-byte lanes, ragged batches and every kind of wiring."""
    from oracle import connections as oc
    rng = np.random.default_rng(in_dim + W + k + widths[-1])
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, (in_dim, W), dtype=np.int64, endpoint=True)
    layers = random_layers(rng, in_dim, widths)
    top_in = in_dim if len(widths) == 1 else widths[-2]
    torch.manual_seed(k)
    if kind == "random":
        ta, tb = oc.random_connections(top_in, widths[-1])
    elif kind == "unique":
        ta, tb = oc.unique_connections(top_in, widths[-1])
    elif kind == "self":
        ta = torch.as_tensor(layers[-1][0])
        tb = ta.clone()
    else:
        ta, tb = torch.as_tensor(layers[-1][0]), torch.as_tensor(layers[-1][1])
    layers[-1] = (np.asarray(ta), np.asarray(tb), layers[-1][2])
    dev_layers = [tuple(_dev(t) for t in l) for l in layers]
    y = x
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    want = po.groupbitsum(y, pad, k)
    got = ext.eval_chained_groupbitsum(_dev(x), dev_layers, pad, k)
    assert got is not None and got.dtype == torch.int32 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
    assert torch.equal(got, ext.eval_fused_groupbitsum(_dev(x), dev_layers, pad, k))


@pytest.mark.parametrize("top", ["ones", "zeros", "mixed", "one class constant"])
def test_chained_groupbitsum_leaves_constant_neurons_out(ext, top):
    """Neurons of the top layer whose gate is constant are neither parked nor counted; the ones among them are added
    to every sample's count at the end.  All of them constant, none of a class, or every other one: the oracle's counts."""
    rng = np.random.default_rng(5)
    in_dim, widths, W, k, pad = 90, [300, 2400], 5, 12, 9
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, (in_dim, W), dtype=np.int64, endpoint=True)
    layers = random_layers(rng, in_dim, widths)
    a, b, op = layers[-1]
    op = op.copy()
    if top == "ones":
        op[:] = 15
    elif top == "zeros":
        op[:] = 0
    elif top == "mixed":
        op[::2] = np.where(np.arange(len(op[::2])) % 3 == 0, 0, 15)
    else:
        op[200:400] = 15                                     # class 1 of 12 (200 neurons each)
    layers[-1] = (a, b, op)
    dev_layers = [tuple(_dev(t) for t in l) for l in layers]
    y = x
    for la, lb, lop in layers:
        y = po.eval_layer(y, la, lb, lop)
    want = po.groupbitsum(y, pad, k)
    for depth in (2, 1):
        xin = x if depth == 2 else po.eval_layer(x, *layers[0])
        got = ext.eval_chained_groupbitsum(_dev(xin), dev_layers[-depth:], pad, k)
        assert got is not None and np.array_equal(got.cpu().numpy(), want), depth
    if top == "ones":
        assert (want == widths[-1] // k).all()


def test_chained_groupbitsum_declines_where_it_does_not_apply(ext):
    rng = np.random.default_rng(3)
    layers, dev_layers = _chain(rng, 30, [60, 170])
    x = _dev(rng.integers(0, 1 << 62, (30, 2), dtype=np.int64))
    assert ext.eval_chained_groupbitsum(x, dev_layers, 0, 34) is None                 # more classes than the waves own
    assert ext.eval_chained_groupbitsum(x, dev_layers, 0, 10) is not None
    # 3000 neurons on one trail: with 12 classes (250 each) a workgroup walks 16 blocks, with one class as many as
    # keep its count below 256
    a = torch.arange(3000) % 2999
    b = (torch.arange(3000) + 1) % 2999
    sched = ext.schedule_for(_dev(a.numpy()), _dev(b.numpy()), 2999)
    block = ext._lib.load().dl_count_chain_block()
    fit = max(1, 255 // block)
    assert sched.count_plan(12)[3] == 16 and fit // 2 < sched.count_plan(1)[3] <= fit and sched.count_plan(40) is None
    x32 = torch.zeros((30, 3), dtype=torch.int32, device="cuda")
    assert ext.eval_chained_groupbitsum(x32, dev_layers, 0, 10) is None               # rows are not whole 64-bit words


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
def test_gate_ids_match_torch_argmax(ext, dtype):
    """dl_gate_ids against weights.argmax(-1).to(uint8) (difflogic/difflogic.py:146): ties go to the
    first maximal value, a NaN counts as maximal."""
    g = torch.Generator().manual_seed(3)
    w = torch.randn(5000, 16, generator=g)
    w[::7] = torch.randint(0, 3, (w[::7].shape[0], 16), generator=g).float()      # many ties
    w[5, 3] = float("nan")
    w[6, 0] = float("nan")
    w[8, 15] = float("nan")
    w[8, 9] = float("nan")
    w[9] = float("-inf")
    w[10, 4] = float("inf")
    w = w.to(dtype).cuda()
    got = ext.gate_ids(w)
    assert got.dtype == torch.uint8 and torch.equal(got, w.argmax(-1).to(torch.uint8))
    assert ext.gate_ids(w[:0]).shape == (0,)
    with pytest.raises(RuntimeError):
        ext.gate_ids(w[:, :8].contiguous())


@pytest.mark.parametrize("in_dim,widths,B,k", [
    (32, [60], 100, 3),                                   # a single layer: the class phase reads the input rows
    (48, [100, 640], 7 * 64 + 1, 10), (16, [33, 130, 77, 130], 129 * 64 - 5, 2),
    (784, [8000] * 6, 9 * 64 + 3, 10),                    # C2's net: 2 columns per workgroup, odd column count, ragged
    (784, [4000] * 3, 11 * 64, 10),                       # 4 columns per workgroup, 3 columns left over
    (2048, [3000, 8000, 3000], 200, 3),                   # input + widest hidden layer just fit next to each other
    (96, [300, 4096], 5 * 64, 2),                         # 2048 neurons per class: 8 counter planes per lane
    (64, [80, 400], 300, 40),                             # more classes than waves
    (1024, [8190, 8250, 20], 130, 4),                     # schedules around 8192 steps
])
def test_net_lds_from_the_bool_input(ext, in_dim, widths, B, k):
    """dl_logic_net_lds_groupbitsum_bool: packing on the way into LDS gives the counts of packing
    first (any non-zero byte is true), for ragged batches too."""
    rng = np.random.default_rng(in_dim + B + k + widths[-1] + len(widths))
    raw = (rng.integers(0, 256, (B, in_dim), dtype=np.uint8) * (rng.random((B, in_dim)) < 0.4)).astype(np.uint8)
    layers, dev_layers = _chain(rng, in_dim, widths)
    xb = torch.as_tensor(raw).cuda().view(torch.bool)
    got = ext.eval_net_lds_bool(xb, dev_layers, k)
    assert got is not None and got.dtype == torch.int32 and tuple(got.shape) == (B, k)
    words, pad = po.packbits((raw != 0).T, 64)
    y = words
    for a, b, op in layers:
        y = po.eval_layer(y, a, b, op)
    assert np.array_equal(got.cpu().numpy(), po.groupbitsum(y, pad, k))
    packed, pad2 = ext.tensor_packbits_batch_major(xb, 64)
    assert torch.equal(got, ext.eval_net_lds(packed, dev_layers, pad2, k))
    assert torch.equal(got, ext.eval_net_lds_bool(xb, dev_layers, k, scheduled=False))
    assert torch.equal(got, ext.eval_net_lds_bool(xb, dev_layers, k, thin=True))


def test_net_lds_from_the_bool_input_declines_what_does_not_fit(ext):
    rng = np.random.default_rng(4)
    _, dev_layers = _chain(rng, 40, [60, 30])
    assert ext.eval_net_lds_bool(torch.zeros(10, 40, dtype=torch.bool, device="cuda"), dev_layers, 3) is None   # 40 % 16
    _, dev_layers = _chain(rng, 4096, [8000, 30])
    assert ext.eval_net_lds_bool(torch.zeros(10, 4096, dtype=torch.bool, device="cuda"), dev_layers, 3) is None  # no room
    _, dev_layers = _chain(rng, 48, [60, 30])
    assert ext.eval_net_lds_bool(torch.zeros(0, 48, dtype=torch.bool, device="cuda"), dev_layers, 3).shape == (0, 3)
    with pytest.raises(ValueError):
        ext.eval_net_lds_bool(torch.zeros(10, 48, dtype=torch.bool, device="cuda"), dev_layers, 7)


@pytest.mark.parametrize("seed", range(6))
def test_random_nets_end_to_end(seed):
    """Nets of random depth, widths (narrow ones for the LDS kernel, wide ones for the streaming groups), class
    count, word width and batch, through PackBitsTensor and GroupSum as a user runs them, against the oracle."""
    import difflogic_amd as dl
    rng = np.random.default_rng(1000 + seed)
    for case in range(10):
        F = int(rng.integers(1, 70)) if case % 3 else int(rng.integers(1, 9)) * 16
        L = int(rng.integers(1, 8)) if case % 4 else int(rng.integers(1, 5))
        k = int(rng.choice([1, 2, 3, 5, 10, 16]))
        widths, d = [], F
        for i in range(L):
            lo = max(1, (d + 1) // 2)
            w = int(rng.integers(lo, lo + 200)) if case % 4 else int(rng.integers(max(lo, 2000), max(lo, 2000) + 11000))
            if i == L - 1:
                w = -(-w // k) * k
            widths.append(w)
            d = w
        bits = int(rng.choice([8, 16, 32, 64]))
        B = int(rng.choice([1, 7, 63, 64, 65, 200, 1000, 4096, 5000]))
        layers = random_layers(rng, F, widths)
        x = rng.random((B, F)) < 0.5
        want = po.net_eval_bitwise(x, layers, k)
        model = build_model(F, layers, k).eval()
        with torch.no_grad():
            got = model(dl.PackBitsTensor(torch.as_tensor(x).cuda(), bit_count=bits)).cpu().numpy()
        assert got.shape == want.shape and np.array_equal(got, want), (seed, case, F, widths, k, bits, B)
