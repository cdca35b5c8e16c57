"""Pins the packed-bit oracle (numpy words, C interpreter, generated C) against library
routines, brute force, and each other."""
import itertools

import numpy as np
import pytest

from oracle import cgen, interp
from oracle import packed_oracle as po
from oracle.gates import TRUTH


def _net(rng, F, widths):
    layers, d = [], F
    for o in widths:
        layers.append((rng.integers(0, d, o), rng.integers(0, d, o), rng.integers(0, 16, o).astype(np.uint8)))
        d = o
    return layers


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("B", [1, 7, 64, 65, 200])
def test_packbits_is_numpy_packbits_little(bits, B):
    rng = np.random.default_rng(B * 100 + bits)
    t = rng.random((5, B)) < 0.4
    words, pad = po.packbits(t, bits)
    assert pad == (bits - B % bits) % bits and words.shape == (5, -(-B // bits))
    ref = np.ascontiguousarray(np.packbits(np.pad(t, ((0, 0), (0, pad))), axis=1, bitorder="little"))
    assert (words.view(np.uint8) == ref).all()           # little-endian words == LSB-first bytes
    assert (po.unpackbits(words, B) == t).all()


def test_packbits_rejects_other_widths():
    with pytest.raises(ValueError):
        po.packbits(np.zeros((1, 8), bool), 12)


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
def test_eval_layer_brute_force_all_ops_all_inputs(bits):
    # 2 input rows holding the four (a,b) combinations in 4 sample positions, all 16 ops
    t = np.array([[0, 0, 1, 1], [0, 1, 0, 1]], dtype=bool)
    x, _ = po.packbits(t, bits)
    ops = np.arange(16, dtype=np.uint8)
    y = po.eval_layer(x, np.zeros(16, int), np.ones(16, int), ops)
    got = po.unpackbits(y, 4)
    for i, (k, (a, b)) in itertools.product(range(16), enumerate(itertools.product((0, 1), repeat=2))):
        assert got[i, k] == TRUTH[i, a, b]


def test_eval_layer_pad_bits_follow_the_gate():
    x, pad = po.packbits(np.zeros((2, 3), bool), 8)
    y = po.eval_layer(x, [0], [1], [15])
    assert pad == 5 and y.view(np.uint8)[0, 0] == 0xFF    # constant-1 sets the pad bits too
    assert (po.groupbitsum(y, pad, 1) == 1).all() and po.groupbitsum(y, pad, 1).shape == (3, 1)


def test_groupbitsum_against_unpackbits():
    rng = np.random.default_rng(3)
    t = rng.random((30, 150)) < 0.5
    words, pad = po.packbits(t, 64)
    got = po.groupbitsum(words, pad, 5)
    bits = np.unpackbits(np.ascontiguousarray(words).view(np.uint8), axis=1, bitorder="little")[:, :150]
    want = bits.reshape(5, 6, 150).sum(1).T
    assert got.dtype == np.int32 and (got == want).all()
    with pytest.raises(ValueError):
        po.groupbitsum(words, pad, 7)


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
def test_word_net_equals_bit_at_a_time(bits):
    rng = np.random.default_rng(bits)
    layers = _net(rng, 12, [24, 24, 30])
    x = rng.random((150, 12)) < 0.3
    assert (po.net_eval_words(x, layers, 3, bits) == po.net_eval_bitwise(x, layers, 3)).all()


@pytest.mark.parametrize("B", [1, 63, 64, 65, 300])
def test_c_interpreter_equals_bit_at_a_time(B):
    rng = np.random.default_rng(B)
    layers = _net(rng, 17, [40, 35, 50])
    x = rng.random((B, 17)) < 0.3
    want = po.net_eval_bitwise(x, layers, 5)
    assert (interp.net_eval(x, layers, 5) == want).all()
    assert (interp.net_eval(x, layers, 5, threads=3) == want).all()


def test_c_interpreter_layer_equals_numpy_layer():
    rng = np.random.default_rng(0)
    x = rng.integers(-2**63, 2**63 - 1, (20, 9), dtype=np.int64)
    a, b, ops = rng.integers(0, 20, 50), rng.integers(0, 20, 50), rng.integers(0, 16, 50)
    assert (interp.eval_layer(x, a, b, ops) == po.eval_layer(x, a, b, ops)).all()


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
def test_generated_c_equals_bit_at_a_time(bits):
    rng = np.random.default_rng(bits + 7)
    layers = _net(rng, 12, [24, 24, 30])
    x = rng.random((150, 12)) < 0.3
    net = cgen.CompiledNet(layers, 12, 3, bits)
    assert (net(x) == po.net_eval_bitwise(x, layers, 3)).all()


def test_generated_c_single_layer_and_counter_width():
    # counts up to the class size need ceil(log2(size+1)) planes: 7 neurons -> 3, 8 -> 4
    rng = np.random.default_rng(1)
    for per_class in (7, 8):
        layers = [(rng.integers(0, 6, 2 * per_class), rng.integers(0, 6, 2 * per_class),
                   np.full(2 * per_class, 15, np.uint8))]
        x = rng.random((64, 6)) < 0.5
        net = cgen.CompiledNet(layers, 6, 2, 64)
        assert (net(x) == per_class).all()
        assert (interp.net_eval(x, layers, 2) == per_class).all()
