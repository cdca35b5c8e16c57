"""Pins the oracle's three statements of the 16 gates against the truth table alone."""
import itertools

import numpy as np
import pytest
import torch

from oracle import float_oracle as fo
from oracle.gates import NUM_GATES, TRUTH, bit_gate, real_gate, truth


def test_truth_rows_are_binary_expansion():
    for i in range(NUM_GATES):
        row = [truth(i, 0, 0), truth(i, 0, 1), truth(i, 1, 0), truth(i, 1, 1)]
        assert row == [int(c) for c in format(i, "04b")]
        assert (TRUTH[i].reshape(-1) == row).all()
    # spot names: 1 = AND, 6 = XOR, 7 = OR, 3 = A, 5 = B, 14 = NAND
    assert [truth(1, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [0, 0, 0, 1]
    assert [truth(6, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [0, 1, 1, 0]
    assert [truth(7, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [0, 1, 1, 1]
    assert [truth(3, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [0, 0, 1, 1]
    assert [truth(5, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [0, 1, 0, 1]
    assert [truth(14, a, b) for a, b in itertools.product((0, 1), repeat=2)] == [1, 1, 1, 0]


@pytest.mark.parametrize("i", range(NUM_GATES))
def test_real_gate_is_the_tables_multilinear_extension(i):
    # value on the corners
    for a, b in itertools.product((0.0, 1.0), repeat=2):
        assert float(real_gate(np.float64(a), np.float64(b), i)) == TRUTH[i, int(a), int(b)]
    # multilinear: affine in a for fixed b, and in b for fixed a  => second differences vanish
    rng = np.random.default_rng(i)
    a, b, h = rng.random(50), rng.random(50), 0.37
    f = lambda u, v: real_gate(u, v, i)
    assert np.allclose(f(a + h, b) - 2 * f(a, b) + f(a - h, b), 0, atol=1e-12)
    assert np.allclose(f(a, b + h) - 2 * f(a, b) + f(a, b - h), 0, atol=1e-12)


@pytest.mark.parametrize("i", range(NUM_GATES))
@pytest.mark.parametrize("bits", [8, 16, 32, 64])
def test_bit_gate_matches_table(i, bits):
    dt = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]
    ones = dt(np.iinfo(dt).max)
    for a, b in itertools.product((0, 1), repeat=2):
        wa = np.array([ones if a else 0], dtype=dt)
        wb = np.array([ones if b else 0], dtype=dt)
        got = bit_gate(wa, wb, i)
        assert got.dtype == dt
        assert got[0] == (ones if TRUTH[i, a, b] else 0)


def test_sequential_equals_multilinear_closed_form():
    torch.manual_seed(0)
    x = torch.rand(33, 20, dtype=torch.float64)
    a = torch.randint(0, 20, (50,))
    b = torch.randint(0, 20, (50,))
    w = torch.softmax(torch.randn(50, 16, dtype=torch.float64), -1)
    y1 = fo.layer_forward_sequential(x, a, b, w)
    y2 = fo.layer_forward_multilinear(x, a, b, w)
    assert torch.allclose(y1, y2, atol=1e-14)


def test_one_hot_on_binary_inputs_is_the_boolean_gate():
    torch.manual_seed(1)
    x = (torch.rand(64, 10) < 0.5).float()
    a = torch.randint(0, 10, (160,))
    b = torch.randint(0, 10, (160,))
    ops = torch.arange(160) % 16
    w = torch.nn.functional.one_hot(ops, 16).float()
    y = fo.layer_forward_sequential(x, a, b, w)
    want = TRUTH[ops.numpy()[None, :], x[:, a].long().numpy(), x[:, b].long().numpy()]
    assert (y.numpy() == want).all()
