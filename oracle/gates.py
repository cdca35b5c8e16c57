"""The 16 two-input gates, stated three ways.  Test infrastructure (see oracle/__init__.py).

Gate ``i`` has the truth table whose row (f(0,0), f(0,1), f(1,0), f(1,1)) is the 4-bit
binary expansion of ``i``, most significant bit first (reference table:
difflogic/functional.py:7-24, repeated at difflogic/cuda/difflogic_kernel.cu:418-435).
"""
import numpy as np

NUM_GATES = 16

GATE_NAMES = (
    "0", "a&b", "a&~b", "a", "~a&b", "b", "a^b", "a|b",
    "~(a|b)", "~(a^b)", "~b", "a|~b", "~a", "~a|b", "~(a&b)", "1",
)


def truth(i: int, a: int, b: int) -> int:
    """f_i(a, b) for a, b in {0, 1}: bit (3 - 2a - b) of i."""
    return (i >> (3 - 2 * a - b)) & 1


# TRUTH[i, a, b]
TRUTH = np.array([[[truth(i, a, b) for b in (0, 1)] for a in (0, 1)] for i in range(NUM_GATES)],
                 dtype=np.int64)


def real_gate(a, b, i: int):
    """Real-valued relaxation of gate i, term for term as the reference writes it
    (difflogic/functional.py:31-62).  Works on torch tensors and numpy arrays."""
    if i == 0:
        return a * 0
    if i == 1:
        return a * b
    if i == 2:
        return a - a * b
    if i == 3:
        return a
    if i == 4:
        return b - a * b
    if i == 5:
        return b
    if i == 6:
        return a + b - 2 * a * b
    if i == 7:
        return a + b - a * b
    if i == 8:
        return 1 - (a + b - a * b)
    if i == 9:
        return 1 - (a + b - 2 * a * b)
    if i == 10:
        return 1 - b
    if i == 11:
        return 1 - b + a * b
    if i == 12:
        return 1 - a
    if i == 13:
        return 1 - a + a * b
    if i == 14:
        return 1 - a * b
    if i == 15:
        return a * 0 + 1
    raise ValueError(i)


def bit_gate(a, b, i: int):
    """Bitwise form of gate i on integer words (numpy unsigned arrays or Python ints
    masked by the caller), as in difflogic/cuda/difflogic_kernel.cu:437-472 and
    difflogic/compiled_model.py:97-128."""
    if i == 0:
        return a & ~a
    if i == 1:
        return a & b
    if i == 2:
        return a & ~b
    if i == 3:
        return a
    if i == 4:
        return b & ~a
    if i == 5:
        return b
    if i == 6:
        return a ^ b
    if i == 7:
        return a | b
    if i == 8:
        return ~(a | b)
    if i == 9:
        return ~(a ^ b)
    if i == 10:
        return ~b
    if i == 11:
        return ~b | a
    if i == 12:
        return ~a
    if i == 13:
        return ~a | b
    if i == 14:
        return ~(a & b)
    if i == 15:
        return ~(a & ~a)
    raise ValueError(i)
