"""Packed-bit oracle in numpy.  Test infrastructure (see oracle/__init__.py).

Layout, as in the reference's PackBitsTensor (difflogic/packbitstensor.py:15-16): words are
feature-major ``[features, W]`` with ``W = ceil(B / bits)``; bit ``i`` of word ``c`` of a row
is sample ``bits*c + i`` (least significant bit = lowest sample index,
difflogic_kernel.cu:568-576).  Words are signed integers of ``bits`` bits, like torch's.
"""
import numpy as np

from .gates import TRUTH, bit_gate

SIGNED = {8: np.int8, 16: np.int16, 32: np.int32, 64: np.int64}
UNSIGNED = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}


def packbits(t_bool, bits: int = 64):
    """bool [F,B] -> (int{bits} [F,W], pad_len)   (difflogic_kernel.cu:547-625)."""
    if bits not in SIGNED:
        raise ValueError("`bit_count` has to be in { 8, 16, 32, 64 }")
    t = np.asarray(t_bool).astype(bool)
    F, B = t.shape
    W = -(-B // bits)
    pad_len = (bits - B % bits) % bits
    padded = np.zeros((F, W * bits), dtype=UNSIGNED[bits])
    padded[:, :B] = t
    lanes = padded.reshape(F, W, bits)
    out = np.zeros((F, W), dtype=UNSIGNED[bits])
    for i in range(bits):
        out |= lanes[:, :, i] << UNSIGNED[bits](i)
    return out.view(SIGNED[bits]), pad_len


def unpackbits(words, batch: int):
    """int [F,W] -> bool [F,batch]: inverse of packbits (pad samples dropped)."""
    w = np.ascontiguousarray(words)
    bits = w.dtype.itemsize * 8
    u = w.view(UNSIGNED[bits])
    F, W = u.shape
    out = np.zeros((F, W, bits), dtype=bool)
    for i in range(bits):
        out[:, :, i] = (u >> UNSIGNED[bits](i)) & UNSIGNED[bits](1)
    return out.reshape(F, W * bits)[:, :batch]


def eval_layer(x_words, idx_a, idx_b, ops):
    """y[n,c] = op_{ops[n]}(x[a[n],c], x[b[n],c]) on words (difflogic_kernel.cu:437-501).
    Pad bits are *not* kept zero, exactly like the reference (e.g. op 15 sets them)."""
    x = np.ascontiguousarray(x_words)
    bits = x.dtype.itemsize * 8
    xu = x.view(UNSIGNED[bits])
    a, b, ops = (np.asarray(v) for v in (idx_a, idx_b, ops))
    va, vb = xu[a], xu[b]
    y = np.zeros_like(va)
    for i in range(16):
        sel = ops == i
        if sel.any():
            y[sel] = bit_gate(va[sel], vb[sel], i)
    return y.view(SIGNED[bits])


def groupbitsum(words, pad_len: int, k: int):
    """int [out,W] -> int32 [B,k]: per sample, the number of set bits over each class's
    contiguous block of out/k neurons (difflogic_kernel.cu:631-700)."""
    w = np.asarray(words)
    if w.shape[0] % k != 0:
        raise ValueError(f"in_dim ({w.shape[0]}) has to be divisible by k ({k}) but it is not")
    bits = w.dtype.itemsize * 8
    batch = w.shape[1] * bits - pad_len
    bools = unpackbits(w, batch)                                  # [out, B]
    return bools.reshape(k, w.shape[0] // k, batch).sum(1, dtype=np.int64).astype(np.int32).T.copy()


def net_eval_words(x_bool, layers, k: int, bits: int = 64):
    """bool [B,F] -> int32 [B,k] through packbits, eval_layer per layer, groupbitsum.
    ``layers`` is a list of (idx_a, idx_b, ops)."""
    t, pad_len = packbits(np.asarray(x_bool).T, bits)
    for a, b, ops in layers:
        t = eval_layer(t, a, b, ops)
    return groupbitsum(t, pad_len, k)


def net_eval_bitwise(x_bool, layers, k: int):
    """The same function one boolean at a time from the truth table alone: no words, no
    bitwise gate forms.  Slow; for tiny cases that pin the word-level functions."""
    x = np.asarray(x_bool).astype(np.int64)                       # [B,F]
    for a, b, ops in layers:
        a, b, ops = (np.asarray(v) for v in (a, b, ops))
        x = TRUTH[ops[None, :], x[:, a], x[:, b]]
    B, out = x.shape
    return x.reshape(B, k, out // k).sum(-1).astype(np.int32)
