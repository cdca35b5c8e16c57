"""PackBitsTensor: a batch of boolean feature vectors packed along the batch into integer
words, feature-major (reference: difflogic/packbitstensor.py)."""
import numpy as np
import torch

from . import difflogic_cuda


class PackBitsTensor:
    """``.t`` is int{bit_count} [features, ceil(B / bit_count)]; bit i of word c of a row is
    sample ``bit_count*c + i``; ``.pad_len`` samples at the end of the last word are padding.

    The most recent LogicLayer applied to the object is held back (``defer_layer``) until
    ``.t`` is read or ``group_sum`` is called, so that a layer followed directly by GroupSum
    runs as one fused kernel and its output words are never written to memory.  Reading
    ``.t`` always returns the up-to-date words, as in the reference."""

    def __init__(self, t: torch.BoolTensor, bit_count=32, device="cuda"):
        assert len(t.shape) == 2, t.shape
        self.bit_count = bit_count
        self.device = device
        self._t = None
        self._pending = None          # (a, b, w) of a layer applied to _t but not yet evaluated
        if device == "cuda":
            t = t.to(device)
            if t.dtype == torch.bool and t.is_contiguous():
                # transpose + pack in one kernel
                self.t, self.pad_len = difflogic_cuda.tensor_packbits_batch_major(t, self.bit_count)
            else:
                self.t, self.pad_len = difflogic_cuda.tensor_packbits_cuda(t.T.contiguous(), self.bit_count)
        else:
            raise NotImplementedError(device)

    @property
    def t(self):
        if self._pending is not None:
            a, b, w = self._pending
            self._pending = None
            self._t = difflogic_cuda.eval(self._t, a, b, w)
        return self._t

    @t.setter
    def t(self, value):
        self._pending = None
        self._t = value

    def defer_layer(self, a, b, w):
        """Applies the gate layer (a, b, w) lazily: evaluates any earlier deferred layer now and
        holds this one back."""
        self._t = self.t
        self._pending = (a, b, w)
        return self

    def group_sum(self, k):
        assert self.device == "cuda", self.device
        if self._pending is not None:
            a, b, w = self._pending
            if w.shape[0] % k != 0:
                raise ValueError(f"in_dim ({w.shape[0]}) has to be divisible by k ({k}) but it is not")
            return difflogic_cuda.eval_groupbitsum(self._t, a, b, w, self.pad_len, k)
        return difflogic_cuda.groupbitsum(self.t, self.pad_len, k)

    def flatten(self, start_dim=0, end_dim=-1, **kwargs):
        """Returns the object itself; the arguments are ignored."""
        return self

    def _row_repr(self, row):
        def word(v):
            return np.binary_repr(int(v), width=self.bit_count)[::-1]     # lowest sample first
        if len(row) <= 4:
            return " ".join(word(v) for v in row)
        return "{} ... {}".format(" ".join(word(v) for v in row[:3]), word(row[-1]))

    def __repr__(self):
        return "\n".join(self._row_repr(row) for row in self.t.cpu().numpy())
