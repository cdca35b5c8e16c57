"""PackBitsTensor: a batch of boolean feature vectors packed along the batch into integer
words, feature-major (reference: difflogic/packbitstensor.py)."""
import numpy as np
import torch

from . import difflogic_cuda


class PackBitsTensor:
    """``.t`` is int{bit_count} [features, ceil(B / bit_count)]; bit i of word c of a row is
    sample ``bit_count*c + i``; ``.pad_len`` samples at the end of the last word are padding."""

    def __init__(self, t: torch.BoolTensor, bit_count=32, device="cuda"):
        assert len(t.shape) == 2, t.shape
        self.bit_count = bit_count
        self.device = device
        if device == "cuda":
            t = t.to(device)
            if t.dtype == torch.bool and t.is_contiguous():
                # transpose + pack in one kernel
                self.t, self.pad_len = difflogic_cuda.tensor_packbits_batch_major(t, self.bit_count)
            else:
                self.t, self.pad_len = difflogic_cuda.tensor_packbits_cuda(t.T.contiguous(), self.bit_count)
        else:
            raise NotImplementedError(device)

    def group_sum(self, k):
        assert self.device == "cuda", self.device
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
