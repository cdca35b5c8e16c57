"""PackBitsTensor: a batch of boolean feature vectors packed along the batch into integer
words, feature-major (reference: difflogic/packbitstensor.py)."""
import numpy as np
import torch

from . import difflogic_cuda

# Inputs with at most this many rows stay resident in the L2 caches while a 1 KB column tile of
# all neurons is swept, so gathers from them are cheap and deeper fusion pays off.
_L2_RESIDENT_ROWS = 2048


def _chained(depth):
    """Groups of two or more layers run along the top layer's evaluation schedule."""
    return depth >= 2


def plan_groups(dims, count_at_end):
    """Splits consecutive layers into fused groups.

    ``dims`` = [in_dim, width_1, ..., width_L].  Returns a list of group sizes summing to L; when
    ``count_at_end`` the last group is the one fused with the bit count.  Chosen by dynamic
    programming over a traffic model: a group of depth D gathers 2^D rows per output neuron,
    2^(D-1) when it runs chained, from L2 when its input has few rows and through the memory fabric
    otherwise, and writes one row per output neuron unless it ends in the count."""
    n = len(dims) - 1
    if n == 0:
        return []

    def cost(first, depth, last):
        # milliseconds per 64000 rows of 16384 words, fitted to launches measured on MI355X
        rows_in, out = dims[first], dims[first + depth]
        counted = last and count_at_end
        gathers = (1 << depth) * out
        if _chained(depth) and not counted:
            gathers = gathers * 9 / 16             # half, plus one extra subtree per chunk of 8
        written = 0 if counted else out
        if rows_in <= _L2_RESIDENT_ROWS:           # gathers hit in L2; writes stream to HBM
            t = max(1.5 * written, 0.3 * gathers + 0.5 * out)
        else:                                      # L2 <-> fabric traffic, with the HBM copy rate as floor
            t = max(1.1 * (gathers + written), 1.68 * (rows_in + written))
        if counted:
            t += 0.2 * out                         # second pass over the partial counters
        return t

    best = [(0.0, [])] + [None] * n    # best[i] = (cost, groups) for the first i layers
    for i in range(1, n + 1):
        for depth in range(1, min(i, difflogic_cuda.MAX_FUSE_DEPTH) + 1):
            last = i == n
            if last and count_at_end and depth > difflogic_cuda.MAX_FUSE_DEPTH_COUNT:
                continue
            prev = best[i - depth]
            c = prev[0] + cost(i - depth, depth, last)
            if best[i] is None or c < best[i][0]:
                best[i] = (c, prev[1] + [depth])
    return best[n][1]


def lds_tail(dims):
    """Number of layers at the end of the net (``dims`` = [in_dim, width_1, ..., width_L]) that the
    LDS-resident whole-net kernel takes together with the count: the longest run of trailing layers
    whose input and widths all fit its buffer, if that run is at least two layers long (a single
    layer gains nothing over the streaming kernel fused with the count)."""
    limit = difflogic_cuda.net_lds_max_width()
    n = 0
    while n < len(dims) - 1 and n < difflogic_cuda.MAX_NET_DEPTH and max(dims[len(dims) - 2 - n:]) <= limit:
        n += 1
    return n if n >= 2 else 0


class PackBitsTensor:
    """``.t`` is int{bit_count} [features, ceil(B / bit_count)]; bit i of word c of a row is
    sample ``bit_count*c + i``; ``.pad_len`` samples at the end of the last word are padding.

    Layers applied to the object are held back (``defer_layer``) until ``.t`` is read or
    ``group_sum`` is called; consecutive layers are then evaluated in fused groups (and the last
    group together with the bit count), so most intermediate activations never reach memory.
    Reading ``.t`` always returns the up-to-date words, as in the reference."""

    def __init__(self, t: torch.BoolTensor, bit_count=32, device="cuda"):
        assert len(t.shape) == 2, t.shape
        self.bit_count = bit_count
        self.device = device
        self._t = None
        self._pending = []            # [(a, b, w)] applied to _t but not yet evaluated
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
    def features(self):
        """Number of rows ``.t`` has (after the deferred layers)."""
        return self._pending[-1][2].shape[0] if self._pending else self._t.shape[0]

    def _dims(self):
        return [self._t.shape[0]] + [w.shape[0] for _, _, w in self._pending]

    def _run_groups(self, groups):
        pos = 0
        for depth in groups:
            run = difflogic_cuda.eval_chained if _chained(depth) else difflogic_cuda.eval_fused
            self._t = run(self._t, self._pending[pos:pos + depth])
            pos += depth
        self._pending = self._pending[pos:]

    @property
    def t(self):
        if self._pending:
            self._run_groups(plan_groups(self._dims(), count_at_end=False))
        return self._t

    @t.setter
    def t(self, value):
        self._pending = []
        self._t = value

    def defer_layer(self, a, b, w):
        """Applies the gate layer (a, b, w) lazily."""
        self._pending.append((a, b, w))
        return self

    def group_sum(self, k):
        assert self.device == "cuda", self.device
        if self._pending:
            if self.features % k != 0:
                raise ValueError(f"in_dim ({self.features}) has to be divisible by k ({k}) but it is not")
            dims = self._dims()
            tail = lds_tail(dims)
            if tail:
                # the narrow end of the net runs resident in LDS; what lies before it streams
                head = len(self._pending) - tail
                if head:
                    self._run_groups(plan_groups(dims[:head + 1], count_at_end=False))
                out = difflogic_cuda.eval_net_lds(self._t, self._pending, self.pad_len, k)
                if out is not None:
                    return out
            groups = plan_groups(self._dims(), count_at_end=True)
            self._run_groups(groups[:-1])
            # the last group stays pending: the object's state does not change by counting
            out = difflogic_cuda.eval_chained_groupbitsum(self._t, self._pending, self.pad_len, k)
            if out is not None:
                return out
            order = difflogic_cuda.count_order_for(self._pending, self._t.shape[0], k)
            return difflogic_cuda.eval_fused_groupbitsum(self._t, self._pending, self.pad_len, k, order)
        return difflogic_cuda.groupbitsum(self._t, self.pad_len, k)

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
