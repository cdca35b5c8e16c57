"""PackBitsTensor: a batch of boolean feature vectors packed along the batch into integer
words, feature-major (reference: difflogic/packbitstensor.py)."""
import functools

import numpy as np
import torch

from . import difflogic_cuda

# ---------------------------------------------------------------------------------------------
# Launch planning.  The cost of a fused group is modelled from the bytes it moves through each
# level of the memory system, at the rates plain kernels with the same access pattern sustain on
# MI355X (`python bench.py --ceilings`; profiles/ceilings_mi355x.txt), so the plan follows the
# shapes (rows, widths, words per row) instead of constants fitted to one workload.
# ---------------------------------------------------------------------------------------------
_L2_GATHER_RATE = 31e12      # B/s: row gathers + stores through the L2s when the input tile stays L2-resident
_FABRIC_RATE = 7.5e12        # B/s: row gathers + stores between the L2s and Infinity Cache / HBM
_WRITE_RATE = 6.1e12         # B/s: streaming stores to HBM
_COUNT_RATE = 5.6e12         # B/s of counted rows: what the chained count kernel parks in LDS, sorts by class and adds up
_LIVE_INPUT = 0.75           # share of gate inputs a gate looks at when the gate ids are uniform (10 of 16 gates use both
                             # inputs, 4 one, 2 none); rows that no gate looks at are not fetched.  The default where
                             # the net's own share has not been measured (PackBitsTensor._live_share)
_TILE_BYTES = 1024           # one wave covers 64 lanes x 16 bytes of a row
_L2_RESIDENT_BYTES = 4 << 20     # input tiles (rows x 1 KB each) in flight up to this size are re-read from L2 (4 MB per XCD)
_LDS_GATE_WORD_SECONDS = 7.9e-13     # LDS-resident whole-net kernel: seconds per gate and 64-sample word
_LDS_THIN_BELOW = 0.9        # share of looked-at gate inputs below which the LDS kernel runs the net thinned for the call
                             # (neuron by neuron over the neurons left) instead of whole along its schedules
_LDS_THIN_GAIN = 0.78        # what thinning leaves of the gates' time: measured 0.61-0.63 ms against 0.74 ms on
                             # 784 -> 6 x 8000 for shares of 0.5 to 0.75 (all looked at: 0.77 ms, hence the threshold)
_BOOL_STAGE_RATE = 5.2e12    # B/s of bool input bytes that the LDS kernel packs on their way into LDS
_PACKED_STAGE_RATE = 1.5e12  # B/s of packed input rows on their way into LDS (16 or 32 bytes of every row per workgroup)
_PACK_RATE = 4.8e12          # B/s (bool bytes read + words written) of the transpose-and-pack kernel
_STREAM_CALL_SECONDS = 6e-5  # per call of the streaming path: constant folding, liveness and record kernels
_LAUNCH_SECONDS = 3e-6       # per kernel on the stream; decides between plans for small batches only


def _chained(depth):
    """Groups of two or more layers run along the top layer's evaluation schedule."""
    return depth >= 2


def group_cost(rows_in, out, depth, words, counted, live=_LIVE_INPUT):
    """Modelled seconds of one fused group: `depth` layers from `rows_in` input rows to `out` output
    rows of `words` 64-bit words, ending in the per-class count when `counted`.  ``live``: share of the gate
    inputs that their gate looks at (1.0: two-input gates only)."""
    row_bytes = 8.0 * words
    # rows gathered per output row: the leaves of a tree of gates that are looked at.  Along a schedule the tree is
    # the subtree under the vertex two consecutive neurons share (needed unless both ignore it).
    shared_needed = 1 - (1 - live) ** 2
    if counted:                                    # walked along the schedule: one seed per 128 steps
        gathers = (2 * live) ** (depth - 1) * shared_needed * (1 + 1 / 128) * out
    elif _chained(depth):                          # one seed per 32 steps
        gathers = (2 * live) ** (depth - 1) * shared_needed * (1 + 1 / 32) * out
    else:
        gathers = (2 * live) ** depth * out
    gathered = gathers * row_bytes
    written = 0.0 if counted else out * row_bytes
    # The chip sweeps all output rows of one 1 KB column tile before the next, but a narrow layer
    # does not fill it: several tiles are then in flight and their input rows share the L2s.
    steps_per_workgroup = 1024 if counted else 64
    resident_workgroups = 256 if counted else 2048
    tiles_in_flight = max(1.0, resident_workgroups * steps_per_workgroup / max(out, 1))
    hit = min(1.0, _L2_RESIDENT_BYTES / (rows_in * _TILE_BYTES * tiles_in_flight))     # share of gathers served by L2
    through_l2 = (hit * gathered + written) / _L2_GATHER_RATE
    beyond_l2 = ((1 - hit) * gathered + written) / (_WRITE_RATE if hit == 1.0 else _FABRIC_RATE)
    t = max(through_l2, beyond_l2) + 0.3 * min(through_l2, beyond_l2)                  # the two overlap only in part
    if counted:
        counting = out * row_bytes / _COUNT_RATE                         # overlaps with the gathers only in part, too
        t = max(t, counting) + 0.3 * min(t, counting)
        t += 2 * (out / 128.0) * row_bytes / _FABRIC_RATE                # partial counters: written, then read once
    # kernels on the stream: the per-call table builders, the group's kernel, the count's second pass
    return t + _LAUNCH_SECONDS * (3 if counted or _chained(depth) else 1)


def plan_groups(dims, count_at_end, words=16384, live=_LIVE_INPUT):
    """Splits consecutive layers into fused groups.

    ``dims`` = [in_dim, width_1, ..., width_L]; ``words`` = 64-bit words per row.  Returns a list of
    group sizes summing to L; when ``count_at_end`` the last group is the one fused with the bit
    count.  Chosen by dynamic programming over group_cost (remembered per shape: a call on a small batch is
    bound by the host)."""
    return list(_plan_groups(tuple(dims), bool(count_at_end), int(words), float(live)))


@functools.lru_cache(maxsize=512)
def _plan_groups(dims, count_at_end, words, live):
    n = len(dims) - 1
    if n == 0:
        return []
    best = [(0.0, [])] + [None] * n    # best[i] = (cost, groups) for the first i layers
    for i in range(1, n + 1):
        for depth in range(1, min(i, difflogic_cuda.MAX_FUSE_DEPTH) + 1):
            counted = i == n and count_at_end
            if counted and depth > difflogic_cuda.MAX_FUSE_DEPTH_COUNT:
                continue
            prev = best[i - depth]
            c = prev[0] + group_cost(dims[i - depth], dims[i], depth, words, counted, live)
            if best[i] is None or c < best[i][0]:
                best[i] = (c, prev[1] + [depth])
    return best[n][1]


def plan_cost(dims, groups, count_at_end, words=16384, live=_LIVE_INPUT):
    """Modelled seconds of running ``groups`` (as plan_groups returns them) over ``dims``."""
    t, pos = 0.0, 0
    for j, depth in enumerate(groups):
        t += group_cost(dims[pos], dims[pos + depth], depth, words, count_at_end and j == len(groups) - 1, live)
        pos += depth
    return t


def lds_cost(dims, words, from_bool=False, live=1.0):
    """Modelled seconds of the LDS-resident whole-net kernel over all of ``dims``; ``from_bool``: it reads the bool
    input itself (64 bytes per word and feature) instead of packed words; ``live``: the share of gate inputs that
    are looked at (decides whether the net is thinned for the call)."""
    staging = dims[0] * words * (64 / _BOOL_STAGE_RATE if from_bool else 8 / _PACKED_STAGE_RATE)
    gates = sum(dims[1:]) * words * _LDS_GATE_WORD_SECONDS * (_LDS_THIN_GAIN if live < _LDS_THIN_BELOW else 1.0)
    return gates + staging + 2 * _LAUNCH_SECONDS


def lds_tail(dims, words=16384, live=_LIVE_INPUT, from_bool=False):
    """Number of layers at the end of the net (``dims`` = [in_dim, width_1, ..., width_L]) to run
    in the LDS-resident whole-net kernel together with the count: the longest run of trailing
    layers whose input and widths all fit its buffer, if the model prices it below the streaming
    plan for the same layers (0 otherwise).  Both skip what no gate looks at (the LDS kernel by thinning the net
    for the call when ``live`` is low enough to pay for it).
    ``from_bool``: the input has not been packed yet; if the whole net runs in LDS it never is, while the
    streaming kernels need the pack kernel first.  (Remembered per shape, like plan_groups.)"""
    return _lds_tail(tuple(dims), int(words), float(live), bool(from_bool))


@functools.lru_cache(maxsize=512)
def _lds_tail(dims, words, live, from_bool):
    limit = difflogic_cuda.net_lds_max_width()
    n = 0
    while n < len(dims) - 1 and n < difflogic_cuda.MAX_NET_DEPTH and max(dims[len(dims) - 2 - n:]) <= limit:
        n += 1
    if n == 0:
        return 0
    tail = dims[len(dims) - 1 - n:]
    whole = from_bool and n == len(dims) - 1
    streaming = plan_cost(tail, plan_groups(tail, True, words, live), True, words, live) + _STREAM_CALL_SECONDS
    if whole:
        streaming += dims[0] * words * 72 / _PACK_RATE
    return n if lds_cost(tail, words, whole, live) < streaming else 0


# share of the gate inputs that their gate looks at, per set of weight tensors (see PackBitsTensor._live_share)
_LIVE_SHARES = {}
_USES_INPUTS = (0, 2, 2, 1, 2, 1, 2, 2, 2, 2, 1, 2, 1, 2, 2, 0)      # inputs gate id i looks at


def measured_live_share(layers):
    """Share of the gate inputs of ``layers`` = [(a, b, gate ids), ...] that their gate looks at (0.75 for uniformly
    drawn ids, 1.0 for two-input gates only, 0.5 for pass-through gates only).  Reads the device: one
    synchronisation."""
    ids = torch.cat([w.reshape(-1) for _, _, w in layers]).long()
    uses = torch.tensor(_USES_INPUTS, dtype=torch.float32, device=ids.device)
    return float(uses[ids].mean().item()) / 2 if ids.numel() else _LIVE_INPUT


class PackBitsTensor:
    """``.t`` is int{bit_count} [features, ceil(B / bit_count)]; bit i of word c of a row is
    sample ``bit_count*c + i``; ``.pad_len`` samples at the end of the last word are padding.

    Layers applied to the object are held back (``defer_layer``) until ``.t`` is read or
    ``group_sum`` is called; consecutive layers are then evaluated in fused groups (and the last
    group together with the bit count), so most intermediate activations never reach memory.
    Reading ``.t`` always returns the up-to-date words, as in the reference.

    Inside, a row is a little-endian bit stream padded with zeros to a multiple of 16 bytes and held
    as int64 words: the same bytes as words of any of the four widths, so every batch size and word
    width runs the same vector kernels.  ``.t`` is a view of those rows where their length allows
    it and a copy cut to ``ceil(B / bit_count)`` words otherwise."""

    def __init__(self, t: torch.BoolTensor, bit_count=32, device="cuda"):
        assert len(t.shape) == 2, t.shape
        self.bit_count = bit_count
        self.device = device
        self._src = None              # the bool input [B, F] while it has not been packed yet
        self._rows = None             # int64 [features, 2 * ceil(B / 128)]: the padded rows
        self._public = None           # what `.t` handed out or was set to, while it is current
        self._pending = []            # [(a, b, w)] applied to the rows but not yet evaluated
        self._keys = []               # per pending layer: what identifies the weights its gate ids came from, or None
        self._folded = True           # constants folded through the pending layers' gate ids (_fold_pending)
        self._state = None            # which rows of the deferred result are constant (uint8 [features]: 0 varies, 1 all
                                      # zeros, 2 all ones), where the layers that made it said so; None: not known
        if device == "cuda":
            if bit_count not in (8, 16, 32, 64):
                raise ValueError("`bit_count` has to be in { 8, 16, 32, 64 }")
            t = t.to(device)
            self._batch = t.shape[0]
            self.pad_len = (bit_count - t.shape[0] % bit_count) % bit_count
            if t.dtype == torch.bool and t.is_contiguous():
                # packed (transpose + pack in one kernel) when the words are first needed: a narrow net
                # that runs resident in LDS reads the bool input itself
                self._src = t
            else:
                self._public, self.pad_len = difflogic_cuda.tensor_packbits_cuda(t.T.contiguous(), self.bit_count)
        else:
            raise NotImplementedError(device)

    @staticmethod
    def _row_bytes(batch):
        """Length of a padded row: whole 16-byte vectors; from 2 KB on whole 128-byte lines, so that every row starts
        on a line and the 1 KB piece of a row that a wave reads is 8 lines, not 9 (batch 10^6 on the 784 -> 6 x 64000
        net: 2.70 -> 2.48 ns per sample; at most 6 % more columns)."""
        n = 16 * -(-batch // 128)
        return n if n < 2048 else 128 * -(-n // 128)

    def _adopt(self, value):
        """(rows, shared): ``value`` (words as `.t` shows them) as padded int64 rows; ``shared`` says
        whether the rows are the same memory."""
        bits = difflogic_cuda._WORD_BITS.get(value.dtype)
        if bits is None or value.dim() != 2:
            raise RuntimeError(f"expected 2-D integer words, got {value.dtype} with {value.dim()} dims")
        row_bytes = value.shape[1] * bits // 8
        if row_bytes % 16 == 0 and value.is_contiguous() and value.data_ptr() % 16 == 0:
            return value.view(torch.int64), True
        rows = torch.zeros((value.shape[0], 2 * -(-row_bytes // 16)), dtype=torch.int64, device=value.device)
        rows.view(torch.uint8)[:, :row_bytes] = value.contiguous().view(torch.uint8)
        return rows, False

    def _words(self):
        """The padded rows, packing the bool input now if that has not happened yet."""
        if self._rows is not None:
            return self._rows
        if self._public is not None:
            rows, shared = self._adopt(self._public)
            if shared:
                self._rows = rows
            return rows               # a copy is not kept: writes into `.t` have to stay visible
        self._rows = difflogic_cuda.tensor_packbits_batch_major_rows(self._src, self._row_bytes(self._batch))
        self._src = None
        return self._rows

    def _pad(self, rows):
        """Padding bits at the end of a padded row."""
        return rows.shape[1] * 64 - self._batch

    def _in_features(self):
        for held in (self._rows, self._public):
            if held is not None:
                return held.shape[0]
        return self._src.shape[1]

    @property
    def features(self):
        """Number of rows ``.t`` has (after the deferred layers)."""
        return self._pending[-1][2].shape[0] if self._pending else self._in_features()

    def _words64(self):
        """Row length in 64-bit words (what the planner's byte counts are based on)."""
        return max(1, self._row_bytes(self._batch) // 8)

    def _dims(self):
        return [self._in_features()] + [w.shape[0] for _, _, w in self._pending]

    def _fold_pending(self):
        """Before the streaming kernels run: constants folded through the deferred layers' gate ids, so that the
        kernels fetch nothing for inputs that are constant (same words, bit for bit)."""
        if not self._folded and self._pending:
            self._pending = difflogic_cuda.fold_gate_constants(self._pending)
        self._folded = True

    def _live_share(self):
        """Share of the pending layers' gate inputs that their gate looks at, for the launch planner.  Measured
        once per set of weight tensors (and their version counters) and remembered: a stale or default value
        changes the plan, never the result.  The default where it cannot be measured without disturbing the
        caller (weights of unknown origin, a stream being captured into a graph)."""
        if not self._pending or any(k is None for k in self._keys):
            return _LIVE_INPUT
        key = tuple(self._keys)
        share = _LIVE_SHARES.get(key)
        if share is None:
            if torch.cuda.is_current_stream_capturing():
                return _LIVE_INPUT
            share = measured_live_share(self._pending)
            if len(_LIVE_SHARES) >= 256:
                _LIVE_SHARES.clear()
            _LIVE_SHARES[key] = share
        return share

    def _run_groups(self, groups, live=None):
        """Evaluates the first sum(groups) pending layers group by group.  ``live`` (difflogic_cuda.live_inputs of
        the pending layers): rows that the layers still pending afterwards do not look at need not be written; the
        rows then kept are for those layers only (`.t` of them is never handed out: reading `.t` evaluates the rest)."""
        self._fold_pending()
        rows = self._words()
        pos = 0
        for depth in groups:
            group = self._pending[pos:pos + depth]
            pos += depth
            if _chained(depth):
                rows = difflogic_cuda.eval_chained(rows, group, out_live=live[pos] if live and pos < len(live) else None)
            else:
                rows = difflogic_cuda.eval_fused(rows, group)
        if pos:
            self._rows, self._public = rows, None
        self._pending = self._pending[pos:]
        self._keys = self._keys[pos:]

    @property
    def t(self):
        if self._pending:
            self._run_groups(plan_groups(self._dims(), False, self._words64(), self._live_share()))
        self._state = None            # the caller may write into the words: nothing is known about the rows from here on
        if self._public is None:
            rows = self._words()
            dtype = difflogic_cuda._BITS_TO_DTYPE[self.bit_count]
            row_bytes = -(-self._batch // self.bit_count) * (self.bit_count // 8)
            if row_bytes == rows.shape[1] * 8:
                self._public = rows.view(dtype)
            else:
                self._public = rows.view(torch.uint8)[:, :row_bytes].contiguous().view(dtype)
                self._rows = None     # the copy the caller holds is the state from here on
        return self._public

    @t.setter
    def t(self, value):
        self._pending = []
        self._keys = []
        self._folded = True
        self._state = None
        self._src = None
        self._rows = None
        self._public = value
        bits = difflogic_cuda._WORD_BITS.get(value.dtype, self.bit_count)
        self._batch = max(0, value.shape[1] * bits - self.pad_len)

    def row_state(self, device):
        """What a layer applied next may assume about the rows it reads: uint8 [features] (0 varies, 1 all zeros,
        2 all ones) or None (every row may vary).  See defer_layer."""
        state = self._state
        return state if state is not None and state.device == device else None

    def defer_layer(self, a, b, w, key=None, state=None):
        """Applies the gate layer (a, b, w) lazily.  ``key``: a hashable that changes whenever the gate ids ``w`` may
        have (the weights' address and version counter); lets the planner remember what it measured for them.
        ``state``: the caller folded the constants among the rows it reads (row_state) into ``w`` already and says
        which of the layer's own outputs are constant (difflogic_cuda.gate_ids_folded); without it the folding is
        done before the layers run."""
        self._pending.append((a, b, w))
        self._keys.append(key)
        if state is None:
            self._folded = False
        self._state = state
        return self

    def group_sum(self, k):
        assert self.device == "cuda", self.device
        if self._pending:
            if self.features % k != 0:
                raise ValueError(f"in_dim ({self.features}) has to be divisible by k ({k}) but it is not")
            dims = self._dims()
            share = self._live_share()
            tail = lds_tail(dims, self._words64(), share, from_bool=self._src is not None)
            if tail:
                # the narrow end of the net runs resident in LDS; what lies before it streams
                head = len(self._pending) - tail
                if head == 0 and self._src is not None:
                    # the whole net, straight from the bool input: packing happens on the way into LDS
                    out = difflogic_cuda.eval_net_lds_bool(self._src, self._pending, k, thin=share < _LDS_THIN_BELOW,
                                                           folded=self._folded)
                    if out is not None:
                        return out
                if head:
                    self._run_groups(plan_groups(dims[:head + 1], False, self._words64(), share))
                rows = self._words()
                out = difflogic_cuda.eval_net_lds(rows, self._pending, self._pad(rows), k, thin=share < _LDS_THIN_BELOW,
                                                  folded=self._folded)
                if out is not None:
                    return out
            self._fold_pending()
            groups = plan_groups(self._dims(), True, self._words64(), share)
            # output rows of the groups before the last that no gate above them looks at are not computed
            live = difflogic_cuda.live_inputs(self._pending) if len(groups) > 1 else None
            self._run_groups(groups[:-1], live)
            # the last group stays pending: the object's state does not change by counting
            rows = self._words()
            out = difflogic_cuda.eval_chained_groupbitsum(rows, self._pending, self._pad(rows), k)
            if out is not None:
                return out
            order = difflogic_cuda.count_order_for(self._pending, rows.shape[0], k)
            return difflogic_cuda.eval_fused_groupbitsum(rows, self._pending, self._pad(rows), k, order)
        rows = self._words()
        return difflogic_cuda.groupbitsum(rows, self._pad(rows), k)

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
