"""LogicLayer, GroupSum and the autograd glue (reference: difflogic/difflogic.py), running on
the gfx950 kernels through ``difflogic_cuda``."""
import torch

from . import difflogic_cuda
from .functional import (GradFactor, bin_op_s, build_reverse_index, get_random_connections,
                         get_unique_connections)
from .packbitstensor import PackBitsTensor


class LogicLayer(torch.nn.Module):
    """A layer of ``out_dim`` two-input logic gates, each a learnable mixture of the 16 gates
    over two fixed inputs (difflogic/difflogic.py:11-169).

    :param in_dim:      number of inputs
    :param out_dim:     number of gates
    :param device:      'cuda' (the MI355X; torch-ROCm names it cuda) or 'cpu'
    :param grad_factor: scales the gradient passed to the layer's input (use >1 for deep nets)
    :param implementation: 'cuda' (HIP kernels, default on 'cuda') or 'python' (eager torch,
                        default on 'cpu'); never chosen implicitly for a 'cuda' layer
    :param connections: 'random' or 'unique'
    """

    def __init__(self, in_dim: int, out_dim: int, device: str = "cuda", grad_factor: float = 1.,
                 implementation: str = None, connections: str = "random"):
        super().__init__()
        # drawn before the connections, from the device's generator (difflogic.py:33)
        self.weights = torch.nn.parameter.Parameter(torch.randn(out_dim, 16, device=device))
        self.in_dim = in_dim
        self.out_dim = out_dim
        self.device = device
        self.grad_factor = grad_factor

        if implementation is None:
            implementation = {"cuda": "cuda", "cpu": "python"}.get(device)
        assert implementation in ["cuda", "python"], implementation
        self.implementation = implementation

        assert connections in ["random", "unique"], connections
        self.connections = connections
        self.set_connections(*self.get_connections(connections, device))

        self.num_neurons = out_dim
        self.num_weights = out_dim

    def set_connections(self, a, b):
        """Installs the wiring ``a, b`` ([out_dim] integer tensors with values in [0, in_dim))
        and rebuilds the reverse index the backward pass walks.  The wiring is not part of the
        state_dict (only ``weights`` is), so a model restored from a state_dict needs the
        wiring of the model that was saved: same seed, or this method."""
        a = torch.as_tensor(a).to(torch.int64).to(self.device).contiguous()
        b = torch.as_tensor(b).to(torch.int64).to(self.device).contiguous()
        if a.shape != (self.out_dim,) or b.shape != (self.out_dim,):
            raise ValueError(f"expected two index tensors of shape ({self.out_dim},), got {tuple(a.shape)}, "
                             f"{tuple(b.shape)}")
        if self.out_dim and (min(int(a.min()), int(b.min())) < 0 or max(int(a.max()), int(b.max())) >= self.in_dim):
            raise ValueError(f"connection indices have to lie in [0, {self.in_dim})")
        if getattr(self, "indices", None) is not None:
            difflogic_cuda.invalidate_wiring(*self.indices)     # what was derived from the wiring being replaced
        self.indices = (a, b)
        if self.implementation == "cuda":
            # reverse index for backward_x (difflogic.py:56-69)
            start, idx = build_reverse_index(a, b, self.in_dim)
            self.given_x_indices_of_y_start = start.to(self.device)
            self.given_x_indices_of_y = idx.to(self.device)

    def invalidate_wiring(self):
        """Drops what is derived from the wiring (evaluation schedules, count plans, the reverse index that
        backward_x walks) and rebuilds the reverse index from the current contents of ``indices``.  Call it after
        changing the index tensors in any way other than ``set_connections``.  (The schedule caches notice
        in-place operations that bump the tensors' version counter by themselves; a write through
        ``indices[i].data`` bumps nothing, and the reverse index follows neither.)"""
        difflogic_cuda.invalidate_wiring(*self.indices)
        if self.implementation == "cuda" and hasattr(self, "given_x_indices_of_y"):
            start, idx = build_reverse_index(self.indices[0], self.indices[1], self.in_dim)
            self.given_x_indices_of_y_start = start.to(self.device)
            self.given_x_indices_of_y = idx.to(self.device)

    def forward(self, x):
        if isinstance(x, PackBitsTensor):
            assert not self.training, "PackBitsTensor is not supported for the differentiable training mode."
            assert self.device == "cuda", (
                "PackBitsTensor is only supported for CUDA, not for {}. If you want fast inference on CPU, "
                "please use CompiledDiffLogicModel.".format(self.device))
            assert self.implementation == "cuda", self.implementation
            return self.forward_cuda_eval(x)
        if self.implementation == "cuda":
            return self.forward_cuda(x)
        if self.implementation == "python":
            if self.grad_factor != 1.:
                x = GradFactor.apply(x, self.grad_factor)
            return self.forward_python(x)
        raise ValueError(self.implementation)

    def forward_python(self, x):
        assert x.shape[-1] == self.in_dim, (x.shape[-1], self.in_dim)
        a, b = x[..., self.indices[0]], x[..., self.indices[1]]
        if self.training:
            w = torch.nn.functional.softmax(self.weights, dim=-1)
        else:
            w = torch.nn.functional.one_hot(self.weights.argmax(-1), 16).to(torch.float32)
        return bin_op_s(a, b, w.to(x.dtype))

    def forward_cuda(self, x):
        if self.training:
            assert x.device.type == "cuda", x.device
        assert x.ndim == 2, x.ndim
        x = x.transpose(0, 1).contiguous()                  # feature-major [in, B]
        assert x.shape[0] == self.in_dim, (x.shape, self.in_dim)
        a, b = self.indices
        tail = (self.given_x_indices_of_y_start, self.given_x_indices_of_y, float(self.grad_factor))
        if self.training:
            same = self.weights.dtype == x.dtype
            mixed = self.weights.dtype == torch.float32 and x.dtype in (torch.float16, torch.float64)
            if (same or mixed) and x.shape[1] > 0:
                # softmax and its backward run inside the layer kernels; fp32 weights next to half / double
                # activations (the reference's --training-bit-count 16 / 64) are read as they are
                return LogicLayerLogitsFunction.apply(x, a, b, self.weights, *tail,
                                                      self._train_schedule()).transpose(0, 1)
            w = torch.nn.functional.softmax(self.weights, dim=-1).to(x.dtype)
            return LogicLayerCudaFunction.apply(x, a, b, w, *tail, self._train_schedule()).transpose(0, 1)
        # eval mode: the discretised net on float inputs (no gradients)
        w = torch.nn.functional.one_hot(self.weights.argmax(-1), 16).to(x.dtype)
        with torch.no_grad():
            return difflogic_cuda.forward(x, a, b, w, self._train_schedule()).transpose(0, 1)

    def forward_cuda_eval(self, x: PackBitsTensor):
        """Packed inference.  Updates ``x`` in place (as the reference rebinds ``x.t``) and
        returns it.  The evaluation is deferred until ``x.t`` is read or GroupSum consumes it;
        deferred layers run in fused groups (PackBitsTensor.plan_groups)."""
        assert not self.training
        assert isinstance(x, PackBitsTensor)
        assert x.features == self.in_dim, (x.features, self.in_dim)
        a, b = self.indices
        key = (self.weights.data_ptr(), self.weights._version, self.out_dim)
        w = self.weights.detach()
        if w.is_cuda and w.is_contiguous() and w.dtype in (torch.float16, torch.float32, torch.float64):
            # the argmax gates with the constants among x's rows folded in, in one kernel (x tracks which rows those are)
            ids, state = difflogic_cuda.gate_ids_folded(w, a, b, x.row_state(a.device))
            return x.defer_layer(a, b, ids, key=key, state=state)
        return x.defer_layer(a, b, self._gate_ids(), key=key)

    # Below this many inputs a 1 KB column tile of the whole input stays in the L2 caches and the
    # second gather of a row hits there; above it the chained kernels halve the gathered rows.
    _CHAIN_MIN_IN_DIM = 4096
    # Narrower layers are latency-bound; a wave walking 8 neurons in sequence only lengthens that.
    _CHAIN_MIN_OUT_DIM = 32768

    def _train_schedule(self):
        """Evaluation schedule of this layer's wiring for the chained forward / backward_w
        kernels (cached per wiring), or None where chaining does not pay."""
        if self.in_dim < self._CHAIN_MIN_IN_DIM or self.out_dim < self._CHAIN_MIN_OUT_DIM:
            return None
        return difflogic_cuda.schedule_for(self.indices[0], self.indices[1], self.in_dim)

    def _gate_ids(self):
        """uint8 [out_dim] argmax gate per neuron.  Recomputed on every call like the reference
        (difflogic/difflogic.py:146): a cache could not see writes through ``weights.data``."""
        w = self.weights.detach()
        if w.is_cuda and w.is_contiguous() and w.dtype in (torch.float16, torch.float32, torch.float64):
            return difflogic_cuda.gate_ids(w)
        return w.argmax(-1).to(torch.uint8)

    def extra_repr(self):
        return "{}, {}, {}".format(self.in_dim, self.out_dim, "train" if self.training else "eval")

    def get_connections(self, connections, device="cuda"):
        assert self.out_dim * 2 >= self.in_dim, (
            "The number of neurons ({}) must not be smaller than half of the number of inputs ({}) because "
            "otherwise not all inputs could be used or considered.".format(self.out_dim, self.in_dim))
        if connections == "random":
            return get_random_connections(self.in_dim, self.out_dim, device)
        if connections == "unique":
            return get_unique_connections(self.in_dim, self.out_dim, device)
        raise ValueError(connections)


class GroupSum(torch.nn.Module):
    """Sums contiguous groups of out/k neurons into k scores and divides by tau
    (difflogic/difflogic.py:175-199).  On a PackBitsTensor: undivided int32 bit counts."""

    def __init__(self, k: int, tau: float = 1., device="cuda"):
        super().__init__()
        self.k = k
        self.tau = tau
        self.device = device

    # grid limits of dl_group_sum_forward / dl_group_sum_backward (one grid row per class, one per 64
    # neurons); beyond them the torch formulation below runs, in forward and backward alike
    _HIP_MAX_K = 65535
    _HIP_MAX_OUT_DIM = 65535 * 64

    def forward(self, x):
        if isinstance(x, PackBitsTensor):
            return x.group_sum(self.k)
        assert x.shape[-1] % self.k == 0, (x.shape, self.k)
        if (x.is_cuda and x.dim() == 2 and x.dtype in (torch.float16, torch.float32, torch.float64)
                and x.numel() > 0 and x.stride(0) == 1 and x.stride(1) == x.shape[0]
                and self.k <= self._HIP_MAX_K and x.shape[1] <= self._HIP_MAX_OUT_DIM):
            # the transposed view a 'cuda' LogicLayer returns: sum on the feature-major storage
            return GroupSumCudaFunction.apply(x.transpose(0, 1), self.k, float(self.tau))
        return x.reshape(*x.shape[:-1], self.k, x.shape[-1] // self.k).sum(-1) / self.tau

    def extra_repr(self):
        return "k={}, tau={}".format(self.k, self.tau)


class LogicLayerCudaFunction(torch.autograd.Function):
    """Feature-major forward/backward of one layer (difflogic/difflogic.py:205-221).  The
    optional trailing ``grad_factor`` is folded into backward_x instead of a separate
    elementwise pass over the input gradient; ``schedule`` (the layer's evaluation schedule) selects
    the kernels that walk the wiring along its trails."""

    @staticmethod
    def forward(ctx, x, a, b, w, given_x_indices_of_y_start, given_x_indices_of_y, grad_factor=1.0, schedule=None):
        ctx.save_for_backward(x, a, b, w, given_x_indices_of_y_start, given_x_indices_of_y)
        ctx.grad_factor = grad_factor
        ctx.schedule = schedule
        return difflogic_cuda.forward(x, a, b, w, schedule)

    @staticmethod
    def backward(ctx, grad_y):
        x, a, b, w, given_x_indices_of_y_start, given_x_indices_of_y = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        grad_w = grad_x = None
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[3] and ctx.schedule is not None:
            # one pass along the schedule yields both gradients
            both = difflogic_cuda.backward_chained(x, w, grad_y, ctx.schedule, ctx.grad_factor)
            if both is not None:
                return both[1], None, None, both[0], None, None, None, None
        if ctx.needs_input_grad[0]:
            grad_x = difflogic_cuda.backward_x(x, a, b, w, grad_y, given_x_indices_of_y_start,
                                               given_x_indices_of_y, ctx.grad_factor)
        if ctx.needs_input_grad[3]:
            grad_w = difflogic_cuda.backward_w(x, a, b, grad_y, ctx.schedule)
        return grad_x, None, None, grad_w, None, None, None, None


class LogicLayerLogitsFunction(torch.autograd.Function):
    """LogicLayerCudaFunction on the raw gate logits: ``forward(x, a, b, softmax(logits))`` and
    its gradients, with the softmax and the softmax backward inside the layer kernels."""

    @staticmethod
    def forward(ctx, x, a, b, logits, given_x_indices_of_y_start, given_x_indices_of_y, grad_factor=1.0,
                schedule=None):
        y, probs = difflogic_cuda.forward_logits(x, a, b, logits.detach().contiguous(), schedule)
        ctx.save_for_backward(x, a, b, probs, given_x_indices_of_y_start, given_x_indices_of_y)
        ctx.grad_factor = grad_factor
        ctx.schedule = schedule
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, a, b, probs, given_x_indices_of_y_start, given_x_indices_of_y = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        grad_logits = grad_x = None
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[3] and ctx.schedule is not None:
            # one pass along the schedule yields both gradients
            both = difflogic_cuda.backward_chained(x, probs, grad_y, ctx.schedule, ctx.grad_factor,
                                                   softmax_backward=True)
            if both is not None:
                return both[1], None, None, both[0], None, None, None, None
        if ctx.needs_input_grad[0]:
            grad_x = difflogic_cuda.backward_x(x, a, b, probs, grad_y, given_x_indices_of_y_start,
                                               given_x_indices_of_y, ctx.grad_factor)
        if ctx.needs_input_grad[3]:
            grad_logits = difflogic_cuda.backward_logits(x, a, b, grad_y, probs, ctx.schedule)
        return grad_x, None, None, grad_logits, None, None, None, None


class GroupSumCudaFunction(torch.autograd.Function):
    """GroupSum on a feature-major [out, B] activation: -> [B, k].  The gradient comes back
    feature-major too, so the layer below needs no transposing copy of it."""

    @staticmethod
    def forward(ctx, x, k, tau):
        ctx.out_dim, ctx.tau = x.shape[0], tau
        return difflogic_cuda.group_sum_forward(x, k, tau)

    @staticmethod
    def backward(ctx, grad_y):
        return difflogic_cuda.group_sum_backward(grad_y.contiguous(), ctx.out_dim, ctx.tau), None, None


class LogicLayerGroupSumFunction(torch.autograd.Function):
    """The last LogicLayer and the GroupSum after it as one autograd node: feature-major input
    [in, B] and gate logits -> class scores [B, k].  Neither the layer's [out, B] output nor the
    broadcast gradient GroupSum's backward would return is ever materialised."""

    @staticmethod
    def forward(ctx, x, a, b, logits, given_x_indices_of_y_start, given_x_indices_of_y, grad_factor, schedule, k, tau):
        y, probs = difflogic_cuda.forward_group_sum(x, a, b, logits.detach().contiguous(), k, tau)
        ctx.save_for_backward(x, a, b, probs, given_x_indices_of_y_start, given_x_indices_of_y)
        ctx.grad_factor, ctx.schedule, ctx.tau = grad_factor, schedule, tau
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, a, b, probs, start, idx = ctx.saved_tensors
        grad_cls = (grad_y / ctx.tau).t().contiguous()                 # [k, B]: a few KB
        grad_logits, grad_x = difflogic_cuda.backward_group_sum(
            x, a, b, probs, grad_cls, start, idx, ctx.schedule, ctx.grad_factor,
            want_x=ctx.needs_input_grad[0], want_w=ctx.needs_input_grad[3])
        return grad_x, None, None, grad_logits, None, None, None, None, None, None


class FusedLogicLayerGroupSum(torch.nn.Module):
    """``GroupSum(LogicLayer(x))`` as one module (see fuse_group_sum).  Holds the two original
    modules; the LogicLayer's ``weights`` stay registered under their own name, so the
    state_dict of a fused ``nn.Sequential`` has the keys of the unfused one.  Takes the fused kernels
    in training mode on float inputs; everything else (eval mode, PackBitsTensor, dtypes that
    differ from the weights') runs the two modules one after the other."""

    def __init__(self, layer: LogicLayer, group_sum: GroupSum):
        super().__init__()
        assert isinstance(layer, LogicLayer) and isinstance(group_sum, GroupSum)
        self.weights = layer.weights                                    # same Parameter, same key as before
        object.__setattr__(self, "layer", layer)                        # not registered: no second state_dict entry
        object.__setattr__(self, "group_sum", group_sum)

    def train(self, mode=True):
        self.layer.train(mode)
        self.group_sum.train(mode)
        return super().train(mode)

    def _apply(self, fn, recurse=True):
        self.layer._apply(fn)
        self.group_sum._apply(fn)
        super()._apply(fn, recurse)
        self.weights = self.layer.weights
        return self

    def forward(self, x):
        layer, gs = self.layer, self.group_sum
        if (isinstance(x, PackBitsTensor) or not self.training or layer.implementation != "cuda" or not x.is_cuda
                or x.ndim != 2 or x.dtype != layer.weights.dtype or x.shape[0] == 0 or layer.out_dim % gs.k != 0
                or gs.k > GroupSum._HIP_MAX_K or layer.out_dim > GroupSum._HIP_MAX_OUT_DIM):
            return gs(layer(x))                                         # (the limits GroupSum itself falls back beyond)
        xt = x.transpose(0, 1).contiguous()
        assert xt.shape[0] == layer.in_dim, (xt.shape, layer.in_dim)
        a, b = layer.indices
        return LogicLayerGroupSumFunction.apply(xt, a, b, layer.weights, layer.given_x_indices_of_y_start,
                                                layer.given_x_indices_of_y, float(layer.grad_factor),
                                                layer._train_schedule(), int(gs.k), float(gs.tau))

    def extra_repr(self):
        return "{}, {}".format(self.layer.extra_repr(), self.group_sum.extra_repr())


class LogicLayerPairFunction(torch.autograd.Function):
    """A model's first two LogicLayers as one autograd node: feature-major input [in, B] that
    needs no gradient and both layers' gate logits -> the second layer's output [out2, B].  In the
    backward pass the first layer's grad_y (= the second layer's grad_x) is consumed row by row
    where the second layer's one-pass backward finishes it and never touches memory.  When the
    input is small enough to stay in the L2 caches (and the dtype is fp32 / fp64) the first layer's
    output does not exist in memory either: forward and backward recompute its rows from the
    input."""

    # the input [in, B] stays cache-resident below this size: recomputing a row of the first layer's
    # output (two gathered input rows) is then cheaper than storing and re-reading it
    RECOMPUTE_MAX_INPUT_BYTES = 4 << 20

    @staticmethod
    def forward(ctx, x, a1, b1, logits1, schedule1, a2, b2, logits2, start2, idx2, grad_factor2, schedule2):
        l1, l2 = logits1.detach().contiguous(), logits2.detach().contiguous()
        fused = None
        if (x.dtype in (torch.float32, torch.float64)
                and x.numel() * x.element_size() <= LogicLayerPairFunction.RECOMPUTE_MAX_INPUT_BYTES):
            fused = difflogic_cuda.forward_logits_lower(x, a1, b1, l1, l2, schedule2)
        if fused is not None:
            y2, probs1, probs2 = fused
            y1 = None
            ctx.save_for_backward(x, a1, b1, probs1, a2, b2, probs2, start2, idx2)
        else:
            y1, probs1 = difflogic_cuda.forward_logits(x, a1, b1, l1, schedule1)
            y2, probs2 = difflogic_cuda.forward_logits(y1, a2, b2, l2, schedule2)
            ctx.save_for_backward(x, a1, b1, probs1, a2, b2, probs2, start2, idx2, y1)
        ctx.recompute = y1 is None
        ctx.grad_factor2, ctx.schedule1, ctx.schedule2 = grad_factor2, schedule1, schedule2
        return y2

    @staticmethod
    def backward(ctx, grad_y):
        x, a1, b1, probs1, a2, b2, probs2, start2, idx2 = ctx.saved_tensors[:9]
        y1 = None if ctx.recompute else ctx.saved_tensors[9]
        grad_y = grad_y.contiguous()
        want1, want2 = ctx.needs_input_grad[3], ctx.needs_input_grad[7]
        g1 = g2 = None
        if want1 and want2:
            both = difflogic_cuda.backward_chained_lower(y1, probs2, grad_y, ctx.schedule2, x, a1, b1, probs1,
                                                         ctx.grad_factor2, softmax_backward=True)
            if both is not None:
                g2, g1 = both
                return None, None, None, g1, None, None, None, g2, None, None, None, None
        # the separate kernels, as two LogicLayers in a row would run them
        if y1 is None:
            y1 = difflogic_cuda.forward(x, a1, b1, probs1, ctx.schedule1)
        if want1:
            both = difflogic_cuda.backward_chained(y1, probs2, grad_y, ctx.schedule2, ctx.grad_factor2,
                                                   softmax_backward=True) if want2 else None
            if both is not None:
                g2, grad_y1 = both
            else:
                grad_y1 = difflogic_cuda.backward_x(y1, a2, b2, probs2, grad_y, start2, idx2, ctx.grad_factor2)
            g1 = difflogic_cuda.backward_logits(x, a1, b1, grad_y1, probs1, ctx.schedule1)
        if want2 and g2 is None:
            g2 = difflogic_cuda.backward_logits(y1, a2, b2, grad_y, probs2, ctx.schedule2)
        return None, None, None, g1, None, None, None, g2, None, None, None, None


class FusedLogicLayerPair(torch.nn.Module):
    """``layer2(layer1(x))`` for a model's first two LogicLayers as one module (see
    fuse_first_layers).  Registered under the first layer's position with the first layer's
    ``weights``; the second layer's ``weights`` stay registered at its own position (_LayerDone),
    so the state_dict keys are those of the unfused model.  Takes the fused path in training mode
    on float inputs that need no gradient when the second layer is wide enough to be walked along
    its schedule; everything else runs the two layers one after the other."""

    def __init__(self, layer1: LogicLayer, layer2: LogicLayer):
        super().__init__()
        assert isinstance(layer1, LogicLayer) and isinstance(layer2, LogicLayer)
        assert layer1.out_dim == layer2.in_dim, (layer1.out_dim, layer2.in_dim)
        self.weights = layer1.weights
        object.__setattr__(self, "layer1", layer1)
        object.__setattr__(self, "layer2", layer2)                      # trained / moved through _LayerDone

    def train(self, mode=True):
        self.layer1.train(mode)
        return super().train(mode)

    def _apply(self, fn, recurse=True):
        self.layer1._apply(fn)
        super()._apply(fn, recurse)
        self.weights = self.layer1.weights
        return self

    def forward(self, x):
        l1, l2 = self.layer1, self.layer2
        if (isinstance(x, PackBitsTensor) or not self.training or not l2.training or l1.implementation != "cuda"
                or l2.implementation != "cuda" or not x.is_cuda or x.ndim != 2 or x.requires_grad
                or x.dtype != l1.weights.dtype or x.dtype != l2.weights.dtype or x.shape[0] == 0
                or l2._train_schedule() is None):
            return l2(l1(x))
        xt = x.transpose(0, 1).contiguous()
        assert xt.shape[0] == l1.in_dim, (xt.shape, l1.in_dim)
        return LogicLayerPairFunction.apply(xt, l1.indices[0], l1.indices[1], l1.weights, l1._train_schedule(),
                                            l2.indices[0], l2.indices[1], l2.weights, l2.given_x_indices_of_y_start,
                                            l2.given_x_indices_of_y, float(l2.grad_factor),
                                            l2._train_schedule()).transpose(0, 1)

    def extra_repr(self):
        return "({}) -> ({})".format(self.layer1.extra_repr(), self.layer2.extra_repr())


class _LayerDone(torch.nn.Module):
    """Stands where the second layer stood after fuse_first_layers: the module before it already
    evaluated that layer.  Keeps the layer's ``weights`` registered at this position."""

    def __init__(self, layer: LogicLayer):
        super().__init__()
        self.weights = layer.weights
        object.__setattr__(self, "layer", layer)

    def train(self, mode=True):
        self.layer.train(mode)
        return super().train(mode)

    def _apply(self, fn, recurse=True):
        self.layer._apply(fn)
        super()._apply(fn, recurse)
        self.weights = self.layer.weights
        return self

    def forward(self, x):
        return x


class _GroupSumDone(torch.nn.Module):
    """Stands where the GroupSum stood after fuse_group_sum: the module before it already summed."""

    def forward(self, x):
        return x


def fuse_group_sum(model: torch.nn.Sequential) -> torch.nn.Sequential:
    """Returns a ``nn.Sequential`` in which every ``LogicLayer`` directly followed by a ``GroupSum``
    (normally the model's last two modules) is replaced by one fused module, which in training
    saves writing and re-reading the layer's output and GroupSum's broadcast gradient.  Module
    positions, parameters and state_dict keys are unchanged; the input model is not modified and
    shares its parameters with the result."""
    mods = list(model)
    for i in range(len(mods) - 1):
        if isinstance(mods[i], LogicLayer) and isinstance(mods[i + 1], GroupSum) and mods[i].implementation == "cuda":
            mods[i], mods[i + 1] = FusedLogicLayerGroupSum(mods[i], mods[i + 1]), _GroupSumDone()
    return torch.nn.Sequential(*mods)


def fuse_first_layers(model: torch.nn.Sequential) -> torch.nn.Sequential:
    """Returns a ``nn.Sequential`` in which the first two ``LogicLayer`` modules, when they follow
    each other directly, are replaced by one fused module: in training the first layer's weight
    gradient is then formed inside the second layer's backward pass, and the gradient between the
    two layers (``[width, batch]``) is neither written nor read back.  Module positions, parameters
    and state_dict keys are unchanged; the input model is not modified and shares its parameters
    with the result."""
    mods = list(model)
    first = next((i for i, m in enumerate(mods) if isinstance(m, LogicLayer)), None)
    if (first is not None and first + 1 < len(mods) and isinstance(mods[first + 1], LogicLayer)
            and mods[first].implementation == "cuda" and mods[first + 1].implementation == "cuda"):
        l1, l2 = mods[first], mods[first + 1]
        mods[first], mods[first + 1] = FusedLogicLayerPair(l1, l2), _LayerDone(l2)
    return torch.nn.Sequential(*mods)


class _Node:
    """Stands in for an autograd context where a Function's ``forward`` / ``backward`` are called directly."""

    def __init__(self, needs_input_grad):
        self.needs_input_grad = needs_input_grad
        self.saved_tensors = ()

    def save_for_backward(self, *tensors):
        self.saved_tensors = tensors


class LogicNetFunction(torch.autograd.Function):
    """A run of logic layers (and the GroupSum at its end) as ONE autograd node: the stages' own Functions
    (LogicLayerPairFunction, LogicLayerLogitsFunction, LogicLayerGroupSumFunction) are called one after the other on
    feature-major activations, forwards and then backwards, with stand-in contexts.  Same kernels, same values; what
    goes is the host work per layer (module call, two transposes, an autograd node each way), which is what a
    training step costs at the reference's batch sizes (784 -> 4 x 8000 at batch 128: 0.44 -> 0.3 ms per step).

    ``stages``: list of (Function, args, weight positions); ``args[0]`` is replaced by the running activation and
    the weights at ``weight positions`` are the Function's inputs ``weights`` in order."""

    @staticmethod
    def forward(ctx, x, stages, *weights):
        nodes, cur, needs_x = [], x, ctx.needs_input_grad[0]
        for fn, args, weight_pos in stages:
            needs = [False] * len(args)
            needs[0] = needs_x
            for pos in weight_pos:
                needs[pos] = args[pos].requires_grad
            node = _Node(needs)
            cur = fn.forward(node, cur, *args[1:])
            nodes.append((fn, node, weight_pos))
            needs_x = needs_x or any(needs[pos] for pos in weight_pos)
        # what the stages saved goes through the node's own save_for_backward, so that autograd frees it after the
        # backward pass (and notices writes into it) as it does for the stages run as nodes of their own
        ctx.save_for_backward(*[t for _, node, _ in nodes for t in node.saved_tensors])
        ctx.saved_counts = [len(node.saved_tensors) for _, node, _ in nodes]
        for _, node, _ in nodes:
            node.saved_tensors = ()
        ctx.nodes = nodes
        return cur

    @staticmethod
    def backward(ctx, grad):
        saved, at = ctx.saved_tensors, 0
        for (_, node, _), count in zip(ctx.nodes, ctx.saved_counts):
            node.saved_tensors = saved[at:at + count]
            at += count
        grads = []
        for fn, node, weight_pos in reversed(ctx.nodes):
            if grad is None:                                 # nothing below wants a gradient
                grads.extend([None] * len(weight_pos))
                continue
            out = fn.backward(node, grad)
            grads.extend(out[pos] for pos in reversed(weight_pos))
            grad = out[0]
        for _, node, _ in ctx.nodes:
            node.saved_tensors = ()
        return (grad, None) + tuple(reversed(grads))


class FusedSequential(torch.nn.Sequential):
    """The ``nn.Sequential`` fuse_for_training returns: the modules of the fused model, run as ONE autograd node
    (LogicNetFunction) from the first logic layer to the end where every one of them would take its HIP training
    path (training mode, a 2-D float CUDA input of a dtype the layers take, a GroupSum the kernels cover), and one
    after the other otherwise (eval mode, PackBitsTensor, the python implementation, other modules in between).
    Positions, parameters and state_dict keys are those of the model it was made from."""

    def _stages(self, mods, x):
        """The stages of LogicNetFunction for ``mods`` on feature-major input of x's kind, or None."""
        stages, i, first = [], 0, True
        dtype = x.dtype
        while i < len(mods):
            m = mods[i]
            if isinstance(m, FusedLogicLayerPair) and i + 1 < len(mods) and isinstance(mods[i + 1], _LayerDone):
                l1, l2 = m.layer1, m.layer2
                pair_ok = (first and not x.requires_grad and l2._train_schedule() is not None
                           and dtype == l1.weights.dtype and dtype == l2.weights.dtype)
                for layer in (l1, l2):
                    if not layer.training or layer.implementation != "cuda":
                        return None
                if pair_ok:
                    stages.append((LogicLayerPairFunction,
                                   (None, l1.indices[0], l1.indices[1], l1.weights, l1._train_schedule(), l2.indices[0],
                                    l2.indices[1], l2.weights, l2.given_x_indices_of_y_start, l2.given_x_indices_of_y,
                                    float(l2.grad_factor), l2._train_schedule()), (3, 7)))
                else:
                    for layer in (l1, l2):
                        st = self._layer_stage(layer, dtype)
                        if st is None:
                            return None
                        stages.append(st)
                i += 2
            elif isinstance(m, LogicLayer):
                st = self._layer_stage(m, dtype) if m.training and m.implementation == "cuda" else None
                if st is None:
                    return None
                stages.append(st)
                i += 1
            elif (isinstance(m, FusedLogicLayerGroupSum) and i + 2 == len(mods) and isinstance(mods[i + 1], _GroupSumDone)):
                layer, gs = m.layer, m.group_sum
                if (not m.training or layer.implementation != "cuda" or layer.out_dim % gs.k != 0
                        or gs.k > GroupSum._HIP_MAX_K or layer.out_dim > GroupSum._HIP_MAX_OUT_DIM):
                    return None
                if dtype == layer.weights.dtype:
                    stages.append((LogicLayerGroupSumFunction,
                                   (None, layer.indices[0], layer.indices[1], layer.weights, layer.given_x_indices_of_y_start,
                                    layer.given_x_indices_of_y, float(layer.grad_factor), layer._train_schedule(), int(gs.k),
                                    float(gs.tau)), (3,)))
                else:
                    # half / double activations over fp32 weights: the layer takes them, the fused kernels of layer +
                    # GroupSum do not; the two run as stages of their own on the feature-major activation
                    st = self._layer_stage(layer, dtype)
                    if st is None:
                        return None
                    stages += [st, (GroupSumCudaFunction, (None, int(gs.k), float(gs.tau)), ())]
                i += 2
            else:
                return None
            first = False
        # (a run that does not end in the fused GroupSum would hand a feature-major activation on: not taken)
        return stages if stages and stages[-1][0] in (LogicLayerGroupSumFunction, GroupSumCudaFunction) else None

    @staticmethod
    def _layer_stage(layer, dtype):
        w = layer.weights.dtype
        if not (w == dtype or (w == torch.float32 and dtype in (torch.float16, torch.float64))):
            return None
        return (LogicLayerLogitsFunction,
                (None, layer.indices[0], layer.indices[1], layer.weights, layer.given_x_indices_of_y_start,
                 layer.given_x_indices_of_y, float(layer.grad_factor), layer._train_schedule()), (3,))

    def forward(self, x):
        mods = list(self)
        start = next((i for i, m in enumerate(mods) if isinstance(m, (LogicLayer, FusedLogicLayerPair,
                                                                     FusedLogicLayerGroupSum))), None)
        if start is None or not self.training:
            return super().forward(x)
        for m in mods[:start]:
            x = m(x)
        stages = None
        if (torch.is_tensor(x) and x.is_cuda and x.ndim == 2 and x.shape[0] > 0 and x.is_floating_point()
                and x.shape[1] == getattr(mods[start], "layer1", getattr(mods[start], "layer", mods[start])).in_dim):
            stages = self._stages(mods[start:], x)
        if stages is None:
            for m in mods[start:]:
                x = m(x)
            return x
        weights = [args[pos] for _, args, weight_pos in stages for pos in weight_pos]
        return LogicNetFunction.apply(x.transpose(0, 1).contiguous(), stages, *weights)


def fuse_for_training(model: torch.nn.Sequential) -> torch.nn.Sequential:
    """fuse_first_layers and fuse_group_sum together (the last layer is left to fuse_group_sum
    when a model has only two layers), in a Sequential that runs the logic layers as one autograd node where it can
    (FusedSequential: less host work per step, which is what small nets at small batches are bound by)."""
    fused = fuse_group_sum(model)
    return FusedSequential(*fuse_first_layers(fused))
