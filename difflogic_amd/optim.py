"""Adam for a model's weight tensors in one kernel launch.

The reference trains with ``torch.optim.Adam(model.parameters(), lr=...)``
(experiments/main.py:169,179).  ``FusedAdam`` computes the same update (amsgrad and maximize
off) for every fp32 parameter of a group with a single launch of the library's ``dl_adam_step``
and keeps its step count on the device, so the step can be captured into a HIP graph together
with forward and backward (``difflogic_amd.graphs.GraphedTrainStep``).  For the small tensors of
a LogicLayer net ([out, 16] logits per layer) this is several times faster than torch's
multi-tensor kernel, whose blocks each walk 65536 elements.
"""
import ctypes

import torch

from . import _lib


class FusedAdam(torch.optim.Optimizer):
    """Drop-in for ``torch.optim.Adam`` on contiguous fp32 GPU parameters.

    State per parameter: ``exp_avg``, ``exp_avg_sq`` (as torch's Adam) and ``step``, a device
    scalar shared by the parameters that are updated by one launch (a view of ``_counter``, the
    four floats the library keeps per launch).

    Differences from ``torch.optim.Adam`` that a caller can meet:

    * Parameters that share a step counter step together.  A parameter without a gradient is
      skipped as in torch, but only if ALL parameters of its counter have none on that step;
      a step on which some members of a counter have gradients and others do not raises
      ``RuntimeError`` (the shared count would otherwise run ahead of the skipped parameter's own,
      and its bias correction would differ from torch's from then on).
    * ``load_state_dict`` of a state saved by ``torch.optim.Adam`` (``step`` per parameter, no
      ``_counter``) is accepted: the counters are rebuilt from ``step``; parameters whose step
      counts differ get counters of their own.
    * ``lr``, ``betas``, ``eps`` and ``weight_decay`` are kernel arguments read from the param
      group at every ``step()``.  A step captured into a HIP graph (``GraphedTrainStep``) replays
      the values it was captured with: a learning-rate scheduler has no effect on replays; capture
      again after changing them.
    """

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps < 0.0:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 0: {betas[0]}")
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 1: {betas[1]}")
        if weight_decay < 0.0:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._tables = {}

    def load_state_dict(self, state_dict):
        """Accepts a state saved by this class or by ``torch.optim.Adam``.  The shared step counters are not
        restored as saved (a loaded copy would no longer be shared): they are rebuilt from every parameter's
        ``step`` on the next ``step()``."""
        super().load_state_dict(state_dict)
        for st in self.state.values():
            st.pop("_counter", None)
        self._tables = {}

    def _table(self, gi, device, ps):
        """ctypes pointer tables for one launch, rebuilt only when a tensor moved."""
        key = tuple((p.data_ptr(), p.grad.data_ptr()) for p in ps)
        hit = self._tables.get((gi, device))
        if hit is not None and hit[0] == key:
            return hit[1]
        n = len(ps)
        arr = lambda vals: (ctypes.c_void_p * n)(*vals)
        tab = (arr([p.data_ptr() for p in ps]), arr([p.grad.data_ptr() for p in ps]),
               arr([self.state[p]["exp_avg"].data_ptr() for p in ps]),
               arr([self.state[p]["exp_avg_sq"].data_ptr() for p in ps]),
               (ctypes.c_int64 * n)(*[p.numel() for p in ps]))
        self._tables[(gi, device)] = (key, tab)
        return tab

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _lib.load()
        most = lib.dl_adam_max_tensors()
        for gi, group in enumerate(self.param_groups):
            by_device = {}
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse or not p.is_cuda or p.dtype != torch.float32 or p.grad.dtype != torch.float32:
                    raise RuntimeError("FusedAdam takes dense fp32 parameters and gradients on a GPU; got "
                                       f"{p.dtype} on {p.device}")
                if not p.is_contiguous() or not p.grad.is_contiguous():
                    raise RuntimeError("FusedAdam needs contiguous parameters and gradients")
                by_device.setdefault(p.device, []).append(p)
            for device, ps in by_device.items():
                fresh, restored = [], {}
                for p in ps:
                    st = self.state[p]
                    if "exp_avg" not in st:
                        st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                        st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    if "step" not in st:
                        fresh.append(p)
                    elif "_counter" not in st:
                        # a state loaded from torch.optim.Adam (or from a state_dict that dropped the counter):
                        # parameters with the same step count share a rebuilt counter
                        restored.setdefault(float(st["step"]), []).append(p)
                # one step counter per launch: the kernel advances it, so tensors that share one go together
                for done, members in [(0.0, fresh)] + sorted(restored.items()):
                    for lo in range(0, len(members), most):
                        # [updates done, two factors the library derives from it per update, unused]
                        counter = torch.zeros(4, dtype=torch.float32, device=device)
                        counter[0] = done
                        for p in members[lo:lo + most]:
                            self.state[p]["step"] = counter[0]
                            self.state[p]["_counter"] = counter
                runs = {}
                for p in ps:
                    runs.setdefault(self.state[p]["_counter"].data_ptr(), []).append(p)
                # a counter steps for all of its members or for none of them
                for p in group["params"]:
                    st = self.state.get(p)
                    if p.grad is None and st and "_counter" in st and st["_counter"].data_ptr() in runs:
                        raise RuntimeError("FusedAdam: a parameter without a gradient shares its step counter with "
                                           "parameters that have one; give parameters that are not always trained "
                                           "together a param group (or optimizer) of their own")
                stream = torch.cuda.current_stream(device).cuda_stream
                with torch.cuda.device(device):
                    for si, members in enumerate(runs.values()):
                        if len(members) > most:
                            raise RuntimeError(f"FusedAdam: {len(members)} tensors share one step counter, at most {most} can")
                        tp, tg, tm, tv, tn = self._table((gi, si), device, members)
                        rc = lib.dl_adam_step(len(members), tp, tg, tm, tv, tn,
                                              ctypes.c_void_p(self.state[members[0]]["_counter"].data_ptr()),
                                              float(group["lr"]), float(group["betas"][0]), float(group["betas"][1]),
                                              float(group["eps"]), float(group["weight_decay"]), ctypes.c_void_p(stream))
                        if rc:
                            raise RuntimeError(f"dl_adam_step: {_lib.status_string(rc)}")
        return loss
