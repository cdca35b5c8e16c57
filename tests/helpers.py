"""Shared builders for the parity tests."""
import numpy as np
import torch


def random_layers(rng, F, widths, ops=None):
    """List of (a, b, op) numpy tables of a random discretised net."""
    layers, d = [], F
    for o in widths:
        op = rng.integers(0, 16, o).astype(np.uint8) if ops is None else np.full(o, ops, np.uint8)
        layers.append((rng.integers(0, d, o).astype(np.int64), rng.integers(0, d, o).astype(np.int64), op))
        d = o
    return layers


def build_model(F, layers, k, tau=1.0, device="cuda", grad_factor=1.0, logits=None):
    """Flatten -> LogicLayer x L -> GroupSum with the given wiring.  With ``logits`` None every
    neuron's logits are one-hot on its gate id (argmax == op); else ``logits[i]`` [out,16]."""
    import difflogic_amd as dl
    mods = [torch.nn.Flatten()]
    d = F
    for i, (a, b, op) in enumerate(layers):
        layer = dl.LogicLayer(d, len(a), device=device, grad_factor=grad_factor,
                              implementation="cuda" if device == "cuda" else "python")
        layer.set_connections(torch.as_tensor(a), torch.as_tensor(b))
        with torch.no_grad():
            if logits is None:
                layer.weights.copy_(torch.nn.functional.one_hot(torch.as_tensor(op).long(), 16).float())
            else:
                layer.weights.copy_(torch.as_tensor(logits[i]))
        mods.append(layer)
        d = len(a)
    mods.append(dl.GroupSum(k, tau, device=device))
    return torch.nn.Sequential(*mods)


RTOL = 1e-5      # the fp32 tolerance of the training path (relative error against the python implementation)


def within_budget(got, want64, ref32=None, rtol=RTOL):
    """The fp32 parity bar of the training path, with its error budget made explicit.

    ``want64`` is the python implementation evaluated in fp64 (the exact answer for this purpose),
    ``ref32`` the same python implementation evaluated in fp32, as the reference runs it.  An
    element passes if  |got - want64| <= rtol * max|want64| + rtol * |want64|  (1e-5 relative, with
    the tensor's scale as the floor for entries that cancel to ~0), or if it is no further from the
    fp64 value than the fp32 python implementation itself gets on this case
    (max |ref32 - want64|): fp32 batch sums carry ~sqrt(B) * 6e-8 of rounding whatever the
    summation order, so where the reference's own arithmetic cannot meet 1e-5 the kernel is only
    asked to be as good.  Returns (ok, report) with both errors relative to the tensor's scale."""
    got, want64 = got.detach().double().cpu(), want64.detach().double().cpu()
    if want64.numel() == 0:
        return True, {}
    scale = want64.abs().max().item()
    err = (got - want64).abs()
    ref_err = 0.0 if ref32 is None else (ref32.detach().double().cpu() - want64).abs().max().item()
    ok = bool((err <= torch.clamp(rtol * scale + rtol * want64.abs(), min=ref_err)).all())
    denom = scale + 1e-300
    return ok, {"err_hip": float(err.max()) / denom, "err_fp32_python": ref_err / denom, "rtol": rtol}
