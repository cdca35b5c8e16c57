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
