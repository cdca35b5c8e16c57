"""Writes the golden fixtures in this directory.  Runs ONLY in the build container, where
the reference checkout is mounted read-only at /root/reference; the fixtures (plain .npz
data: inputs and expected outputs) are what travels.

Only the two things nothing else pins are taken from the reference by running it:

* the index tensors its connectivity initialisers return for fixed seeds
  (difflogic/difflogic.py:154-169, difflogic/functional.py:76-124), and
* the int32 class counts its CompiledLogicNet (generated C, compiled here with gcc)
  returns for seeded tiny nets (difflogic/compiled_model.py:159-370).

``difflogic/__init__.py`` imports a CUDA extension that cannot exist here, so the package
is loaded with an empty placeholder module under that name; no function of it is called
(the layers are built with device='cpu', implementation='python').

    python tests/golden/make_golden.py
"""
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference"


def load_reference():
    sys.modules.setdefault("difflogic_cuda", types.ModuleType("difflogic_cuda"))
    sys.path.insert(0, REF)
    import difflogic  # noqa: F401
    from difflogic import CompiledLogicNet, GroupSum, LogicLayer
    from difflogic.functional import get_unique_connections
    return LogicLayer, GroupSum, CompiledLogicNet, get_unique_connections


def connections_fixture(LogicLayer, get_unique_connections):
    out = {}
    cases = []
    # unique: only torch.randperm(out) is drawn
    for in_dim, out_dim, seed in [(20, 16, 0), (7, 20, 1), (784, 8000, 0), (8000, 8000, 3), (10, 40, 2),
                                  (11, 6, 5)]:
        torch.manual_seed(seed)
        a, b = get_unique_connections(in_dim, out_dim, "cpu")
        key = f"unique_{in_dim}_{out_dim}_{seed}"
        out[key + "_a"], out[key + "_b"] = a.numpy(), b.numpy()
        cases.append(key)
    # random, through the layer's constructor on CPU: randn(out,16) is drawn first
    for in_dim, out_dim, seed in [(20, 16, 0), (7, 30, 1), (784, 8000, 0), (8000, 8000, 3)]:
        torch.manual_seed(seed)
        layer = LogicLayer(in_dim, out_dim, device="cpu", implementation="python", connections="random")
        key = f"randomctor_{in_dim}_{out_dim}_{seed}"
        out[key + "_a"], out[key + "_b"] = layer.indices[0].numpy(), layer.indices[1].numpy()
        out[key + "_w00"] = layer.weights.detach().numpy()[0]
        cases.append(key)
    out["cases"] = np.array(cases)
    np.savez_compressed(os.path.join(HERE, "connections.npz"), **out)
    print("connections.npz:", len(cases), "cases")


def compiled_fixture(LogicLayer, GroupSum, CompiledLogicNet):
    out = {}
    cases = []
    specs = [
        # name, F, widths, k, connections, bits, batch, seed, opt
        ("tiny64", 12, [24, 24, 30], 3, "random", 64, 200, 0, 1),
        ("tiny32", 12, [24, 24, 30], 3, "random", 32, 100, 1, 1),
        ("tiny16", 9, [18, 20], 2, "unique", 16, 50, 2, 1),
        ("tiny8", 9, [18, 20], 5, "unique", 8, 27, 3, 0),
        ("ragged_k", 16, [40, 33], 3, "random", 64, 130, 4, 1),   # 33 % 3 == 0; 40 -> 33
        ("deep64", 20, [40, 40, 40, 40, 40, 50], 10, "random", 64, 64, 5, 0),
        ("wide64", 60, [600, 600, 1000], 10, "unique", 64, 192, 6, 0),
    ]
    for name, F, widths, k, conn, bits, batch, seed, opt in specs:
        torch.manual_seed(seed)
        mods = [torch.nn.Flatten()]
        d = F
        for w in widths:
            mods.append(LogicLayer(d, w, device="cpu", implementation="python", connections=conn))
            d = w
        mods.append(GroupSum(k, 1.0, device="cpu"))
        model = torch.nn.Sequential(*mods)
        net = CompiledLogicNet(model, num_bits=bits, cpu_compiler="gcc")
        net.compile(opt_level=opt)
        g = torch.Generator().manual_seed(1000 + seed)
        x = torch.rand(batch, F, generator=g) < 0.35
        y = net(x.numpy()).numpy().astype(np.int32)
        out[name + "_x"] = x.numpy()
        out[name + "_y"] = y
        out[name + "_meta"] = np.array([F, k, bits, batch, len(widths)], dtype=np.int64)
        for li, layer in enumerate(m for m in model if isinstance(m, LogicLayer)):
            out[f"{name}_a{li}"] = layer.indices[0].numpy()
            out[f"{name}_b{li}"] = layer.indices[1].numpy()
            out[f"{name}_op{li}"] = layer.weights.argmax(-1).numpy().astype(np.uint8)
        cases.append(name)
    out["cases"] = np.array(cases)
    np.savez_compressed(os.path.join(HERE, "compiled.npz"), **out)
    print("compiled.npz:", len(cases), "cases")


if __name__ == "__main__":
    LogicLayer, GroupSum, CompiledLogicNet, get_unique_connections = load_reference()
    connections_fixture(LogicLayer, get_unique_connections)
    compiled_fixture(LogicLayer, GroupSum, CompiledLogicNet)
