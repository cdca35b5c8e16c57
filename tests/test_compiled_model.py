"""CompiledLogicNet (product, CPU codegen) against the reference's own outputs and the oracle."""
import os

import numpy as np
import pytest
import torch

import difflogic_amd as dl
from oracle import packed_oracle as po
from tests.helpers import build_model, random_layers


def _fixture_model(comp, name):
    F, k, bits, batch, L = (int(v) for v in comp[name + "_meta"])
    layers = [(comp[f"{name}_a{i}"], comp[f"{name}_b{i}"], comp[f"{name}_op{i}"]) for i in range(L)]
    return F, k, bits, build_model(F, layers, k, device="cpu")


@pytest.mark.parametrize("mode", ["unrolled", "table"])
def test_reference_fixtures(golden_dir, mode, tmp_path):
    comp = np.load(os.path.join(golden_dir, "compiled.npz"))
    for name in (str(c) for c in comp["cases"]):
        F, k, bits, model = _fixture_model(comp, name)
        net = dl.CompiledLogicNet(model, num_bits=bits, mode=mode)
        lib = str(tmp_path / f"{name}_{mode}.so")
        net.compile(opt_level=1, save_lib_path=lib)
        got = net(comp[name + "_x"])
        assert got.dtype == torch.int32 and np.array_equal(got.numpy(), comp[name + "_y"]), (name, mode)
        again = dl.CompiledLogicNet.load(lib, k, bits)
        assert np.array_equal(again(torch.as_tensor(comp[name + "_x"])).numpy(), comp[name + "_y"])


def test_modes_agree_and_single_layer_and_ragged_batches():
    rng = np.random.default_rng(0)
    for widths, k, bits in (([40], 4, 64), ([30, 30], 3, 8), ([64, 64, 50], 5, 32)):
        layers = random_layers(rng, 20, widths)
        model = build_model(20, layers, k, device="cpu")
        nets = [dl.CompiledLogicNet(model, num_bits=bits, mode=m) for m in ("unrolled", "table")]
        for n in nets:
            n.compile(opt_level=0)
        for B in (1, bits - 1, bits, 3 * bits + 5):
            x = rng.random((B, 20)) < 0.4
            want = po.net_eval_bitwise(x, layers, k)
            for n in nets:
                assert np.array_equal(n(x).numpy(), want), (widths, bits, B)


def test_default_mode_and_checks():
    rng = np.random.default_rng(1)
    model = build_model(10, random_layers(rng, 10, [20, 20]), 2, device="cpu")
    assert dl.CompiledLogicNet(model)._resolved_mode() == "unrolled"
    with pytest.raises(AssertionError):
        dl.CompiledLogicNet(torch.nn.Sequential(model[0], model[1]))          # no GroupSum at the end
    with pytest.raises(AssertionError):
        dl.CompiledLogicNet(model, num_bits=12)
    with pytest.raises(AssertionError):
        dl.CompiledLogicNet(model)(np.zeros((4, 10), bool))                    # not compiled yet


@pytest.mark.parametrize("mode", ["unrolled", "table"])
def test_openmp_variant_equals_single_threaded(mode):
    rng = np.random.default_rng(3)
    layers = random_layers(rng, 24, [96, 96, 60])
    model = build_model(24, layers, 6, device="cpu")
    x = rng.random((64 * 37 + 11, 24)) < 0.5
    want = po.net_eval_bitwise(x, layers, 6)
    for threads in (0, 3):
        net = dl.CompiledLogicNet(model, num_bits=64, mode=mode, num_threads=threads)
        assert "#pragma omp parallel" in net.get_c_code()
        net.compile(opt_level=1)
        assert np.array_equal(net(x).numpy(), want), (mode, threads)
    assert "omp" not in dl.CompiledLogicNet(model, mode=mode).get_c_code()        # the reference's single-threaded form
