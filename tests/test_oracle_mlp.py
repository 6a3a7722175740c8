"""CPU: pins oracle/mlp.py — a hand-computed tiny network, dead-ReLU and
linear special cases, fp32-vs-fp64 agreement, seed-0 reproducibility."""
import json
import os

import numpy as np
import torch

from conftest import GOLDEN
from habitat_amd import synthetic
from oracle import mlp as omlp


def _sd(layers):
    """layers: [(W, b)] as nested lists -> state dict with the reference's keys."""
    names = omlp.layer_names(len(layers) - 2)
    sd = {}
    for name, (w, b) in zip(names, layers):
        sd[name + ".weight"] = torch.tensor(w, dtype=torch.float32)
        sd[name + ".bias"] = torch.tensor(b, dtype=torch.float32)
    return sd


def test_layer_names_are_the_reference_state_dict_keys():
    assert omlp.layer_names(2) == ["fc1", "mlp.layers.0", "mlp.layers.2", "fc2"]
    sd = omlp.seed0_state_dict("bmm", hidden=2, width=8)
    assert sorted(sd) == sorted(
        [n + s for n in ("fc1", "mlp.layers.0", "mlp.layers.2", "fc2") for s in (".weight", ".bias")])
    assert sd["fc1.weight"].shape == (8, 8) and sd["fc2.weight"].shape == (1, 8)


def test_hand_computed_network():
    # 2 inputs, width 2, one hidden layer; every number checked on paper:
    # x = (raw - mu) / sigma = ((3-1)/2, (10-4)/3) = (1, 2)
    # fc1: [1*1 + 2*(-1) + 0.5, 2*1 + 0*2 - 1] = [-0.5, 1] -> relu [0, 1]
    # hidden: [0*3 + 1*2 + 0, 0*1 + 1*(-4) + 1] = [2, -3] -> relu [2, 0]
    # fc2: 2*0.25 + 0*7 + 0.125 = 0.625
    sd = _sd([([[1, -1], [2, 0]], [0.5, -1.0]), ([[3, 2], [1, -4]], [0.0, 1.0]),
              ([[0.25, 7.0]], [0.125])])
    raw = np.array([[3.0, 10.0]])
    mu, sigma = np.array([1.0, 4.0]), np.array([2.0, 3.0])
    assert omlp.forward_fp64(sd, raw, mu, sigma)[0] == 0.625
    assert omlp.forward_fp32(sd, raw, mu, sigma)[0] == np.float32(0.625)


def test_dead_relu_gives_fc2_bias():
    sd = omlp.seed0_state_dict("linear", hidden=2, width=16, seed=3)
    sd["mlp.layers.2.bias"] = torch.full((16,), -1e6)
    x, mu, sigma = synthetic.mlp_features("linear", 64, seed=2)
    y = omlp.forward_fp64(sd, x, mu, sigma)
    assert np.all(y == float(sd["fc2.bias"][0]))
    assert np.all(omlp.forward_fp32(sd, x, mu, sigma) == sd["fc2.bias"][0].item())


def test_linear_when_relu_is_inactive():
    # Large positive biases keep every ReLU open, so the network is affine in
    # its standardised input: f(a) + f(b) - f(0) = f(a + b).
    sd = omlp.seed0_state_dict("bmm", hidden=2, width=16, seed=4)
    for k in sd:
        if k.endswith(".bias") and not k.startswith("fc2"):
            sd[k] = torch.full_like(sd[k], 50.0)
    mu, sigma = np.zeros(8), np.ones(8)
    rng = np.random.default_rng(0)
    a, b = rng.normal(size=(5, 8)), rng.normal(size=(5, 8))
    f = lambda x: omlp.forward_fp64(sd, x, mu, sigma)
    np.testing.assert_allclose(f(a) + f(b) - f(np.zeros((5, 8))), f(a + b), rtol=1e-9)


def test_standardisation_is_fp64_then_cast():
    raw = np.array([[1e9 + 1.0, 3.0]])
    mu, sigma = np.array([1e9, 1.0]), np.array([3.0, 7.0])
    x = omlp.standardise(raw, mu, sigma)
    assert x.dtype == np.float32
    assert x[0, 0] == np.float32(1.0 / 3.0)      # exact in fp64, lost if cast first
    assert x[0, 1] == np.float32(2.0 / 7.0)


def test_seed0_networks_are_reproducible_and_two_evaluations_agree():
    with open(os.path.join(GOLDEN, "mlp_seed0.json")) as f:
        golden = json.load(f)
    for kind, g in golden.items():
        sd = omlp.seed0_state_dict(kind)
        assert omlp.state_dict_sha256(sd) == g["sha256"], kind
        x, mu, sigma = synthetic.mlp_features(kind, 4096, seed=2)
        assert np.array_equal(x[:16], np.array(g["rows"]))
        np.testing.assert_array_equal(mu, np.array(g["mu"]))
        y64 = omlp.forward_fp64(sd, x[:16], mu, sigma)
        np.testing.assert_allclose(y64, np.array(g["fp64"]), rtol=1e-12)
        y32 = omlp.forward_fp32(sd, x[:16], mu, sigma)
        np.testing.assert_allclose(y32, y64, rtol=1e-4)
        np.testing.assert_allclose(y32, np.array(g["fp32"]), rtol=1e-5)
