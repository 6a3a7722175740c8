"""TEST INFRASTRUCTURE — CPU oracle, not product code.

The per-operation MLP of the reference, restated on the CPU:
  topology            analyzer/habitat/analysis/mlp/mlp.py:17-109
                      fc1 (F+4 -> W), ReLU, L x [Linear(W, W), ReLU], fc2 (W -> 1)
  prediction          analyzer/habitat/analysis/mlp/mlp.py:252-267
                      x = (raw - mu) / sigma in fp64, cast to fp32, forward
  construction order  fc1, hidden layers, fc2 (mlp.py:80-82, :21-25), which fixes
                      what torch.manual_seed(0) produces

Two evaluations of the same weights:
  forward_fp64   numpy, every product and sum in fp64 (the mathematical truth
                 for fp32 inputs and weights)
  forward_fp32   torch on the CPU in fp32, which is what the reference runs

The arithmetic inside nn.Linear belongs to PyTorch (the reference pins
torch==1.4.0, docker/Dockerfile:14; its source is not in the reference tree and
the reference holds no vectors for it), so the only thing the reference itself
fixes is the formula y = x W^T + b: beyond that formula this function is
"parity unpinned" by the reference, and pinned by mathematics instead.
pins (tests/test_oracle_mlp.py): a
hand-computed 2-layer width-4 network; the all-ReLU-dead case (output =
fc2.bias); linearity with ReLU inactive; agreement of the two evaluations;
committed golden rows for the seed-0 networks (tests/golden/mlp_seed0.json).
"""
import hashlib

import numpy as np
import torch

FEATURES = {
    "linear": 4, "lstm": 7, "conv2d": 8, "bmm": 4,   # operation features; +4 device features
}


def layer_names(hidden):
    return ["fc1"] + ["mlp.layers.%d" % (2 * i) for i in range(hidden)] + ["fc2"]


def seed0_state_dict(kind, hidden=8, width=1024, seed=0):
    """Random-init weights exactly as `torch.manual_seed(seed)` followed by the
    reference's constructor would produce them: nn.Linear layers created in the
    order fc1, hidden[0..], fc2, each with torch's default initialisation."""
    torch.manual_seed(seed)
    in_features = FEATURES[kind] + 4
    layers = [torch.nn.Linear(in_features, width)]
    layers += [torch.nn.Linear(width, width) for _ in range(hidden)]
    layers += [torch.nn.Linear(width, 1)]
    sd = {}
    for name, lin in zip(layer_names(hidden), layers):
        sd[name + ".weight"] = lin.weight.detach().clone()
        sd[name + ".bias"] = lin.bias.detach().clone()
    return sd


def state_dict_sha256(sd):
    h = hashlib.sha256()
    for k in sorted(sd):
        h.update(k.encode())
        h.update(sd[k].detach().cpu().contiguous().numpy().tobytes())
    return h.hexdigest()


def _layers(sd):
    hidden = sorted(int(k.split(".")[2]) for k in sd
                    if k.startswith("mlp.layers.") and k.endswith(".weight"))
    names = ["fc1"] + ["mlp.layers.%d" % i for i in hidden] + ["fc2"]
    return [(sd[n + ".weight"], sd[n + ".bias"]) for n in names]


def standardise(raw, mu, sigma):
    """mlp.py:258-264: fp64 standardisation, then the cast to fp32."""
    x = (np.asarray(raw, np.float64) - np.asarray(mu, np.float64)) / np.asarray(sigma, np.float64)
    return x.astype(np.float32)


def forward_fp64(sd, raw, mu, sigma):
    x = standardise(raw, mu, sigma).astype(np.float64)
    layers = _layers(sd)
    for i, (w, b) in enumerate(layers):
        x = x @ w.detach().cpu().numpy().astype(np.float64).T + b.detach().cpu().numpy().astype(np.float64)
        if i + 1 < len(layers):
            x = np.maximum(x, 0.0)
    return x[:, 0]


def forward_fp32(sd, raw, mu, sigma, threads=None):
    if threads is not None:
        torch.set_num_threads(threads)
    x = torch.from_numpy(standardise(raw, mu, sigma))
    layers = _layers(sd)
    with torch.no_grad():
        for i, (w, b) in enumerate(layers):
            x = torch.nn.functional.linear(x, w.float(), b.float())
            if i + 1 < len(layers):
                x = torch.relu(x)
    return x[:, 0].numpy()
