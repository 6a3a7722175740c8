"""Writes tests/golden/mlp_seed0.json: for each of the four networks, the
SHA-256 of the seed-0 random-init state dict (so that every machine can check
it built the same weights), 16 seeded raw feature rows with their mu/sigma, and
the fp64 and torch-CPU fp32 outputs of oracle/mlp.py for those rows.

These vectors come from this repository's oracle, not from the reference (the
reference ships neither weights nor expected outputs); what pins the oracle's
arithmetic is tests/test_oracle_mlp.py.  The fixture pins reproducibility of
the weights and inputs across machines and torch builds.

    python tests/golden/make_mlp_golden.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from habitat_amd import synthetic  # noqa: E402
from oracle import mlp as omlp  # noqa: E402

out = {}
for kind in ("conv2d", "linear", "bmm", "lstm"):
    sd = omlp.seed0_state_dict(kind)
    x, mu, sigma = synthetic.mlp_features(kind, 4096, seed=2)
    rows = x[:16]
    out[kind] = {
        "sha256": omlp.state_dict_sha256(sd),
        "mu": mu.tolist(), "sigma": sigma.tolist(), "rows": rows.tolist(),
        "fp64": omlp.forward_fp64(sd, rows, mu, sigma).tolist(),
        "fp32": [float(v) for v in omlp.forward_fp32(sd, rows, mu, sigma)],
    }
with open(os.path.join(ROOT, "tests", "golden", "mlp_seed0.json"), "w") as f:
    json.dump(out, f, indent=1)
print({k: v["sha256"][:12] for k, v in out.items()})
