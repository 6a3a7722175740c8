"""GPU: the fused MFMA MLP (through the C ABI) against the CPU oracle.
fp32 outputs within 1e-4 relative of the fp64 evaluation of the same weights
(floor 1e-3 on |reference| for outputs near zero), and no further from it than
a small multiple of what torch-CPU fp32 — the reference's own arithmetic — is."""
import json
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN
from habitat_amd import synthetic
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from oracle import mlp as omlp

pytestmark = pytest.mark.gpu

RTOL = 1e-4
ABS_FLOOR = 1e-3


def assert_close(y, y64, floor=ABS_FLOOR):
    """|y - y64| <= 1e-4 * max(|y64|, 1e-3) for every row; prints the largest
    observed ratio |y - y64| / max(|y64|, floor) (shown by pytest -rP)."""
    err = np.abs(y.astype(np.float64) - y64)
    scale = np.maximum(np.abs(y64), floor)
    if err.size:
        print("mlp: %d rows, max relative error vs fp64 %.3g (bound %.0e)"
              % (err.size, float(np.max(err / scale)), RTOL))
    assert np.all(err <= RTOL * scale), float(err.max())


def assert_no_worse_than_torch_fp32(y, y64, y32, factor, slack=0.0):
    """The criterion where outputs are differences of much larger terms, so that
    no floor for a relative bound is natural: the largest error against the fp64
    evaluation stays within `factor` times the largest error the reference's
    own arithmetic (torch CPU fp32) makes on the same rows."""
    ours = float(np.max(np.abs(y.astype(np.float64) - y64)))
    torch32 = float(np.max(np.abs(y32.astype(np.float64) - y64)))
    print("mlp: %d rows, max abs error vs fp64 %.3g; torch CPU fp32 makes %.3g (allowed: %g x)"
          % (y.shape[0], ours, torch32, factor))
    assert ours <= factor * torch32 + slack


def make(kind, seed=0, hidden=8):
    torch.manual_seed(seed)
    rp = RuntimePredictor(kind, hidden, 1024)
    return rp


@pytest.mark.parametrize("kind", ["conv2d", "linear", "bmm", "lstm"])
def test_seed0_network_4096_rows(kind):
    rp = make(kind)
    sd = rp.model.state_dict()
    with open(os.path.join(GOLDEN, "mlp_seed0.json")) as f:
        g = json.load(f)[kind]
    assert omlp.state_dict_sha256(sd) == g["sha256"]
    x, mu, sigma = synthetic.mlp_features(kind, 4096, seed=2)
    rp.set_normalization(mu, sigma)
    y = rp.predict_batch(x).cpu().numpy()
    y64 = omlp.forward_fp64(sd, x, mu, sigma)
    y32 = omlp.forward_fp32(sd, x, mu, sigma)
    assert_close(y, y64)
    assert np.max(np.abs(y - y64)) <= 8 * max(np.max(np.abs(y32 - y64)), 1e-8)
    # committed golden rows
    assert_close(y[:16], np.array(g["fp64"]))


def test_trained_like_weights_with_wide_output_range():
    # Random-init outputs barely move; scale the layers and centre the output so
    # that predictions spread over several units and change sign, which is what
    # exercises cancellation in the last dot product.
    rp = make("conv2d", seed=7)
    with torch.no_grad():
        for name, p in rp.model.named_parameters():
            if name.endswith("weight"):
                p.mul_(2.5)
            else:
                p.add_(0.05 * torch.randn_like(p))
        rp.model.fc2.weight.copy_(torch.randn(1, 1024) * 0.05)
        rp.model.fc2.bias.fill_(-1.5)
    x, mu, sigma = synthetic.mlp_features("conv2d", 8192, seed=21)
    rp.set_normalization(mu, sigma)
    sd = rp.model.state_dict()
    y = rp.predict_batch(x).cpu().numpy()
    y64 = omlp.forward_fp64(sd, x, mu, sigma)
    assert y64.max() - y64.min() > 1.0 and y64.min() < 0 < y64.max()
    # Outputs near zero are differences of terms of size |fc2.bias| = 1.5, so the
    # error is held against what torch-CPU fp32 itself makes on these rows.
    assert_no_worse_than_torch_fp32(y, y64, omlp.forward_fp32(sd, x, mu, sigma), 4)


# up to 7168 rows run one launch per layer (K split over workgroups up to 20 rows
# and over two up to 128; above that a wave per output tile, with K in four
# parts up to 2048 rows, two up to 4096 or one, whichever rounds best), more rows
# the fused kernel in whole rounds of 32 rows x 256 compute units, and up to 7168
# rows left over after the last whole round one launch per layer again
@pytest.mark.parametrize("n", [1, 2, 20, 21, 31, 32, 33, 63, 64, 65, 96, 97, 128, 129, 160, 161,
                               511, 512, 513, 1000, 1025, 2048, 2049, 2081, 4095, 4096, 4097, 4161,
                               5000, 7168, 7169, 8191, 8192, 8193, 8192 + 4096, 8192 + 7168,
                               8192 + 7169])
def test_ragged_row_counts(n):
    rp = make("lstm")
    x, mu, sigma = synthetic.mlp_features("lstm", 8192 + 7169, seed=5)
    rp.set_normalization(mu, sigma)
    y = rp.predict_batch(x[:n]).cpu().numpy()
    assert y.shape == (n,)
    assert_close(y, omlp.forward_fp64(rp.model.state_dict(), x[:n], mu, sigma))


def test_the_three_paths_agree_on_the_same_rows():
    """The same rows alone in a batch of 20 (K split over workgroups), of 300
    (one launch per layer, a wave per output tile) and inside a batch of 7500
    (fused kernel): different summation orders, same answer to rounding."""
    rp = make("conv2d")
    x, mu, sigma = synthetic.mlp_features("conv2d", 7500, seed=11)
    rp.set_normalization(mu, sigma)
    few = rp.predict_batch(x[:20]).cpu().numpy()
    alone = rp.predict_batch(x[:300]).cpu().numpy()
    inside = rp.predict_batch(x).cpu().numpy()[:300]
    y64 = omlp.forward_fp64(rp.model.state_dict(), x[:300], mu, sigma)
    assert_close(few, y64[:20])
    assert_close(alone, y64)
    assert_close(inside, y64)
    assert np.max(np.abs(alone - inside)) <= 1e-5 * np.max(np.abs(y64))
    assert np.max(np.abs(few - inside[:20])) <= 1e-5 * np.max(np.abs(y64))
    # and the per-layer paths are reproducible bit for bit
    assert np.array_equal(alone, rp.predict_batch(x[:300]).cpu().numpy())
    assert np.array_equal(few, rp.predict_batch(x[:20]).cpu().numpy())


@pytest.mark.parametrize("hidden", [0, 1, 3])
@pytest.mark.parametrize("rows", [5, 40, 130, 1500, 4200, 7500])
def test_other_depths(hidden, rows):
    """Networks with no, one and three hidden layers through all three paths
    (the kernels take the depth from the handle; without hidden layers the final
    dot product reads fc1's activations)."""
    rp = make("lstm", seed=4, hidden=hidden)
    x, mu, sigma = synthetic.mlp_features("lstm", rows, seed=8)
    rp.set_normalization(mu, sigma)
    y = rp.predict_batch(x).cpu().numpy()
    sd = rp.model.state_dict()
    y64 = omlp.forward_fp64(sd, x, mu, sigma)
    # among thousands of rows some outputs are differences of terms a hundred
    # times their size: the error is held against what torch-CPU fp32 itself
    # makes on these rows
    assert_no_worse_than_torch_fp32(y, y64, omlp.forward_fp32(sd, x, mu, sigma), 8, slack=8e-8)


@pytest.mark.parametrize("features", [21, 36, 60])
def test_wide_inputs_up_to_64_features(features):
    """The C ABI takes up to 64 input features (fc1's K padded to 32 or 64);
    the reference's predictors stop at 12, so this goes through a model class of
    the test's own."""
    from habitat_amd.analysis.mlp.mlp import _DeviceMLP, _OperationMLP

    Wide = type("Wide", (_OperationMLP,), {"features": ["f%d" % i for i in range(features)]})

    torch.manual_seed(9)
    model = Wide(1, 1024)
    rng = np.random.default_rng(9)
    f = features + 4
    x = rng.normal(3.0, 2.0, size=(7500, f))
    mu, sigma = x.mean(axis=0), x.std(axis=0)
    gpu = _DeviceMLP(model, mu, sigma)
    want = omlp.forward_fp64(model.state_dict(), x, mu, sigma)
    for rows in (20, 700, 1500, 4200, 7500):
        y = gpu.forward(torch.from_numpy(x[:rows]).cuda()).cpu().numpy()
        # outputs of this random two-layer net are sums of O(1) terms that nearly
        # cancel: the error is held against what torch-CPU fp32 itself makes
        y32 = omlp.forward_fp32(model.state_dict(), x[:rows], mu, sigma)
        assert_no_worse_than_torch_fp32(y, want[:rows], y32, 4, slack=1e-7)
    # 65 features do not fit
    TooWide = type("TooWide", (_OperationMLP,), {"features": ["f%d" % i for i in range(61)]})
    from habitat_amd import _lib
    with pytest.raises(_lib.HabitatLibraryError) as e:
        _DeviceMLP(TooWide(1, 1024), np.zeros(65), np.ones(65))
    assert e.value.code == _lib.HBT_ESIZE


def test_calls_on_one_predictor_from_two_streams_do_not_overlap():
    """Batches of up to 7168 rows run through scratch memory of the handle.  The
    Python face orders a call on another stream than the one before after that
    stream; interleaved on two streams at 300 and 4 096 rows the results must be
    the serial ones, bit for bit."""
    rp = make("conv2d")
    x, mu, sigma = synthetic.mlp_features("conv2d", 4096, seed=13)
    rp.set_normalization(mu, sigma)
    xa = torch.from_numpy(x[:300]).cuda()
    xb = torch.from_numpy(x).cuda()
    serial_a = rp.predict_batch(xa).clone()
    serial_b = rp.predict_batch(xb).clone()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for rep in range(6):
        oa = torch.empty(300, dtype=torch.float32, device="cuda")
        ob = torch.empty(4096, dtype=torch.float32, device="cuda")
        first, second = (s1, s2) if rep % 2 == 0 else (s2, s1)
        rp.predict_batch(xb, out=ob, stream=first)
        rp.predict_batch(xa, out=oa, stream=second)     # waits for `first` by itself
        rp.predict_batch(xb, out=ob, stream=first)
        outs.append((oa, ob))
    torch.cuda.synchronize()
    for oa, ob in outs:
        assert torch.equal(oa, serial_a) and torch.equal(ob, serial_b)
    # and from two threads at once
    import threading
    results = {}

    def work(name, rows, want, stream):
        torch.cuda.set_device(0)
        ok = True
        for _ in range(20):
            y = rp.predict_batch(rows, stream=stream)
            stream.synchronize()
            ok = ok and torch.equal(y, want)
        results[name] = ok

    threads = [threading.Thread(target=work, args=("a", xa, serial_a, s1)),
               threading.Thread(target=work, args=("b", xb, serial_b, s2))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert results == {"a": True, "b": True}


def test_empty_batch():
    rp = make("bmm")
    rp.set_normalization(np.zeros(8), np.ones(8))
    assert rp.predict_batch(np.zeros((0, 8))).shape == (0,)


@pytest.mark.parametrize("rows", [20, 200, 1500, 4200, 7500])
def test_exact_cases_dead_relu_and_selector_weights(rows):
    rp = make("linear", hidden=2)
    x, mu, sigma = synthetic.mlp_features("linear", rows, seed=6)
    rp.set_normalization(mu, sigma)
    with torch.no_grad():
        rp.model.mlp.layers[2].bias.fill_(-1e6)
    rp.refresh()
    y = rp.predict_batch(x).cpu().numpy()
    assert np.all(y == rp.model.fc2.bias.item())          # every ReLU dead: exact
    # Selector network: fc1 copies feature j to unit j (plus 100 so ReLU stays open),
    # hidden layers are identities, fc2 picks unit `pick` -> out = x_std[pick] + 100.
    with torch.no_grad():
        for p in rp.model.parameters():
            p.zero_()
        for j in range(8):
            rp.model.fc1.weight[j, j] = 1.0
        rp.model.fc1.bias[:8] = 100.0
        for layer in (rp.model.mlp.layers[0], rp.model.mlp.layers[2]):
            layer.weight.copy_(torch.eye(1024))
    for pick in (0, 3, 7):
        with torch.no_grad():
            rp.model.fc2.weight.zero_()
            rp.model.fc2.weight[0, pick] = 1.0
        rp.refresh()
        y = rp.predict_batch(x).cpu().numpy()
        want = (omlp.standardise(x, mu, sigma)[:, pick] + np.float32(100.0)).astype(np.float32)
        assert np.array_equal(y, want), pick


@pytest.mark.parametrize("rows", [17, 96, 600, 1500, 4200, 7500])
def test_every_weight_position_is_wired(rows):
    # One hidden layer holding a random permutation matrix scaled by distinct
    # powers of two: out[r] = sum over units of 2^-(j%8) * in[perm[j]] exactly
    # representable, so a mis-packed weight shows up as a wrong value.
    rp = make("bmm", hidden=1)
    rng = np.random.default_rng(3)
    perm = rng.permutation(1024)
    with torch.no_grad():
        for p in rp.model.parameters():
            p.zero_()
        w1 = torch.zeros(1024, 8)
        for j in range(1024):
            w1[j, j % 8] = float(1 + (j // 8) % 4)
        rp.model.fc1.weight.copy_(w1)
        rp.model.fc1.bias.fill_(64.0)
        wh = torch.zeros(1024, 1024)
        for j in range(1024):
            wh[j, perm[j]] = 2.0 ** -(j % 8)
        rp.model.mlp.layers[0].weight.copy_(wh)
        rp.model.fc2.weight.copy_(torch.from_numpy(
            (rng.integers(0, 2, 1024) * 2 - 1).astype(np.float32))[None])
    rp.set_normalization(np.zeros(8), np.ones(8))
    x = rng.integers(-4, 5, size=(rows, 8)).astype(np.float64)   # small integers: exact sums
    y = rp.predict_batch(x).cpu().numpy()
    y64 = omlp.forward_fp64(rp.model.state_dict(), x, np.zeros(8), np.ones(8))
    assert np.array_equal(y.astype(np.float64), y64)


def test_scalar_predict_and_checkpoint_round_trip(tmp_path):
    rp = make("conv2d")
    x, mu, sigma = synthetic.mlp_features("conv2d", 64, seed=2)
    rp.set_normalization(mu, sigma)
    path = str(tmp_path / "model.pth")
    rp.save_state(path)
    rp2 = RuntimePredictor("conv2d", 8, 1024, path)
    assert np.array_equal(rp2.mu, mu)
    args = [1, 32, 56, 64, 128, 3, 1, 1]
    a, b = rp.predict(args, "V100"), rp2.predict(args, "V100")
    assert isinstance(a, float) and a == b
    row = np.array([args + [16, 900, 80, 14.028]], np.float64)
    assert_close(np.array([a], np.float32), omlp.forward_fp64(rp.model.state_dict(), row, mu, sigma))
    # 64 operations one call at a time, as the reference predicts (mlp.py:252-267)
    one_by_one = np.array([rp.predict(list(r[:8]), "V100") for r in x], np.float32)
    rows = np.concatenate([x[:, :8], np.tile([16, 900, 80, 14.028], (64, 1))], axis=1)
    assert_close(one_by_one, omlp.forward_fp64(rp.model.state_dict(), rows, mu, sigma))
    # the one-row C call is the batch call with n = 1, bit for bit
    for r in rows[:8]:
        alone = rp.predict_batch(r[None, :].copy()).cpu().numpy()
        assert alone[0] == np.float32(rp.predict(list(r[:8]), "V100"))
    # asking again is answered from the table; new weights forget it
    assert len(rp._predicted) == 65
    again = rp.predict(args, "V100")
    assert again == a and len(rp._predicted) == 65
    with torch.no_grad():
        rp.model.fc2.bias.add_(1.0)
    rp.refresh()
    assert len(rp._predicted) == 0
    assert rp.predict(args, "V100") == pytest.approx(a + 1.0, abs=1e-5)
    with pytest.raises(IndexError):
        rp.predict(args, "UnknownGPU")
    with pytest.raises(TypeError):
        RuntimePredictor("conv2d", 8, 1024).predict(args, "V100")     # no mu/sigma


@pytest.mark.parametrize("kind", ["conv2d", "linear", "bmm", "lstm"])
def test_config2_and_config3_full_size_properties(kind):
    # 1M rows (configs[2]: conv2d; configs[3]: the other three): the oracle is
    # too slow for all of them, so check a strided sample against it and, over
    # the whole batch, invariance to row order.
    rp = make(kind)
    n = 1_000_000
    x, mu, sigma = synthetic.mlp_features(kind, n, seed=2)
    rp.set_normalization(mu, sigma)
    xg = torch.from_numpy(x).cuda()
    y = rp.predict_batch(xg)
    idx = np.arange(0, n, 997)
    y_host = y.cpu().numpy()
    assert_close(y_host[idx], omlp.forward_fp64(rp.model.state_dict(), x[idx], mu, sigma))
    # 100 000 rows against the reference's own arithmetic (torch CPU fp32,
    # mlp.py:252-267, batched): the first 50 000 and the last 50 000, which hold
    # the 576 rows left over after the fused kernel's whole rounds
    block = np.r_[0:50_000, n - 50_000:n]
    assert_close(y_host[block], omlp.forward_fp32(rp.model.state_dict(), x[block], mu, sigma))
    perm = torch.randperm(n, device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    y_perm = rp.predict_batch(xg[perm].contiguous())
    # a row's result does not depend on its neighbours: bit for bit where the
    # row is in the fused kernel's whole rounds (32 rows x 256 compute units)
    # both times, to rounding where it is among the rows left over, which take
    # one launch per layer
    whole = n - n % 8192
    pos = torch.arange(n, device="cuda")
    fused_both = (pos < whole) & (perm < whole)
    assert whole == 999_424 and int(fused_both.sum()) > 990_000
    assert torch.equal(y_perm[fused_both], y[perm][fused_both])
    assert torch.allclose(y_perm, y[perm], rtol=1e-5, atol=1e-7)
    assert bool(torch.all(torch.isfinite(y)))


@pytest.mark.parametrize("zero_sigma", [False, True])
def test_nan_and_infinite_features_give_what_torch_gives(zero_sigma):
    """A feature that is NaN or infinite, or a sigma of zero (a constant column
    in the training set), makes the reference's torch forward return NaN for
    that row: ReLU hands a NaN on there, where the hardware's max would return
    0.  Same rows through the three paths; the other rows stay within the
    tolerance."""
    rp = make("conv2d")
    x, mu, sigma = synthetic.mlp_features("conv2d", 9000, seed=2)
    rng = np.random.default_rng(1)
    x = x.copy()
    special = np.array([np.nan, np.inf, -np.inf, 1e300, -1e300, 3e38, 1e-300, 0.0])
    for r in rng.choice(9000, 900, replace=False):
        x[r, rng.integers(0, x.shape[1])] = rng.choice(special)
    if zero_sigma:
        sigma = np.where(np.arange(sigma.shape[0]) == 3, 0.0, sigma)
    rp.set_normalization(mu, sigma)
    sd = rp.model.state_dict()
    for rows in (20, 300, 9000):
        with np.errstate(all="ignore"):
            want = omlp.forward_fp32(sd, x[:rows], mu, sigma)
        got = rp.predict_batch(x[:rows]).cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isposinf(got), np.isposinf(want))
        assert np.array_equal(np.isneginf(got), np.isneginf(want))
        fin = np.isfinite(want)
        assert zero_sigma or (fin.sum() > 0.9 * rows and (~fin).sum() > 0.04 * rows) or rows == 20
        # fp32 against fp32 here: two summation orders of the same numbers
        assert np.all(np.abs(got[fin] - want[fin]) <= 1e-4 * np.maximum(np.abs(want[fin]), 1e-3))
    if zero_sigma:
        assert np.all(np.isnan(want))
