"""GPU: hbt_mlp_forward_static, the MLP forward whose scratch memory is a static
device array of the library (for callers that cannot allocate), called through
the C ABI and held against hbt_mlp_forward on the same handle and rows.  Both
run the same per-layer kernels, so the results must be identical bit for bit;
the oracle's fp64 evaluation bounds both (1e-4 relative, floor 1e-3)."""
import ctypes

import numpy as np
import pytest
import torch

from habitat_amd import _lib, synthetic
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from oracle import mlp as omlp

pytestmark = pytest.mark.gpu


def _forward(entry, handle, raw, n, out):
    stream = torch.cuda.current_stream()
    return getattr(_lib.lib(), entry)(handle, ctypes.c_void_p(raw.data_ptr()), n,
                                      ctypes.c_void_p(out.data_ptr()),
                                      ctypes.c_void_p(stream.cuda_stream))


@pytest.mark.parametrize("kind", ["conv2d", "lstm"])
def test_static_scratch_forward_equals_the_handle_scratch_forward(kind):
    torch.manual_seed(0)
    rp = RuntimePredictor(kind, 8, 1024)
    x, mu, sigma = synthetic.mlp_features(kind, 1024, seed=4)
    rp.set_normalization(mu, sigma)
    handle = rp._device_mlp().handle
    raw = torch.from_numpy(x).cuda()
    y64 = omlp.forward_fp64(rp.model.state_dict(), x, mu, sigma)
    # two calls in a row per pair, the second with fewer rows than the first, so
    # that whatever the larger call left in the array lies beside and behind
    # the smaller one's rows; then the other kernel shapes (K split over
    # workgroups up to 20 rows, over two workgroups up to 128 rows) and the limit
    for n in (700, 45, 1024, 20, 128, 1, 300):
        want = torch.full((n,), -1.0, dtype=torch.float32, device="cuda")
        got = torch.full((n,), -2.0, dtype=torch.float32, device="cuda")
        assert _forward("hbt_mlp_forward", handle, raw, n, want) == 0
        assert _forward("hbt_mlp_forward_static", handle, raw, n, got) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), n
        y = got.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(y - y64[:n]) <= 1e-4 * np.maximum(np.abs(y64[:n]), 1e-3)), n
    # rows from the middle of the matrix: the result belongs to the rows, not to
    # what an earlier call left behind
    part = raw[500:545].contiguous()
    got = torch.empty((45,), dtype=torch.float32, device="cuda")
    assert _forward("hbt_mlp_forward_static", handle, part, 45, got) == 0
    want = torch.empty((45,), dtype=torch.float32, device="cuda")
    assert _forward("hbt_mlp_forward", handle, part, 45, want) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_static_scratch_forward_rejects_what_it_cannot_hold():
    torch.manual_seed(0)
    rp = RuntimePredictor("linear", 8, 1024)
    x, mu, sigma = synthetic.mlp_features("linear", 1100, seed=4)
    rp.set_normalization(mu, sigma)
    handle = rp._device_mlp().handle
    raw = torch.from_numpy(x).cuda()
    out = torch.zeros((1100,), dtype=torch.float32, device="cuda")
    assert _lib.MLP_STATIC_MAX_ROWS == 1024
    assert _forward("hbt_mlp_forward_static", handle, raw, 1025, out) == _lib.HBT_ESIZE
    assert _forward("hbt_mlp_forward_static", handle, raw, -1, out) == _lib.HBT_EINVAL
    assert _forward("hbt_mlp_forward_static", None, raw, 4, out) == _lib.HBT_EINVAL
    assert _forward("hbt_mlp_forward_static", handle, raw, 0, out) == 0
    assert _lib.lib().hbt_mlp_forward_static(handle, None, 4, ctypes.c_void_p(out.data_ptr()),
                                             None) == _lib.HBT_EINVAL
    torch.cuda.synchronize()
    assert not out.any()            # nothing was launched
    # a second handle shares the array: calls one after the other on a stream are ordered
    torch.manual_seed(1)
    other = RuntimePredictor("linear", 8, 1024)
    other.set_normalization(mu, sigma)
    a = torch.empty((64,), dtype=torch.float32, device="cuda")
    b = torch.empty((64,), dtype=torch.float32, device="cuda")
    assert _forward("hbt_mlp_forward_static", handle, raw, 64, a) == 0
    assert _forward("hbt_mlp_forward_static", other._device_mlp().handle, raw, 64, b) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, rp.predict_batch(raw[:64]))
    assert torch.equal(b, other.predict_batch(raw[:64]))
    assert not torch.equal(a, b)


def test_static_scratch_forward_inside_a_hip_graph():
    """What the entry point is for: a caller under graph capture.  The first
    call on a device looks the array's address up and is made eagerly; a
    captured call then replays, with eager work and synchronisations between
    the replays, to the eager result bit for bit, also after the input rows
    changed in place."""
    torch.manual_seed(0)
    rp = RuntimePredictor("conv2d", 8, 1024)
    x, mu, sigma = synthetic.mlp_features("conv2d", 600, seed=9)
    rp.set_normalization(mu, sigma)
    handle = rp._device_mlp().handle
    lib = _lib.lib()
    first, second = torch.from_numpy(x[:300]).cuda(), torch.from_numpy(x[300:]).cuda()
    raw = first.clone()
    eager = torch.empty((300,), dtype=torch.float32, device="cuda")
    assert _forward("hbt_mlp_forward_static", handle, raw, 300, eager) == 0    # outside capture
    torch.cuda.synchronize()
    want_first = eager.clone()
    out = torch.full((300,), -1.0, dtype=torch.float32, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.hbt_mlp_forward_static(handle, ctypes.c_void_p(raw.data_ptr()), 300,
                                        ctypes.c_void_p(out.data_ptr()),
                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert float(out[0]) == -1.0                      # captured, not run
    raw.copy_(second)
    assert _forward("hbt_mlp_forward", handle, raw, 300, eager) == 0
    torch.cuda.synchronize()
    want_second = eager.clone()
    assert not torch.equal(want_first, want_second)
    for rep in range(4):
        rows, want = (first, want_first) if rep % 2 == 0 else (second, want_second)
        raw.copy_(rows)
        out.fill_(-1.0)
        graph.replay()
        # eager work of the program's own between the replays
        other = rp.predict_batch(first[:40])
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        assert torch.equal(other, want_first[:40]) or torch.allclose(other, want_first[:40],
                                                                     rtol=1e-5, atol=1e-7)
