"""GPU: one bounded soak.  About ten thousand calls of the library's entry points,
mixed, three at a time on three streams, over two MLP handles: wave scaling at
ragged sizes with one and several destinations, the MLP forward on both sides
of every path boundary, the static-scratch forward, host records, and a prepared
device sweep.  Every result must equal the first result of the same call bit
for bit, the sweep's totals included (its per-pass sums are added in the
kernels' order, without floating-point atomics).  Stops at the first mismatch."""
import ctypes

import numpy as np
import pytest
import torch

from habitat_amd import Device, _lib, synthetic
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from habitat_amd.analysis.predictor import Predictor
from habitat_amd.analysis.wave_scaling.batch import KernelRecords, WaveScaleOutput, wave_scale
from habitat_amd.analysis.wave_scaling.deferred import RECORD_DTYPE

pytestmark = pytest.mark.gpu

GROUPS = 3334          # x 3 calls


class Call:
    """One kind of call with its own output buffers; `issue(stream)` enqueues it
    and returns the tensors (or arrays) that hold its results."""

    def __init__(self, name, issue):
        self.name, self.issue, self.first = name, issue, None

    def check(self, results):
        if self.first is None:
            self.first = [r.clone() if isinstance(r, torch.Tensor) else r.copy() for r in results]
            return
        for got, want in zip(results, self.first):
            if isinstance(got, torch.Tensor):
                same = torch.equal(got, want) or (
                    got.dtype.is_floating_point and
                    torch.equal(torch.isnan(got), torch.isnan(want)) and
                    torch.equal(torch.nan_to_num(got), torch.nan_to_num(want)))
            else:
                same = np.array_equal(got, want, equal_nan=True)
            assert same, self.name


def test_ten_thousand_mixed_calls_repeat_bit_for_bit():
    torch.manual_seed(0)
    origin = Device.V100
    rec, _ = synthetic.kernel_records(50_000, origin, seed=31, metrics_fraction=0.7)
    streams = [torch.cuda.Stream() for _ in range(3)]
    calls = []

    # --- wave scaling on columns: ragged sizes, one and several destinations
    for n in (1, 63, 64, 65, 129, 1000, 4097, 50_000):
        part = {k: v[:n] for k, v in rec.items()}
        kr = KernelRecords.from_numpy(part)
        for dests in ([Device.MI355X], [Device.T4, Device.P100, Device.P4000, Device.RTX2070]):
            out = WaveScaleOutput(n, len(dests), kr.device)

            def issue(stream, kr=kr, dests=dests, out=out):
                wave_scale(kr, origin, dests, out=out, stream=stream)
                return [out.time_ns, out.occ_dest, out.occ_origin, out.status]
            calls.append(Call("wave_scale n=%d dests=%d" % (n, len(dests)), issue))

    # --- kernel records from host memory (the call waits for its stream)
    host = np.zeros(700, RECORD_DTYPE)
    for src, dst in (("num_blocks", "num_blocks"), ("block_size", "block_size"),
                     ("dynamic_smem", "dynamic_smem"), ("static_smem", "static_smem"),
                     ("regs_per_thread", "regs"), ("run_time_ns", "run_time_ns"),
                     ("flop_sp_efficiency", "flop_sp_efficiency"),
                     ("dram_read_bytes", "dram_read_bytes"), ("dram_write_bytes", "dram_write_bytes")):
        host[dst] = rec[src][:700]
    host["dest_regs"], host["has_metrics"] = -1, 1

    def issue_host(stream):
        t, st = np.empty(700), np.empty(700, np.uint8)
        rc = _lib.lib().hbt_wave_scale_host_records(
            ctypes.byref(origin.spec), ctypes.byref(Device.T4.spec), 700,
            ctypes.c_void_p(host.ctypes.data), ctypes.c_void_p(t.ctypes.data),
            ctypes.c_void_p(st.ctypes.data), None, None, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0
        return [t, st]
    calls.append(Call("host records", issue_host))

    # --- two MLP handles, row counts on both sides of every path boundary
    handles = {}
    for kind in ("conv2d", "lstm"):
        rp = RuntimePredictor(kind, 8, 1024)
        x, mu, sigma = synthetic.mlp_features(kind, 9000, seed=7)
        rp.set_normalization(mu, sigma)
        handles[kind] = (rp, torch.from_numpy(x).cuda())
    for kind, (rp, xg) in handles.items():
        for n in (1, 20, 21, 128, 129, 300, 2048, 2049, 4096, 4097, 7168, 7169, 8192, 9000):
            rows = xg[:n].contiguous()
            out = torch.empty(n, dtype=torch.float32, device="cuda")

            def issue(stream, rp=rp, rows=rows, out=out):
                rp.predict_batch(rows, out=out, stream=stream)
                return [out]
            calls.append(Call("mlp %s n=%d" % (kind, n), issue))

    # --- the static-scratch forward: all its calls share one array per GPU, so
    # they all go to ONE stream (streams[0]) whatever the group's turn says
    for kind, (rp, xg) in handles.items():
        for n in (1, 20, 128, 300, 1024):
            rows = xg[:n].contiguous()
            out = torch.empty(n, dtype=torch.float32, device="cuda")

            def issue(stream, rp=rp, rows=rows, out=out, n=n):
                rc = _lib.lib().hbt_mlp_forward_static(
                    rp._device_mlp().handle, ctypes.c_void_p(rows.data_ptr()), n,
                    ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(streams[0].cuda_stream))
                assert rc == 0
                return [out]
            calls.append(Call("mlp static %s n=%d" % (kind, n), issue))

    # --- a prepared device sweep (predictors of its own: its launches run the
    # networks on side streams of their own)
    sweep_preds = {}
    for kind in ("conv2d", "linear"):
        rp = RuntimePredictor(kind, 8, 1024)
        _, mu, sigma = synthetic.mlp_features(kind, 2048, seed=2)
        rp.set_normalization(mu, sigma)
        sweep_preds[kind] = rp
    trace = synthetic.resnet50_trace(origin, batch=8, seed=3)
    devices, feats = synthetic.device_sweep(16, seed=1)
    features = {d.name: list(f) for d, f in zip(devices, feats)}
    features[origin.name] = [16, 900, 80, 14.028]
    prepared = Predictor(mlp_predictors=sweep_preds).plan_trace(trace).prepare(devices, features)
    sweep_first = []

    def issue_sweep(stream):
        with torch.cuda.stream(stream):
            res = prepared.launch()
        return res
    # issued beside the three calls of every 16th group

    torch.cuda.synchronize()
    n_calls = 0
    for g in range(GROUPS):
        group = [calls[(3 * g + j * 17) % len(calls)] for j in range(3)]
        if len({id(c) for c in group}) < 3:
            group = [calls[(3 * g + j) % len(calls)] for j in range(3)]
        results = [c.issue(streams[(g + j) % 3]) for j, c in enumerate(group)]
        sweep = issue_sweep(streams[g % 3]) if g % 16 == 0 else None
        torch.cuda.synchronize()
        for c, r in zip(group, results):
            c.check(r)
        n_calls += 3
        if sweep is not None:
            n_calls += 1
            total = sweep.total_ms.clone()
            if not sweep_first:
                sweep_first.append(total)
                assert bool(torch.all(torch.isfinite(total)))
            assert torch.equal(total, sweep_first[0]), "sweep"
    assert all(c.first is not None for c in calls)
    print("soak: %d calls of %d kinds on 3 streams, every result equal to its first" %
          (n_calls, len(calls) + 1))
