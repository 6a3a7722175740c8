"""GPU: the fused per-pass sums (hbt_wave_scale_sum), the ratio kernel
(hbt_ratio_scale) and the 256-device sweep of BASELINE's end-to-end
configuration, against the CPU oracle."""
import numpy as np
import pytest
import torch

from conftest import oracle_device
from habitat_amd import Device, DeviceProperties, _lib, synthetic
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from habitat_amd.analysis.predictor import Predictor
from habitat_amd.analysis.wave_scaling.batch import (DeviceTable, KernelRecords, ratio_scale,
                                                     wave_scale, wave_scale_sum)
from oracle import lib as olib
from oracle import mlp as omlp
from oracle import predictor as opred

pytestmark = pytest.mark.gpu


def odev(d):
    return oracle_device(d.as_dict())


def oracle_sums(rec, origin, dest, segment, n_seg):
    want = olib.wave_scale(odev(origin), odev(dest), rec)
    sums = np.zeros(n_seg)
    ok = want["status"] == 0
    np.add.at(sums, segment[ok], want["time_ns"][ok])
    return sums, int((~ok).sum())


@pytest.mark.parametrize("n,n_seg,sorted_segments", [(1, 1, True), (63, 5, True), (64, 1, True),
                                                     (1000, 37, True), (1000, 37, False),
                                                     (5000, 1, True), (4097, 300, True)])
def test_fused_sums_match_oracle(n, n_seg, sorted_segments):
    origin = Device.V100
    rec, _ = synthetic.kernel_records(n, origin, seed=n + n_seg, metrics_fraction=0.5)
    rng = np.random.default_rng(n)
    segment = rng.integers(0, n_seg, n).astype(np.int32)
    if sorted_segments:
        segment.sort()
    dests = [Device.MI355X, Device.T4, Device.P100, Device.P4000, Device.V100]
    table = DeviceTable(origin, dests)
    sums, bad = wave_scale_sum(KernelRecords.from_numpy(rec), table,
                               torch.from_numpy(segment).cuda(), n_seg)
    sums, bad = sums.cpu().numpy(), bad.cpu().numpy()
    worst = 0.0
    for di, d in enumerate(dests):
        want, want_bad = oracle_sums(rec, origin, d, segment, n_seg)
        np.testing.assert_allclose(sums[di], want, rtol=1e-6, atol=0)
        assert bad[di] == want_bad
        nz = want != 0
        if nz.any():
            worst = max(worst, float(np.max(np.abs(sums[di][nz] - want[nz]) / np.abs(want[nz]))))
    print("fused per-segment sums, %d records in %d segments x %d destinations: max relative "
          "error vs oracle %.3g (bound 1e-06)" % (n, n_seg, len(dests), worst))


@pytest.mark.parametrize("n,n_seg", [(1, 1), (900, 245), (5000, 3), (4097, 300), (70_000, 64)])
def test_ordered_sums_are_the_sequential_sums_bit_for_bit(n, n_seg):
    """hbt_wave_scale_sum_ordered adds a segment's scaled times in the records'
    order, as the reference adds a pass's kernels (run_time.py:50-58): the
    result must equal the sequential fp64 sum of the per-record kernel's times,
    bit for bit, whatever the segment lengths (empty ones included), and come
    out the same on every call; the atomic version agrees with it to rounding."""
    origin = Device.V100
    rec, _ = synthetic.kernel_records(n, origin, seed=n + n_seg, metrics_fraction=0.5)
    rng = np.random.default_rng(n)
    cuts = np.sort(rng.integers(0, n + 1, n_seg - 1))
    start = np.concatenate([[0], cuts, [n]]).astype(np.int64)      # some segments are empty
    segment = np.repeat(np.arange(n_seg, dtype=np.int32), np.diff(start))
    dests = [Device.MI355X, Device.T4, Device.P100, Device.P4000, Device.V100]
    kr = KernelRecords.from_numpy(rec)
    table = DeviceTable(origin, dests)
    start_gpu = torch.from_numpy(start).cuda()
    sums, bad = wave_scale_sum(kr, table, n_segments=n_seg, segment_start=start_gpu)
    again, bad_again = wave_scale_sum(kr, table, n_segments=n_seg, segment_start=start_gpu)
    assert torch.equal(sums, again) and torch.equal(bad, bad_again)
    # (one destination per launch: a launch with several forms gamma above the
    # ridge as a product and can differ from these in the last bits)
    single = [wave_scale(kr, origin, [d]) for d in dests]
    t = np.stack([o.time_ns[0].cpu().numpy() for o in single])
    st = np.stack([o.status[0].cpu().numpy() for o in single])
    got = sums.cpu().numpy()
    for di in range(len(dests)):
        for s in range(n_seg):
            want = 0.0
            for j in range(start[s], start[s + 1]):
                if st[di, j] == 0:
                    want += t[di, j]
            assert got[di, s] == want, (di, s)
        assert int(bad[di]) == int((st[di] != 0).sum())
    atomic, atomic_bad = wave_scale_sum(kr, table, torch.from_numpy(segment).cuda(), n_seg)
    assert torch.equal(atomic_bad, bad)
    np.testing.assert_allclose(atomic.cpu().numpy(), got, rtol=1e-12, atol=0)
    # boundaries outside the columns are clamped, not followed
    wild = torch.tensor([-5] + [n + 1000] * n_seg, dtype=torch.int64, device="cuda")
    clamped, _ = wave_scale_sum(kr, table, n_segments=n_seg, segment_start=wild)
    assert bool(torch.all(torch.isfinite(clamped)))


def test_fused_sums_count_records_the_reference_would_raise_on(kat):
    base = dict(kat["scaling_record"])
    rows = [dict(base, num_blocks=10, dynamic_smem=60000),        # status 2 on V100
            dict(base, num_blocks=100, dram_read_bytes=-3e8),     # status 3 everywhere
            dict(base, num_blocks=4096), dict(base, num_blocks=50)]
    rec = {k: np.array([r[k] for r in rows]) for k in rows[0]}
    table = DeviceTable(Device.MI355X, [Device.V100, Device.MI355X])
    sums, bad = wave_scale_sum(KernelRecords.from_numpy(rec), table)
    assert bad.cpu().tolist() == [2, 1]
    for di, d in enumerate([Device.V100, Device.MI355X]):
        want, _ = oracle_sums(rec, Device.MI355X, d, np.zeros(4, np.int32), 1)
        np.testing.assert_allclose(sums[di].cpu().numpy(), want, rtol=1e-6)


def test_fused_sums_equal_the_per_record_kernel_summed():
    origin = Device.V100
    rec, _ = synthetic.kernel_records(20_000, origin, seed=77)
    devices, _ = synthetic.device_sweep(40, seed=1)
    kr = KernelRecords.from_numpy(rec)
    per_record = wave_scale(kr, origin, devices)
    sums, bad = wave_scale_sum(kr, DeviceTable(origin, devices))
    t = torch.where(per_record.status == 0, per_record.time_ns, torch.zeros_like(per_record.time_ns))
    np.testing.assert_allclose(sums[:, 0].cpu().numpy(), t.sum(dim=1).cpu().numpy(), rtol=1e-10)
    assert torch.equal(bad, (per_record.status != 0).sum(dim=1).to(torch.int32))


def test_ratio_scale_matches_python_arithmetic():
    rng = np.random.default_rng(5)
    D, O = 7, 300
    pred = rng.normal(0.05, 0.03, size=(D + 1, O)).astype(np.float32)   # some negative
    pred[D] = np.abs(pred[D]) + 0.01
    ms = rng.uniform(0.01, 20.0, O)
    totals = torch.full((D,), 2.5, dtype=torch.float64, device="cuda")
    out = ratio_scale(torch.from_numpy(pred).cuda(), torch.from_numpy(ms).cuda(), D, totals=totals)
    out = out.cpu().numpy()
    for d in range(D):
        want = [opred.special_op_ms(ms[o], float(pred[d, o]), float(pred[D, o])) for o in range(O)]
        assert np.array_equal(out[d], np.array(want))            # same fp64 operations
        assert totals[d].item() == pytest.approx(2.5 + sum(want), rel=1e-12)
    assert (out == 0).any()
    # operations that share MLP rows: column op_row[o] of pred; the negative
    # predictions the reference warns about (predictor.py:135-141) are counted
    U = 40
    op_row = rng.integers(0, U, O).astype(np.int32)
    shared = np.ascontiguousarray(pred[:, :U])
    totals = torch.zeros((D,), dtype=torch.float64, device="cuda")
    clamped = torch.full((D,), 3, dtype=torch.int32, device="cuda")
    out = ratio_scale(torch.from_numpy(shared).cuda(), torch.from_numpy(ms).cuda(), D,
                      totals=totals, op_row=torch.from_numpy(op_row).cuda(),
                      clamped=clamped).cpu().numpy()
    for d in range(D):
        raw = [ms[o] * float(shared[d, op_row[o]]) / float(shared[D, op_row[o]]) for o in range(O)]
        want = [opred.special_op_ms(ms[o], float(shared[d, op_row[o]]), float(shared[D, op_row[o]]))
                for o in range(O)]
        assert np.array_equal(out[d], np.array(want))
        assert totals[d].item() == pytest.approx(sum(want), rel=1e-12)
        assert clamped[d].item() == 3 + sum(1 for v in raw if v < 0)
    assert int(clamped.sum().item()) > 3 * D
    # a column index outside the table gives NaN instead of a stray read
    op_row[5] = U
    op_row[6] = -1
    out = ratio_scale(torch.from_numpy(shared).cuda(), torch.from_numpy(ms).cuda(), D,
                      op_row=torch.from_numpy(op_row).cuda()).cpu().numpy()
    assert np.isnan(out[:, 5]).all() and np.isnan(out[:, 6]).all()
    assert not np.isnan(np.delete(out, [5, 6], axis=1)).any()
    # counters alone
    only = torch.zeros((D,), dtype=torch.int32, device="cuda")
    assert ratio_scale(torch.from_numpy(pred).cuda(), torch.from_numpy(ms).cuda(), D,
                       want_ms=False, clamped=only) is None
    assert only.cpu().tolist() == [int((pred[d] < 0).sum()) for d in range(D)]


def test_sweep_shares_rows_of_equal_operations_and_counts_clamped_ones(caplog):
    """ResNet-50 repeats its layer shapes: the sweep evaluates each distinct
    feature row once per device and every operation still gets its own time.
    A network that predicts negative times on some devices is clamped to 0 and
    counted, with one warning for the sweep (the reference warns per operation,
    predictor.py:135-141)."""
    import logging
    predictor, trace, devices, feats = _sweep_fixture(12)
    plan = predictor.plan_trace(trace)
    idxs, pred, op_feats, ms, op_row = plan.special["conv2d"]
    assert len(idxs) == 53 and op_feats.shape[0] < 53          # shared rows
    assert op_row.shape == (53,) and int(op_row.max()) == op_feats.shape[0] - 1
    sweep = plan.run(devices, feats)
    per_op = sweep.special_ms["conv2d"].cpu().numpy()
    assert per_op.shape == (12, 53)
    assert int(sweep.clamped_ops.sum().item()) == 0
    # against one operation at a time on three of the devices
    from habitat_amd.analysis.mlp import devices as md
    try:
        for d, f in zip(devices, synthetic.device_sweep(12, seed=1)[1]):
            md.register_device(d.name, *f)
        for di in (0, 5, 11):
            for col in (0, 17, 52):
                op = trace.operations[idxs[col]]
                single = predictor.predict_operation(op, devices[di]).run_time_ms
                assert per_op[di, col] == pytest.approx(single, rel=1e-5)
    finally:
        for d in devices:
            md.unregister_device(d.name)
    # a network whose output is  num_sms - 100  (no normalisation): negative on
    # every device with fewer than 100 SMs, positive on the origin's copy of 150
    rp = predictor.conv2d_pred
    with torch.no_grad():
        for prm in rp.model.parameters():
            prm.zero_()
        rp.model.fc1.weight[0, 10] = 1.0
        for layer in list(rp.model.mlp.layers)[::2]:
            layer.weight.copy_(torch.eye(1024))
        rp.model.fc2.weight[0, 0] = 1.0
        rp.model.fc2.bias.fill_(-100.0)
    rp.set_normalization(np.zeros(12), np.ones(12))
    feats = dict(feats)
    feats[Device.V100.name] = [16, 900, 150, 14.028]
    with caplog.at_level(logging.WARNING, logger="habitat_amd.analysis.sweep"):
        totals = predictor.predict_trace_times(trace, devices, feats)
    sweep = predictor.predict_trace_sweep(trace, devices, feats)
    counts = sweep.clamped_ops.cpu().tolist()
    small = [f[2] < 100 for f in synthetic.device_sweep(12, seed=1)[1]]
    assert any(small) and not all(small)
    assert counts == [53 if s else 0 for s in small]
    per_op = sweep.special_ms["conv2d"].cpu().numpy()
    for di, s in enumerate(small):
        assert (per_op[di] == 0).all() == s
    assert sum("negative predicted run time" in r.message for r in caplog.records) == 1
    assert np.isfinite(totals).all()


def test_end_to_end_256_device_sweep():
    """BASELINE configs[4]: a ResNet-50-shaped trace against 256 destinations."""
    origin = Device.V100
    trace = synthetic.resnet50_trace(origin, batch=32, seed=3)
    preds = {}
    for kind in ("conv2d", "linear", "bmm", "lstm"):
        torch.manual_seed(0)
        rp = RuntimePredictor(kind, 8, 1024)
        x, mu, sigma = synthetic.mlp_features(kind, 2048, seed=2)
        rp.set_normalization(mu, sigma)
        preds[kind] = rp
    predictor = Predictor(mlp_predictors=preds)
    devices, feats = synthetic.device_sweep(256, seed=1)
    device_features = {d.name: list(f) for d, f in zip(devices, feats)}
    device_features[origin.name] = [16, 900, 80, 14.028]
    sweep = predictor.predict_trace_sweep(trace, devices, device_features)
    totals = sweep.total_ms.cpu().numpy()
    assert totals.shape == (256,) and np.all(np.isfinite(totals)) and np.all(totals > 0)
    assert int(sweep.bad_records.sum().item()) == 0

    # oracle, for a sample of destinations
    from test_api_gpu import as_record
    from habitat_amd.analysis import predictor as P
    from habitat_amd.analysis.metrics import Metric
    from oracle import wave_scaling as ows
    o = odev(origin)
    for di in (0, 100, 255):
        d = odev(devices[di])
        total = 0.0
        for op in trace.operations:
            if op.name in ("conv2d", "linear"):
                rp = preds[op.name]
                a = P._ARGUMENTS[op.name](op)
                f = [a[x] for x in rp.model.features]
                rows = np.array([f + device_features[devices[di].name],
                                 f + device_features[origin.name]], np.float64)
                y = omlp.forward_fp64(rp.model.state_dict(), rows, rp.mu, rp.sigma)
                total += opred.special_op_ms(op.run_time_ms, y[0], y[1])
                continue
            for rt in (op.forward, op.backward):
                if rt is None:
                    continue
                pk = []
                for k in rt.kernels:
                    try:
                        m = tuple(k.get_metric(x) for x in (Metric.SinglePrecisionFLOPEfficiency,
                                                            Metric.DRAMReadBytes,
                                                            Metric.DRAMWriteBytes))
                    except AttributeError:
                        m = None
                    pk.append(ows.unified(as_record(k, m), o, d, has_metrics=m is not None))
                total += opred.wave_scaled_pass_ms(rt.run_time_ms,
                                                   [k.run_time_ns for k in rt.kernels], pk)
        assert totals[di] == pytest.approx(total, rel=1e-5)
        print("256-device sweep, destination %d: predicted iteration %.6f ms, oracle %.6f ms, "
              "relative difference %.3g (bound 1e-05: wave-scaled passes 1e-6, fp32 MLP "
              "operations 1e-4 each)" % (di, totals[di], total, abs(totals[di] - total) / total))
    # faster devices predict shorter iterations, on the whole: rank correlation
    # between memory bandwidth and predicted time is clearly negative
    bw = np.array([d.mem_bandwidth_gb for d in devices], float)
    rank = lambda v: np.argsort(np.argsort(v))
    assert np.corrcoef(rank(bw), rank(totals))[0, 1] < -0.3


def _sweep_fixture(n_devices):
    origin = Device.V100
    trace = synthetic.resnet50_trace(origin, batch=32, seed=3)
    preds = {}
    for kind in ("conv2d", "linear"):
        torch.manual_seed(0)
        rp = RuntimePredictor(kind, 8, 1024)
        x, mu, sigma = synthetic.mlp_features(kind, 2048, seed=2)
        rp.set_normalization(mu, sigma)
        preds[kind] = rp
    predictor = Predictor(mlp_predictors=preds)
    devices, feats = synthetic.device_sweep(n_devices, seed=1)
    device_features = {d.name: list(f) for d, f in zip(devices, feats)}
    device_features[origin.name] = [16, 900, 80, 14.028]
    return predictor, trace, devices, device_features


def test_plan_reuse_and_subsets_agree_with_one_shot_sweep():
    predictor, trace, devices, feats = _sweep_fixture(24)
    whole = predictor.predict_trace_sweep(trace, devices, feats).total_ms.cpu().numpy()
    plan = predictor.plan_trace(trace)
    again = plan.run(devices, feats).total_ms.cpu().numpy()
    np.testing.assert_array_equal(whole, again)
    part = plan.run(devices[5:9], feats).total_ms.cpu().numpy()
    # a destination's total does not depend on which others share the launch,
    # up to fp32 rounding in the MLP part: few rows take one launch per layer,
    # many the fused kernel, and the two sum in different orders
    np.testing.assert_allclose(part, whole[5:9], rtol=1e-6)


def test_prepared_sweep_replays_in_a_hip_graph():
    """The GPU work of a prepared sweep allocates through torch only and never
    synchronises, so it can be captured once and replayed; every replay, with
    eager work and synchronisations in between, gives the eager totals."""
    predictor, trace, devices, feats = _sweep_fixture(32)
    call = predictor.plan_trace(trace).prepare(devices, feats)
    eager = call.launch()
    torch.cuda.synchronize()
    want_total = eager.total_ms.clone()
    want_pass = eager.pass_kernel_ns.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):          # warm-up on the capture stream
            call.launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = call.launch()
    for replay in range(4):
        captured.total_ms.fill_(-1.0)
        captured.pass_kernel_ns.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        # order of the fp64 atomic adds within a pass differs between launches
        torch.testing.assert_close(captured.total_ms, want_total, rtol=1e-12, atol=0)
        torch.testing.assert_close(captured.pass_kernel_ns, want_pass, rtol=1e-12, atol=0)
        assert int(captured.bad_records.sum().item()) == 0
        # the program's own eager work between replays
        other = call.launch().total_ms
        torch.cuda.synchronize()
        torch.testing.assert_close(other, want_total, rtol=1e-12, atol=0)


def test_device_table_argument_checks():
    with pytest.raises(ValueError):
        DeviceTable(Device.V100, [])
    bad = DeviceProperties(name="z", **dict(Device.V100.as_dict(), base_clock_mhz=0))
    with pytest.raises(_lib.HabitatLibraryError) as e:
        DeviceTable(Device.V100, [Device.T4, bad])
    assert e.value.code == _lib.HBT_ESPEC
