"""GPU: the host-side mirror of the reference's analysis API — scalar
wave-scaling strategies with the reference's exceptions, the Predictor routing
and the trace-level sums — against the CPU oracle."""
import math

import numpy as np
import pytest
import torch

from conftest import oracle_device
from habitat_amd import Device, synthetic
from habitat_amd.analysis.kernels import KernelInstance, MeasuredKernel, PredictedKernel
from habitat_amd.analysis.metrics import Metric
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from habitat_amd.analysis.predictor import Predictor
from habitat_amd.analysis.trace import Trace
from habitat_amd.analysis.wave_scaling.metadata import NullMetadataManager
from habitat_amd.analysis.wave_scaling.resimplified import resimplified_wave_scaling
from habitat_amd.analysis.wave_scaling.roofline import roofline_wave_scaling
from habitat_amd.analysis.wave_scaling.unified import unified_wave_scaling
from oracle import mlp as omlp
from oracle import predictor as opred
from oracle import wave_scaling as ows

pytestmark = pytest.mark.gpu


def odev(d):
    return oracle_device(d.as_dict())


def make_kernel(device, num_blocks=4096, block=256, dyn=0, stat=0, regs=32, t_ns=1000000,
                metrics=(50.0, 1e8, 1e8), name="k"):
    k = KernelInstance(name, num_blocks, block, dyn, stat, regs, t_ns)
    mk = []
    if metrics is not None:
        eff, rd, wr = metrics
        mk = [KernelInstance(name, num_blocks, block, dyn, stat, regs, t_ns, [
            ("flop_sp_efficiency", eff), ("dram_read_bytes", rd), ("dram_write_bytes", wr)])]
    return MeasuredKernel(k, mk, device)


def as_record(kernel, metrics):
    md = kernel.metadata
    eff, rd, wr = metrics if metrics is not None else (0.0, 0.0, 0.0)
    return dict(num_blocks=kernel.num_blocks, block_size=md["block_size"],
                dynamic_smem=md["dynamic_shared_memory"], static_smem=md["static_shared_memory"],
                regs_per_thread=md["registers_per_thread"], run_time_ns=kernel.run_time_ns,
                flop_sp_efficiency=eff, dram_read_bytes=rd, dram_write_bytes=wr)


class TableManager:
    """A metadata manager backed by a dict, to exercise dest_regs."""

    def __init__(self, table):
        self.table = table

    def kernel_registers_for(self, kernel, device):
        return self.table.get((kernel.name, device.name))


def test_scalar_strategies_known_answers(kat):
    mm = NullMetadataManager()
    for row in kat["scaling"]:
        o, d = getattr(Device, row["origin"]), getattr(Device, row["dest"])
        over = row.get("record", {})
        metrics = (over.get("flop_sp_efficiency", 50.0), 1e8, 1e8)
        has_metrics = row.get("has_metrics", True)
        k = make_kernel(o, num_blocks=row["num_blocks"], metrics=metrics if has_metrics else None)
        manager = mm if "dest_regs" not in row else TableManager({("k", d.name): row["dest_regs"]})
        strategies = (unified_wave_scaling, roofline_wave_scaling) if has_metrics else (
            unified_wave_scaling, resimplified_wave_scaling)
        for strategy in strategies:
            p = strategy(k, o, d, manager)
            assert isinstance(p, PredictedKernel) and p.name == "k"
            assert p.run_time_ns == pytest.approx(row["time_ns"], rel=1e-6)
        if "occ_dest" in row:
            assert k.thread_block_occupancy(d, row.get("dest_regs", -1)) == row["occ_dest"]
    # no metrics: unified falls back, roofline raises AttributeError like the reference
    k = make_kernel(Device.V100, metrics=None)
    assert unified_wave_scaling(k, Device.V100, Device.P100, mm).run_time_ns == pytest.approx(
        1e6 * 739 / 501, rel=1e-12)
    assert resimplified_wave_scaling(k, Device.V100, Device.P100, mm).run_time_ns == pytest.approx(
        1e6 * 739 / 501, rel=1e-12)
    with pytest.raises(AttributeError, match="Unknown metric"):
        roofline_wave_scaling(k, Device.V100, Device.P100, mm)
    small = make_kernel(Device.V100, num_blocks=3, metrics=None)
    assert resimplified_wave_scaling(small, Device.V100, Device.P100, mm).run_time_ns == 1000000


def test_scalar_strategies_raise_what_the_reference_raises():
    mm = NullMetadataManager()
    v100, p100, mi = Device.V100, Device.P100, Device.MI355X
    with pytest.raises(ZeroDivisionError):      # origin cannot hold the block
        unified_wave_scaling(make_kernel(v100, 100, 1024, regs=255), v100, p100, mm)
    with pytest.raises(ZeroDivisionError):      # destination cannot, kernel small on origin
        unified_wave_scaling(make_kernel(mi, 10, dyn=60000), mi, v100, mm)
    big = unified_wave_scaling(make_kernel(mi, 1 << 16, dyn=60000), mi, v100, mm)
    assert big.run_time_ns > 0                  # short-circuit: no exception
    with pytest.raises(AssertionError):         # gamma > 1
        roofline_wave_scaling(make_kernel(v100, 100, metrics=(50.0, -3e8, 1e8)), v100, p100, mm)
    with pytest.raises(ZeroDivisionError):      # num_blocks == 0
        roofline_wave_scaling(make_kernel(v100, 0), v100, p100, mm)
    assert resimplified_wave_scaling(make_kernel(v100, 0, metrics=None), v100, p100,
                                     mm).run_time_ns == 1000000


def test_scalar_strategy_from_several_threads():
    """The one-kernel call shares a staging block per GPU inside the library
    and serialises its callers: four threads scaling different kernels at once
    each get their own kernel's answer."""
    import threading
    mm = NullMetadataManager()
    origin, dest = Device.V100, Device.T4
    kernels = [make_kernel(origin, num_blocks=64 + 997 * i, t_ns=1_000_000 + 12_345 * i,
                           metrics=(10.0 + i, 1e8, 2e8) if i % 3 else None) for i in range(64)]
    want = [unified_wave_scaling(k, origin, dest, mm).run_time_ns for k in kernels]
    assert len(set(want)) > 32
    got = [None] * len(kernels)
    errors = []

    def work(start):
        try:
            torch.cuda.set_device(0)
            for _ in range(5):
                for i in range(start, len(kernels), 4):
                    got[i] = unified_wave_scaling(kernels[i], origin, dest, mm).run_time_ns
        except Exception as exc:       # noqa: BLE001 - reported below
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert got == want


def test_scalar_strategy_uses_the_register_table():
    k = make_kernel(Device.V100, num_blocks=400, name="gemm")
    rec = as_record(k, (50.0, 1e8, 1e8))
    mm = TableManager({("gemm", "P100"): 128})
    got = unified_wave_scaling(k, Device.V100, Device.P100, mm).run_time_ns
    want = ows.unified(rec, odev(Device.V100), odev(Device.P100), dest_regs=128)
    assert got == pytest.approx(want, rel=1e-6)
    # with 128 registers the P100 wave is 112 blocks instead of 448: 400 blocks are no longer "small"
    other = unified_wave_scaling(k, Device.V100, Device.P100, NullMetadataManager()).run_time_ns
    assert other != pytest.approx(want, rel=1e-3)


def seeded_predictors():
    preds = {}
    for kind in ("conv2d", "linear", "bmm", "lstm"):
        torch.manual_seed(0)
        rp = RuntimePredictor(kind, 8, 1024)
        x, mu, sigma = synthetic.mlp_features(kind, 2048, seed=2)
        rp.set_normalization(mu, sigma)
        preds[kind] = rp
    return preds


def oracle_operation_ms(op, dest, preds):
    """Predicted time of one operation by the oracle modules."""
    from habitat_amd.analysis import predictor as P
    o, d = odev(op.device), odev(dest)
    if op.name in ("conv2d", "linear", "bmm", "lstm"):
        rp = preds[op.name]
        a = P._ARGUMENTS[op.name](op)
        feats = [a[x] for x in rp.model.features]
        from habitat_amd.analysis.mlp.devices import get_device_features
        rows = np.array([feats + get_device_features(dest.name, rp.device_params),
                         feats + get_device_features(op.device.name, rp.device_params)], np.float64)
        y = omlp.forward_fp64(rp.model.state_dict(), rows, rp.mu, rp.sigma)
        return opred.special_op_ms(op.run_time_ms, y[0], y[1])
    total = 0.0
    for rt in (op.forward, op.backward):
        if rt is None:
            continue
        pred = []
        for k in rt.kernels:
            try:
                m = tuple(k.get_metric(x) for x in (Metric.SinglePrecisionFLOPEfficiency,
                                                    Metric.DRAMReadBytes, Metric.DRAMWriteBytes))
            except AttributeError:
                m = None
            pred.append(ows.unified(as_record(k, m), o, d, has_metrics=m is not None))
        total += opred.wave_scaled_pass_ms(rt.run_time_ms, [k.run_time_ns for k in rt.kernels], pred)
    return total


def test_predictor_on_resnet50_shaped_trace():
    origin, dest = Device.V100, Device.T4
    trace = synthetic.resnet50_trace(origin, batch=16, seed=3)
    preds = seeded_predictors()
    predictor = Predictor(mlp_predictors=preds)
    predicted = trace.to_device(dest, predictor)
    assert isinstance(predicted, Trace) and predicted.device is dest
    assert len(predicted.operations) == len(trace.operations)
    want = [oracle_operation_ms(op, dest, preds) for op in trace.operations]
    got = [op.run_time_ms for op in predicted.operations]
    for op, g, w in zip(trace.operations, got, want):
        tol = 1e-4 if op.name in ("conv2d", "linear") else 1e-6
        assert g == pytest.approx(w, rel=tol), op.name
    assert predicted.run_time_ms == pytest.approx(opred.trace_ms(want), rel=1e-5)
    # one operation at a time gives the same numbers as the batched call (for
    # the MLP operations up to fp32 rounding: one row and fifty-four rows are
    # summed over K in different orders)
    for idx in (0, 1, 5, len(trace.operations) - 1):
        op = trace.operations[idx]
        single = predictor.predict_operation(op, dest)
        tol = 1e-6 if op.name in ("conv2d", "linear") else 1e-12
        assert single.run_time_ms == pytest.approx(got[idx], rel=tol)
    assert trace.to_device(origin, predictor) is trace
    with pytest.raises(RuntimeError):
        predicted.operations[0].to_device(origin, predictor)


def test_bmm_lstm_and_every_call_form_against_hand_listed_features():
    """A trace holding every case of tests/arguments_kat.py (conv2d with tuple,
    int and keyword arguments, linear with 2 to 4 input dimensions, bmm, lstm
    unpacked and packed) through Trace.to_device, Trace.to_devices and the
    reference's per-operation private scalers.  The expected value feeds the
    oracle the feature lists written by hand there and the device rows of
    analysis/mlp/devices.csv:6-7 typed here, not the package's extraction."""
    from arguments_kat import CASES, arguments_of
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    device_rows = {"V100": [16, 900, 80, 14.028], "T4": [16, 320, 40, 8.1],
                   "P100": [16, 732, 56, 9.3]}
    origin = Device.V100
    preds = seeded_predictors()
    predictor = Predictor(mlp_predictors=preds)
    ops = [MeasuredOperation(case[0], arguments_of(case),
                             RunTimeMeasurement(0.5 + 0.25 * i, [], origin), None, origin)
           for i, case in enumerate(CASES)]
    trace = Trace(origin, ops)

    def want_ms(i, dest):
        kind, feats = CASES[i][0], CASES[i][5]
        rp = preds[kind]
        rows = np.array([feats + device_rows[dest.name], feats + device_rows["V100"]], np.float64)
        y = omlp.forward_fp64(rp.model.state_dict(), rows, rp.mu, rp.sigma)
        return opred.special_op_ms(ops[i].run_time_ms, y[0], y[1]), tolerance_ms(i, y)

    def tolerance_ms(i, y):
        # each fp32 network output is within 1e-4 of max(|y|, 1e-3) (the MLP
        # tests' bar); the quotient of two of them carries both errors
        err = [1e-4 * max(abs(v), 1e-3) / abs(v) for v in y]
        return abs(ops[i].run_time_ms * y[0] / y[1]) * (err[0] + err[1]) * 1.01

    for dest in (Device.T4, Device.P100):
        predicted = trace.to_device(dest, predictor)
        want = [want_ms(i, dest) for i in range(len(CASES))]
        for case, op, (w, tol) in zip(CASES, predicted.operations, want):
            assert op.backward is None and op.device is dest
            assert abs(op.run_time_ms - w) <= tol, case[:2]
        assert abs(predicted.run_time_ms - opred.trace_ms([w for w, _ in want])) <= sum(
            t for _, t in want)
    # the device sweep extracts its rows through the same functions
    totals = trace.to_devices([Device.T4, Device.P100], predictor)
    for dest, total in zip((Device.T4, Device.P100), totals):
        want = [want_ms(i, dest) for i in range(len(CASES))]
        assert abs(total - opred.trace_ms([w for w, _ in want])) <= sum(t for _, t in want)
    # Exact networks make every feature position count: fc1 copies input j to
    # unit j, the hidden layers are identities, fc2 weighs operation feature j
    # with j + 2 and the SM count with 1000 (no normalisation), so a prediction
    # is the integer  sum (j + 2) f_j + 1000 num_sms  and a wrong, swapped or
    # shifted feature changes the quotient far beyond fp64 rounding.
    exact = {}
    for kind, rp in seeded_predictors().items():
        n_op = len(rp.model.features)
        with torch.no_grad():
            for prm in rp.model.parameters():
                prm.zero_()
            for j in range(n_op + 4):
                rp.model.fc1.weight[j, j] = 1.0
            for layer in list(rp.model.mlp.layers)[::2]:
                layer.weight.copy_(torch.eye(1024))
            for j in range(n_op):
                rp.model.fc2.weight[0, j] = float(j + 2)
            rp.model.fc2.weight[0, n_op + 2] = 1000.0
        rp.set_normalization(np.zeros(n_op + 4), np.ones(n_op + 4))
        exact[kind] = rp
    exact_predictor = Predictor(mlp_predictors=exact)
    sms = {"V100": 80, "T4": 40, "P100": 56}
    for dest in (Device.T4, Device.P100):
        predicted = trace.to_device(dest, exact_predictor)
        swept = exact_predictor.predict_trace_sweep(trace, [dest])
        for i, (case, op) in enumerate(zip(CASES, predicted.operations)):
            a = sum((j + 2) * f for j, f in enumerate(case[5]))
            want = ops[i].run_time_ms * (a + 1000 * sms[dest.name]) / (a + 1000 * sms["V100"])
            assert op.run_time_ms == pytest.approx(want, rel=1e-12), case[:2]
        assert float(swept.total_ms[0]) == pytest.approx(predicted.run_time_ms, rel=1e-12)
    # the reference's private per-operation scalers (predictor.py:150-283)
    scalers = {"conv2d": predictor._conv2d_scale, "linear": predictor._linear_scale,
               "bmm": predictor._bmm_scale, "lstm": predictor._lstm_scale}
    for i, case in enumerate(CASES):
        got = predictor._special_scale(ops[i], Device.T4, scalers[case[0]])
        w, tol = want_ms(i, Device.T4)
        assert abs(got.run_time_ms - w) <= tol, case[:2]


def test_changed_kernels_are_seen_without_clearing_the_record_cache():
    """The predictor keeps the GPU-resident record columns of the passes it has
    seen; a pass whose kernels changed since (a time edited in place, a kernel
    replaced, one appended) must be converted afresh, as the reference reads
    every kernel on every call (predictor.py:111-130)."""
    origin, dest = Device.V100, Device.T4
    ops = [o for o in synthetic.resnet50_trace(origin, batch=8, seed=9).operations
           if o.name not in ("conv2d", "linear")][:12]
    trace = Trace(origin, ops)
    predictor = Predictor(mlp_predictors={})

    def oracle_total():
        return opred.trace_ms([oracle_operation_ms(op, dest, {}) for op in ops])

    first = trace.to_device(dest, predictor).run_time_ms
    assert first == pytest.approx(oracle_total(), rel=1e-6)
    assert trace.to_device(dest, predictor).run_time_ms == first          # served from the cache
    # 1. a kernel's time edited in place (and its pass, so that the overhead stays)
    victim = ops[3].forward.kernels[0]
    victim._c._run_time_ns += 7_000_000
    ops[3].forward._run_time_ms += 7.0
    second = trace.to_device(dest, predictor).run_time_ms
    assert second == pytest.approx(oracle_total(), rel=1e-6) and second > first + 1.0
    # 2. a kernel replaced by one with another launch size
    old = ops[5].forward.kernels[0]
    ops[5].forward.kernels[0] = make_kernel(origin, num_blocks=old.num_blocks * 3 + 1,
                                            t_ns=old.run_time_ns, name="other")
    third = trace.to_device(dest, predictor).run_time_ms
    assert third == pytest.approx(oracle_total(), rel=1e-6)
    # 3. a kernel appended
    ops[7].forward.kernels.append(make_kernel(origin, num_blocks=12345, t_ns=2_500_000, name="more"))
    fourth = trace.to_device(dest, predictor).run_time_ms
    assert fourth == pytest.approx(oracle_total(), rel=1e-6) and fourth != third


def test_trace_to_device_keeps_each_operation_s_own_contract():
    """trace.py:46-49 maps operation.to_device over the operations: one measured
    on the destination already comes back as it is (operation.py:82-85), a
    predicted one refuses (operation.py:137)."""
    from habitat_amd.analysis.operation import MeasuredOperation
    origin, dest = Device.V100, Device.T4
    ops = [o for o in synthetic.resnet50_trace(origin, batch=8, seed=9).operations
           if o.name not in ("conv2d", "linear")][:6]
    at_home = [o for o in synthetic.resnet50_trace(dest, batch=8, seed=9).operations
               if o.name not in ("conv2d", "linear")][0]
    assert isinstance(at_home, MeasuredOperation) and at_home.device is dest
    predictor = Predictor(mlp_predictors={})
    mixed = Trace(origin, ops[:3] + [at_home] + ops[3:])
    out = mixed.to_device(dest, predictor)
    assert out.operations[3] is at_home
    for i in (0, 1, 2, 4, 5, 6):
        assert out.operations[i].device is dest and out.operations[i] is not mixed.operations[i]
        want = oracle_operation_ms(mixed.operations[i], dest, {})
        assert out.operations[i].run_time_ms == pytest.approx(want, rel=1e-6)
    # a predicted trace cannot be predicted from
    with pytest.raises(RuntimeError, match="predicted operation"):
        out.to_device(Device.P100, predictor)
    # ... but still answers for the device it is on
    assert out.to_device(dest, predictor) is out


def test_predictor_with_a_caller_supplied_strategy_and_pass_through_ops():
    from habitat_amd.analysis.arguments import Arguments
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    origin, dest = Device.V100, Device.P100
    calls = []

    def halve(kernel, origin_device, dest_device, metadata_manager):
        calls.append(kernel.name)
        return PredictedKernel(kernel, kernel.run_time_ns / 2)

    ks = [make_kernel(origin, name="a", t_ns=2000000), make_kernel(origin, name="b", t_ns=1000000)]
    op = MeasuredOperation("relu_", Arguments((), {}), RunTimeMeasurement(3.5, ks, origin), None, origin)
    gru = MeasuredOperation("gru", Arguments((), {}), RunTimeMeasurement(7.0, [], origin),
                            RunTimeMeasurement(9.0, [], origin), origin)
    p = Predictor(wave_scaling_strategy=halve)
    out = p.predict_operations([op, gru], dest)
    assert calls == ["a", "b"]
    assert out[0].run_time_ms == pytest.approx((0.5e6 + 1.5e6) / 1e6)   # overhead kept, kernels halved
    assert out[1].run_time_ms == 16.0                                     # no predictor: unscaled
    # kernels longer than the measured pass: overhead clamps at zero
    op2 = MeasuredOperation("relu_", Arguments((), {}), RunTimeMeasurement(1.0, ks, origin), None, origin)
    assert p.predict_operation(op2, dest).run_time_ms == pytest.approx(1.5)


def test_device_sweep_matches_per_device_prediction():
    origin = Device.V100
    trace = synthetic.resnet50_trace(origin, batch=8, seed=5)
    preds = seeded_predictors()
    predictor = Predictor(mlp_predictors=preds)
    devices, feats = synthetic.device_sweep(24, seed=1)
    from habitat_amd.analysis.mlp import devices as md
    before = dict(md.DEVICE_FEATURES)
    try:
        for d, f in zip(devices, feats):
            md.register_device(d.name, *f)
        totals = trace.to_devices(devices, predictor)
        assert len(totals) == 24
        for i in (0, 7, 23):
            want = trace.to_device(devices[i], predictor).run_time_ms
            # fp32 rounding in the MLP part: the sweep's 25 x 53 rows take the fused
            # kernel, one device's 2 x 53 rows one launch per layer
            assert totals[i] == pytest.approx(want, rel=1e-6)
        oracle_total = opred.trace_ms([oracle_operation_ms(op, devices[3], preds)
                                       for op in trace.operations])
        assert totals[3] == pytest.approx(oracle_total, rel=1e-5)
    finally:
        for d in devices:
            md.unregister_device(d.name)
        assert md.DEVICE_FEATURES == before


def test_odd_traces_through_both_interfaces():
    """Traces without operations, without kernels, without MLP-predicted
    operations, without wave-scaled ones or without backward passes: per device
    (`to_device`) and as a sweep (`to_devices`) give the same totals."""
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    origin = Device.V100
    ops = synthetic.resnet50_trace(origin, batch=32, seed=3).operations
    predictor = Predictor(mlp_predictors=seeded_predictors())
    scaled = [o for o in ops if o.name not in ("conv2d", "linear")]
    mlp = [o for o in ops if o.name in ("conv2d", "linear")]
    no_backward = [MeasuredOperation(o.name, o.arguments, o.forward, None, o.device)
                   for o in scaled[:7]]
    no_kernels = [MeasuredOperation("relu", scaled[0].arguments,
                                    RunTimeMeasurement(0.25, [], origin), None, origin)]
    dests = [Device.T4, Device.P100, Device.RTX2070]
    cases = {"empty": [], "wave-scaled only": scaled, "mlp only": mlp, "no backward": no_backward,
             "no kernels": no_kernels, "one operation": scaled[:1], "one mlp operation": mlp[:1],
             "mixed": scaled[:3] + mlp[:2] + no_kernels}
    for name, case in cases.items():
        trace = Trace(origin, list(case))
        one_by_one = [trace.to_device(d, predictor).run_time_ms for d in dests]
        swept = trace.to_devices(dests, predictor)
        assert len(swept) == 3, name
        assert np.allclose(one_by_one, swept, rtol=1e-6, atol=1e-12), name
        if name == "empty":
            assert one_by_one == [0, 0, 0]
        if name == "no kernels":
            assert one_by_one == [0.25] * 3      # nothing to scale: the overhead alone
        if name == "no backward":
            want = opred.trace_ms([oracle_operation_ms(op, dests[0], {}) for op in case])
            assert one_by_one[0] == pytest.approx(want, rel=1e-6)


def test_local_device_description_and_measured_ceilings():
    from habitat_amd import device_info
    name, props = device_info.local_device(0)
    assert isinstance(name, str) and len(name) > 0
    assert props["warp_size"] == 64 and props["num_sms"] >= 1
    assert props["max_threads_per_block"] == 1024 and props["shared_mem_per_block"] >= 65536
    from habitat_amd import DeviceProperties
    dev = DeviceProperties(name="local", **props)        # the keys are DeviceProperties' own
    assert dev.num_sms == props["num_sms"]
    m = device_info.measure(iters=20000, copy_bytes=1 << 30)
    # an MI355X: several TB/s of copy bandwidth, tens of TFLOP/s of fp32
    assert m["copy_gbps"] > 500 and m["fp32_fma_gflops"] > 5000 and m["fp32_mfma_gflops"] > 20000
    assert m["fp32_mfma_gflops"] > m["fp32_fma_gflops"]
    # The three figures derived from the reported clocks (the table's
    # mem_bandwidth_gb, base_clock_mhz, peak_gflops_per_second), held against
    # what the box measures and what is published for the MI355X: the bandwidth
    # lies between the measured copy rate and the published 8 TB/s (8192 GB/s
    # by the clocks), the clock in 2.0-2.5 GHz, the vector fp32 peak at most 30 %
    # above the measured FMA rate (10 % on the boxes seen so far; the margin is
    # for one that runs below its clock) and at half the published 157.3
    # TFLOP/s, which counts packed fp32 or the matrix cores.
    assert m["copy_gbps"] < props["mem_bandwidth_gb"] <= 8000 * 1.03
    assert 2000 <= props["base_clock_mhz"] <= 2500
    assert m["fp32_fma_gflops"] <= props["peak_gflops_per_second"] <= 1.30 * m["fp32_fma_gflops"]
    assert props["peak_gflops_per_second"] == pytest.approx(157300 / 2, rel=0.02)
    assert m["fp32_mfma_gflops"] == pytest.approx(157300, rel=0.15)    # measured: 155 000
    # the data-movement yardsticks of wave scaling: one destination and seven
    one = device_info.record_stream_gbps(1_000_000, 200, 200)
    seven = device_info.record_stream_multi_gbps(1_000_000, 7, 100, 100)
    assert 3000 < seven < one < 8000 * 1.03
    from habitat_amd import _lib
    v = __import__("ctypes").c_double(0)
    assert _lib.lib().hbt_measure_record_stream_multi_gbps(1000, 0, 1, 1, v) == _lib.HBT_EINVAL
    # the reading as a compute-unit description: the GPU of the table's MI355X_cdna row
    from habitat_amd.analysis.wave_scaling.cdna import native_description
    native = native_description(dev).as_dict()
    table = Device.MI355X_cdna.as_dict()
    for key in ("compute_major", "compute_minor", "max_threads_per_block",
                "max_threads_per_multiprocessor", "regs_per_multiprocessor", "warp_size",
                "shared_mem_per_block", "shared_mem_per_multiprocessor", "num_sms",
                "base_clock_mhz"):
        assert native[key] == table[key], key
