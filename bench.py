#!/usr/bin/env python3
"""Benchmark of the batched-prediction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of wave scaling over the 1 M synthetic kernel records of
BASELINE.json's configs[1] (V100-like origin -> MI355X-like destination),
inputs resident in HBM.  Prints ONE JSON line:
  value         whole-job wave-scaled kernel records per second (K steps, wall clock)
  roofline      the wave-scaling kernel against HBM bandwidth: 68 algorithmic
                bytes per record / average launch duration (HIP events on the
                launch stream)
  cpu_baseline  the CPU oracle (C restatement of the reference's per-kernel
                Python, one thread) on the same records, same machine; under
                all_cores the same over every host core the box gives this job
  parity        untimed: the timed launch's outputs against the oracle (integer
                and status mismatches, largest relative time error), and the
                MLP against its fp64 evaluation on 4 096 rows
  multi_destination  the same records scaled to the seven other NVIDIA devices of the
                device table in one launch (records read once)
  large         the same kernel at 64 M records (beyond the 256 MB last-level cache);
                large_16M: at 16 M records
  mlp           the fused MFMA MLP (configs[2], conv2d, 1 M rows): rows/s, its
                roofline against fp32 MFMA peak and a torch-CPU fp32 baseline
  scalar_strategy  the reference's one-kernel strategy call through the same kernel
  host_records  the same records as an array of structures in HOST memory, results
                back in host memory, copies and wait included
  sweep         configs[4]: one ResNet-50-shaped trace predicted for 256 devices
                (fused per-pass sums + MLP rows + ratio kernel), eager and as a
                replayed HIP graph, next to the per-device CPU path
Only one GPU is used; --gpus above 1 exits.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published
BYTES_PER_RECORD = 68          # 5 x i32 + 4 x f64 read, f64 + 2 x i32 written
# Measured L2<->fabric bytes per record (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled
# on a copy kernel of known size; profiles/wave_scale_kernel_1M_and_64M_records.md):
# 52.07 read + 17.13 written (the status byte is the 69th).
TRAFFIC_BYTES_PER_RECORD = 69.20
MLP_TRAFFIC_BYTES_PER_ROW = 33040.0  # profiles/mlp_fused_kernel_conv2d_1M_rows.md: weights re-streamed per round


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # Defaults long enough to report the rate under continuous launches (some
    # kernel configurations run several per cent faster for the first
    # milliseconds after idle).
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=2000)
    ap.add_argument("--records", type=int, default=1_000_000)
    ap.add_argument("--large-records", type=int, default=64_000_000)
    ap.add_argument("--mlp-rows", type=int, default=1_000_000)
    ap.add_argument("--mlp-kind", default="conv2d")
    ap.add_argument("--mlp-steps", type=int, default=3)
    ap.add_argument("--no-mlp", action="store_true")
    ap.add_argument("--no-few-rows", action="store_true",
                    help="skip the MLP timings at 1 to 5911 rows (thousands of launches: "
                         "leave them out of a counter run on the fused kernel)")
    ap.add_argument("--no-large", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip configs[4] (one ResNet-50-shaped trace against 256 devices)")
    ap.add_argument("--sweep-devices", type=int, default=256)
    ap.add_argument("--no-ceilings", action="store_true",
                    help="skip measuring the box's own copy bandwidth and FMA/MFMA rates")
    ap.add_argument("--mlp-other-kinds", default="linear,bmm,lstm",
                    help="further MLP kinds timed with one step each (empty to skip)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy (for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return ap.parse_args()


class WaveScaleCall:
    """The C-ABI call with every argument converted once, so the timed loop
    measures the library and the GPU rather than Python argument handling."""

    def __init__(self, records, origin, dest, out):
        """`dest`: one device, or a list of them (outputs [n_dest][n])."""
        import torch
        from habitat_amd import _lib
        self.lib = _lib.lib()
        dests = dest if isinstance(dest, (list, tuple)) else [dest]
        specs = (_lib.DeviceSpec * len(dests))(*[d.spec for d in dests])
        self.keep = (records, out, origin, dests, specs)
        p = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
        c = records.columns
        self.stream = torch.cuda.current_stream()
        self.args = (
            ctypes.byref(origin.spec), specs, len(dests), records.n,
            p(c["num_blocks"]), p(c["block_size"]), p(c["dynamic_smem"]), p(c["static_smem"]),
            p(c["regs_per_thread"]), p(records.dest_regs), p(c["run_time_ns"]),
            p(c["flop_sp_efficiency"]), p(c["dram_read_bytes"]), p(c["dram_write_bytes"]),
            p(records.has_metrics), p(out.time_ns), p(out.occ_origin), p(out.occ_dest),
            p(out.wave_origin), p(out.wave_dest), p(out.status),
            ctypes.c_void_p(self.stream.cuda_stream))

    def __call__(self):
        rc = self.lib.hbt_wave_scale(*self.args)
        if rc != 0:
            raise RuntimeError("hbt_wave_scale failed: %d" % rc)


def time_steps(call, steps, warmup):
    """(wall ms per step, event ms per launch) over exactly `steps` calls."""
    import torch
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    # torch creates an event at its first record(): do that here, not inside
    # the timed region (two creations cost some 10 us: half a microsecond per
    # step of a 20-step run)
    e0.record()
    e1.record()
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        call()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, e0.elapsed_time(e1) / steps


def tile_records(rec, n):
    import numpy as np
    base = rec["num_blocks"].shape[0]
    reps = (n + base - 1) // base
    return {k: np.tile(v, reps)[:n] for k, v in rec.items()}


def mlp_bench(args):
    """configs[2] (and the other kinds of configs[3], one step each): the fused
    MLP at full size, the per-layer path (up to 7168 rows), and a torch CPU baseline."""
    import numpy as np
    import torch
    from habitat_amd import synthetic
    from habitat_amd.analysis.mlp.mlp import RuntimePredictor
    kind = args.mlp_kind
    torch.manual_seed(0)
    rp = RuntimePredictor(kind, 8, 1024)
    x, mu, sigma = synthetic.mlp_features(kind, args.mlp_rows, seed=2)
    rp.set_normalization(mu, sigma)
    xg = torch.from_numpy(x).cuda()
    yg = torch.empty(args.mlp_rows, dtype=torch.float32, device="cuda")
    f_in = x.shape[1]
    flops_per_row = 2.0 * (f_in * 1024 + 8 * 1024 * 1024 + 1024)
    mlp_call = lambda: rp.predict_batch(xg, out=yg)
    m_wall, m_launch = time_steps(mlp_call, args.mlp_steps, 1)
    tflops = flops_per_row * args.mlp_rows / (m_launch * 1e-3) / 1e12
    mlp = {"metric": "MLP op-predictions/s", "value": args.mlp_rows / (m_wall * 1e-3),
           "unit": "rows/s", "steps": args.mlp_steps, "ms_per_step": m_wall, "dtype": "f32",
           "config": {"workload": "configs[2]: %s MLP, %d rows x %d raw fp64 features, "
                                  "fc1 + 8 x 1024 hidden + fc2, seed-0 random init"
                                  % (kind, args.mlp_rows, f_in)},
           "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_FP32_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": tflops / MFMA_FP32_PEAK_TFLOPS,
                        "traffic": (MLP_TRAFFIC_BYTES_PER_ROW * args.mlp_rows
                                    if kind == "conv2d" else None),
                        "kernel": "mlp_fused_kernel<4>",
                        "launch_ms": m_launch, "flops_per_row": flops_per_row}}
    if not args.no_cpu:
        from oracle import mlp as omlp
        sd = rp.model.state_dict()
        m = min(32768, args.mlp_rows)
        threads = torch.get_num_threads()
        omlp.forward_fp32(sd, x[:1024], mu, sigma)
        t0 = time.perf_counter()
        omlp.forward_fp32(sd, x[:m], mu, sigma)
        dt = time.perf_counter() - t0
        mlp["cpu_baseline"] = {
            "value": m / dt, "unit": "rows/s", "cores": threads, "kind": "port",
            "sample": "oracle/mlp.py forward_fp32 (torch CPU fp32, one batched forward) on "
                      "the first %d rows, %d torch threads" % (m, threads)}
    # few rows: the reference's own call pattern is one row per call (mlp.py:252-267)
    if args.no_few_rows:
        return mlp
    few = {}
    for rows in (1, 48, 108, 512, 1536, 4096, 5911):
        xs = xg[:rows].contiguous()
        ys = torch.empty(rows, dtype=torch.float32, device="cuda")
        _, f_launch = time_steps(lambda: rp.predict_batch(xs, out=ys), 200, 50)
        few["rows_%d_us" % rows] = f_launch * 1e3
    # RuntimePredictor.predict as the reference calls it (mlp.py:252-267): what a
    # caller waits per call, wall clock, for arguments not asked before (one
    # hbt_mlp_predict_one: a row through pinned memory, ten launches, a wait) and
    # for arguments asked before (answered from the predictor's table)
    n_feat = len(rp.model.features)
    ops = [list(map(float, x[i, :n_feat])) for i in range(400)]
    for a_ in ops[:100]:
        rp.predict(a_, "V100")
    t0 = time.perf_counter()
    for a_ in ops[100:]:
        rp.predict(a_, "V100")
    few["predict_wall_us"] = (time.perf_counter() - t0) / 300 * 1e6
    t0 = time.perf_counter()
    for a_ in ops[100:]:
        rp.predict(a_, "V100")
    few["predict_again_wall_us"] = (time.perf_counter() - t0) / 300 * 1e6
    if not args.no_cpu:
        from oracle import mlp as omlp
        sd = rp.model.state_dict()
        omlp.forward_fp32(sd, x[:1], mu, sigma)
        t0 = time.perf_counter()
        for i in range(20):
            omlp.forward_fp32(sd, x[i:i + 1], mu, sigma)
        few["cpu_rows_1_us"] = (time.perf_counter() - t0) / 20 * 1e6
        # untimed: the MLP against the fp64 evaluation of the same weights
        m = min(4096, args.mlp_rows)
        y64 = omlp.forward_fp64(sd, x[:m], mu, sigma)
        worst = {}
        for rows in sorted({1, min(20, m), min(300, m), m}):
            y = rp.predict_batch(xg[:rows].contiguous()).cpu().numpy().astype("float64")
            worst["rows_%d" % rows] = float(
                (abs(y - y64[:rows]) / np.maximum(abs(y64[:rows]), 1e-3)).max())
        yf = yg[:m].cpu().numpy().astype("float64")      # the timed 1 M-row launch's own output
        worst["first_%d_of_the_timed_launch" % m] = float(
            (abs(yf - y64) / np.maximum(abs(y64), 1e-3)).max())
        mlp["parity"] = {"max_rel_error_vs_fp64": worst, "tolerance": 1e-4,
                         "floor_on_reference_magnitude": 1e-3,
                         "against": "oracle/mlp.py forward_fp64 on the first %d rows" % m}
    few["note"] = ("rows_N_us: GPU time of one forward (HIP events); up to 7168 rows one "
                   "launch per layer over the whole GPU (mlp_layer_kernel up to 128 rows, "
                   "mlp_layer_tile_kernel above); predict_wall_us: wall time of one "
                   "RuntimePredictor.predict call, predict_again_wall_us: of one with arguments "
                   "asked before; cpu_rows_1_us: torch CPU fp32, batch 1, as the reference "
                   "predicts")
    mlp["few_rows"] = few
    others = {}
    for other in [k for k in args.mlp_other_kinds.split(",") if k and k != kind]:
        torch.manual_seed(0)
        rpo = RuntimePredictor(other, 8, 1024)
        xo, muo, sgo = synthetic.mlp_features(other, args.mlp_rows, seed=2)
        rpo.set_normalization(muo, sgo)
        xog = torch.from_numpy(xo).cuda()
        _, o_launch = time_steps(lambda: rpo.predict_batch(xog, out=yg), 1, 1)
        fl = 2.0 * (xo.shape[1] * 1024 + 8 * 1024 * 1024 + 1024)
        tf = fl * args.mlp_rows / (o_launch * 1e-3) / 1e12
        others[other] = {"rows": args.mlp_rows, "launch_ms": o_launch,
                         "value": args.mlp_rows / (o_launch * 1e-3), "unit": "rows/s",
                         "achieved": tf, "frac": tf / MFMA_FP32_PEAK_TFLOPS}
        del rpo, xog
    if others:
        mlp["other_kinds"] = others
    return mlp


def sweep_bench(args, origin):
    """configs[4]: predicted iteration time of one trace on D devices."""
    import numpy as np
    import torch
    from habitat_amd import synthetic
    from habitat_amd.analysis import predictor as P
    from habitat_amd.analysis.mlp.mlp import RuntimePredictor
    from habitat_amd.analysis.predictor import Predictor
    D = args.sweep_devices
    trace = synthetic.resnet50_trace(origin, batch=32, seed=3)
    preds = {}
    for kind in ("conv2d", "linear"):
        torch.manual_seed(0)
        rp = RuntimePredictor(kind, 8, 1024)
        _, mu, sigma = synthetic.mlp_features(kind, 2048, seed=2)
        rp.set_normalization(mu, sigma)
        preds[kind] = rp
    predictor = Predictor(mlp_predictors=preds)
    devices, feats = synthetic.device_sweep(D, seed=1)
    device_features = {d.name: list(f) for d, f in zip(devices, feats)}
    device_features[origin.name] = [16, 900, 80, 14.028]

    t0 = time.perf_counter()
    plan = predictor.plan_trace(trace)
    call = plan.prepare(devices, device_features)
    torch.cuda.synchronize()
    prepare_ms = (time.perf_counter() - t0) * 1e3
    eager_wall, eager_gpu = time_steps(call.launch, 200, 50)
    totals = call.launch().total_ms
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call.launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = call.launch()
    graph_wall, graph_gpu = time_steps(graph.replay, 200, 50)
    torch.cuda.synchronize()
    same = bool(torch.allclose(captured.total_ms, totals, rtol=1e-12, atol=0))
    n_kernels = len(plan.kernels)
    n_special = sum(len(v[0]) for v in plan.special.values())
    out = {"workload": "configs[4]: ResNet-50-shaped trace (%d operations, %d kernel records in "
                       "%d passes, %d MLP-predicted operations), V100 origin, %d synthetic devices"
                       % (len(trace.operations), n_kernels, len(plan.pass_owner), n_special, D),
           "devices": D, "prepare_ms_once": prepare_ms,
           "eager": {"ms_per_sweep": eager_wall, "gpu_ms_per_sweep": eager_gpu,
                     "device_predictions_per_s": D / (eager_wall * 1e-3)},
           "hip_graph": {"ms_per_sweep": graph_wall, "gpu_ms_per_sweep": graph_gpu,
                         "device_predictions_per_s": D / (graph_wall * 1e-3),
                         "replay_equals_eager": same},
           "unit": "predicted (trace, device) pairs per second"}
    if not args.no_cpu:
        # the reference's shape of work on the host: per device, one Python call
        # chain per kernel and two batch-1 MLP forwards per special operation
        from habitat_amd.analysis.metrics import Metric
        from oracle import lib as olib
        from oracle import mlp as omlp
        from oracle import predictor as opred
        from oracle import wave_scaling as ows
        o = olib.make_device(**origin.as_dict())
        metrics = (Metric.SinglePrecisionFLOPEfficiency, Metric.DRAMReadBytes,
                   Metric.DRAMWriteBytes)
        sample = devices[:2]
        t0 = time.perf_counter()
        cpu_totals = []
        for dev in sample:
            d = olib.make_device(**dev.as_dict())
            total = 0.0
            for op in trace.operations:
                if op.name in preds:
                    rp = preds[op.name]
                    a = P._ARGUMENTS[op.name](op)
                    f = [a[x] for x in rp.model.features]
                    sd = rp.model.state_dict()
                    y_d = omlp.forward_fp32(sd, np.array([f + device_features[dev.name]]),
                                            rp.mu, rp.sigma)[0]
                    y_o = omlp.forward_fp32(sd, np.array([f + device_features[origin.name]]),
                                            rp.mu, rp.sigma)[0]
                    total += opred.special_op_ms(op.run_time_ms, float(y_d), float(y_o))
                    continue
                for rt in (op.forward, op.backward):
                    if rt is None:
                        continue
                    pk = []
                    for k in rt.kernels:
                        try:
                            m = tuple(k.get_metric(x) for x in metrics)
                        except AttributeError:
                            m = None
                        nb, block, dyn, stat, regs, t_ns = P.kernel_fields(k)
                        row = {"num_blocks": nb, "block_size": block, "dynamic_smem": dyn,
                               "static_smem": stat, "regs_per_thread": regs, "run_time_ns": t_ns,
                               "flop_sp_efficiency": m[0] if m else 0.0,
                               "dram_read_bytes": m[1] if m else 0.0,
                               "dram_write_bytes": m[2] if m else 0.0}
                        pk.append(ows.unified(row, o, d, has_metrics=m is not None))
                    total += opred.wave_scaled_pass_ms(rt.run_time_ms,
                                                       [k.run_time_ns for k in rt.kernels], pk)
            cpu_totals.append(total)
        dt = time.perf_counter() - t0
        got = totals[:len(sample)].cpu().numpy()
        out["cpu_baseline"] = {
            "value": len(sample) / dt, "unit": "predicted (trace, device) pairs per second",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "oracle (Python call chain per kernel, two batch-1 torch-CPU fp32 MLP "
                      "forwards per MLP-predicted operation, as the reference does) for the "
                      "first %d devices" % len(sample),
            "max_rel_diff_vs_gpu": float(np.max(np.abs(got - np.array(cpu_totals)) /
                                                np.abs(np.array(cpu_totals))))}
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported "
              "(records and rows are independent and would shard by contiguous ranges)"
              % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from habitat_amd import Device, synthetic
    from habitat_amd.analysis.wave_scaling.batch import KernelRecords, WaveScaleOutput

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    from habitat_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):    # run what is built; compile only when nothing is
        build.build()
    origin, dest = Device.V100, Device.MI355X

    if args.copy_calibration:
        src = torch.ones(1 << 27, dtype=torch.float64, device="cuda")   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    # ---------------- wave scaling, configs[1] ----------------
    rec, stats = synthetic.kernel_records(args.records, origin, seed=0)
    records = KernelRecords.from_numpy(rec)
    out = WaveScaleOutput(records.n, 1, records.device, waves=False, status=True)
    call = WaveScaleCall(records, origin, dest, out)
    # Exactly --warmup untimed and --steps timed launches, nothing before them.
    # (Earlier versions ran 2 000 untimed launches first; with this kernel a short
    # run reads no faster after them, rather a little slower: 11.4-11.8 us without,
    # 11.7-12.1 after 2 000, 11.8-13.0 after 20 000.)
    wall_ms, launch_ms = time_steps(call, args.steps, args.warmup)
    rec_per_s = args.records / (wall_ms * 1e-3)
    achieved = BYTES_PER_RECORD * args.records / (launch_ms * 1e-3) / 1e9
    result = {
        "metric": "wave-scaled kernel records/s (1 GPU); MLP op-predictions/s under 'mlp'",
        "value": rec_per_s, "unit": "records/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": "configs[1]: wave scaling, %d kernel records (SoA, int32 launch "
                               "params, fp64 times/metrics), V100 -> MI355X-like, outputs time + "
                               "2 occupancies + status" % args.records,
                   "records": args.records, "origin": origin.name, "dest": dest.name,
                   "seed": stats["seed"], "rejected_draws": stats["rejected"]},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     # the same bytes over the wall-clock step (launch overhead of the
                     # Python loop included): `value` x 68 B / peak
                     "frac_wall": BYTES_PER_RECORD * rec_per_s / 1e9 / HBM_PEAK_GBS,
                     # 68 MB fit the 256 MB last-level cache and the same buffers are
                     # read every step: this point is cache-resident.  The figure
                     # beyond the cache is copied here from `large` once measured.
                     "cache_resident": args.records * BYTES_PER_RECORD < 256e6,
                     "frac_beyond_cache": None,
                     "traffic": TRAFFIC_BYTES_PER_RECORD * args.records,
                     "traffic_source": "constant from profiles/wave_scale_kernel_1M_and_64M_"
                                       "records.md (rocprofv3 FETCH_SIZE + WRITE_SIZE per "
                                       "record, copy-calibrated), not measured in this run",
                     "kernel": "wave_scale_kernel<1, 1, true, unsigned int>", "launch_us": launch_ms * 1e3,
                     "bytes_per_record": BYTES_PER_RECORD},
    }
    if args.steps < 1000:
        # the rate a stream of batches sees: 2 000 launches after 2 000
        s_wall, s_launch = time_steps(call, 2000, 2000)
        result["sustained"] = {
            "steps": 2000, "warmup": 2000, "ms_per_step": s_wall, "launch_us": s_launch * 1e3,
            "frac": BYTES_PER_RECORD * args.records / (s_launch * 1e-3) / 1e9 / HBM_PEAK_GBS}

    def attempt(key, section):
        """A secondary section must not cost the headline line: on failure its
        entry says what went wrong."""
        try:
            value = section()
        except Exception as exc:   # noqa: BLE001 - reported, not swallowed
            value = {"error": "%s: %s" % (type(exc).__name__, exc)}
        if value is not None:
            result[key] = value

    # ---------------- parity of what was just timed (untimed) ----------------
    def parity_section():
        from oracle import lib as olib
        want = olib.wave_scale(olib.make_device(**origin.as_dict()),
                               olib.make_device(**dest.as_dict()), rec)
        torch.cuda.synchronize()
        t = out.time_ns[0].cpu().numpy()
        st = out.status[0].cpu().numpy()
        ok = want["status"] == 0
        rel = np.abs(t[ok] - want["time_ns"][ok]) / np.abs(want["time_ns"][ok])
        return {"records": args.records,
                "occupancy_mismatches": int((out.occ_origin.cpu().numpy() != want["occ_origin"]).sum()
                                            + (out.occ_dest[0].cpu().numpy() != want["occ_dest"]).sum()),
                "status_mismatches": int((st != want["status"]).sum()),
                "non_ok_records": int((~ok).sum()),
                "nan_where_not_ok": bool(np.all(np.isnan(t[~ok]))),
                "max_rel_time_error": float(rel.max()) if rel.size else 0.0,
                "tolerance": 1e-6,
                "against": "oracle/wave_scaling.c on the same %d records" % args.records}

    if not args.no_cpu:
        attempt("parity", parity_section)

    # ---------------- CPU baseline on the same records ----------------
    def cpu_section():
        from oracle import lib as olib
        from oracle import wave_scaling as ows
        o = olib.make_device(**origin.as_dict())
        d = olib.make_device(**dest.as_dict())
        olib.wave_scale(o, d, rec)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 400):
            olib.wave_scale(o, d, rec)
            reps += 1
        c_rate = reps * args.records / (time.perf_counter() - t0)
        # every core the box gives this job: contiguous slices of the records, one
        # per thread (the C call releases the interpreter lock)
        import concurrent.futures
        cores = max(1, min(int(os.environ.get("OMP_NUM_THREADS", "0")) or os.cpu_count(),
                           os.cpu_count()))
        bounds = np.linspace(0, args.records, cores + 1).astype(np.int64)
        slices = [{k: np.ascontiguousarray(v[a:b]) for k, v in rec.items()}
                  for a, b in zip(bounds[:-1], bounds[1:])]
        with concurrent.futures.ThreadPoolExecutor(cores) as pool:
            one_pass = lambda: list(pool.map(lambda part: olib.wave_scale(o, d, part), slices))
            one_pass()
            a_reps, t0 = 0, time.perf_counter()
            while a_reps < 3 or (time.perf_counter() - t0 < 5.0 and a_reps < 2000):
                one_pass()
                a_reps += 1
            all_rate = a_reps * args.records / (time.perf_counter() - t0)
        m = min(100_000, args.records)
        rows = [{k: v[i].item() for k, v in rec.items()} for i in range(m)]
        t0 = time.perf_counter()
        for row in rows:
            ows.unified(row, o, d)
        py_rate = m / (time.perf_counter() - t0)
        return {
            "value": c_rate, "unit": "records/s", "cores": 1, "kind": "port",
            "sample": "oracle/wave_scaling.c (per-record C restatement of the reference's "
                      "Python, libm pow) over the same %d records x %d passes, one thread of %d "
                      "host cores" % (args.records, reps, os.cpu_count()),
            "all_cores": {
                "value": all_rate, "unit": "records/s", "cores": cores, "kind": "port",
                "sample": "the same C restatement on %d threads, one contiguous slice of the "
                          "%d records each, %d passes" % (cores, args.records, a_reps)},
            "python_per_record": {
                "value": py_rate, "unit": "records/s", "cores": 1,
                "sample": "oracle/wave_scaling.py, one Python call chain per record as the "
                          "reference does, first %d records" % m}}

    if not args.no_cpu:
        attempt("cpu_baseline", cpu_section)

    # ---------------- the reference's plug point: one kernel per call ----------------
    def scalar_section():
        from habitat_amd.analysis.kernels import KernelInstance, MeasuredKernel
        from habitat_amd.analysis.wave_scaling.metadata import NullMetadataManager
        from habitat_amd.analysis.wave_scaling.unified import unified_wave_scaling
        m = 2000
        kernels = []
        for i in range(m):
            f = {k: v[i].item() for k, v in rec.items()}
            args_ = ("k", f["num_blocks"], f["block_size"], f["dynamic_smem"], f["static_smem"],
                     f["regs_per_thread"], int(f["run_time_ns"]))
            with_metrics = KernelInstance(*args_, [
                ("flop_sp_efficiency", f["flop_sp_efficiency"]),
                ("dram_read_bytes", f["dram_read_bytes"]),
                ("dram_write_bytes", f["dram_write_bytes"])])
            kernels.append(MeasuredKernel(KernelInstance(*args_), [with_metrics], origin))
        mm = NullMetadataManager()
        skipped = 0
        for k in kernels[:200]:
            try:
                unified_wave_scaling(k, origin, dest, mm)
            except ZeroDivisionError:
                pass
        t0 = time.perf_counter()
        for k in kernels:
            try:
                unified_wave_scaling(k, origin, dest, mm)
            except ZeroDivisionError:      # destination occupancy 0: the reference raises too
                skipped += 1
        dt = time.perf_counter() - t0
        # the same loop shape with the deferred strategy: note every kernel, then
        # read every time (the first read hands the whole set to the GPU)
        from habitat_amd.analysis.wave_scaling.deferred import deferred_unified_wave_scaling

        def deferred_pass(ks):
            t0 = time.perf_counter()
            preds = [deferred_unified_wave_scaling(k, origin, dest, mm) for k in ks]
            total, raised = 0.0, 0
            for p in preds:
                try:
                    total += p.run_time_ns
                except ZeroDivisionError:
                    raised += 1
            return (time.perf_counter() - t0) / len(ks) * 1e6, raised

        first_us, d_raised = deferred_pass(kernels)       # packs every kernel's record
        again_us = min(deferred_pass(kernels)[0] for _ in range(5))
        trace_sized_us = min(deferred_pass(kernels[:900])[0] for _ in range(5))
        return {"scalar_strategy_us_per_kernel": dt / m * 1e6, "kernels": m, "raised": skipped,
                "deferred_us_per_kernel": again_us,
                "deferred_us_per_kernel_900_kernels": trace_sized_us,
                "deferred_first_pass_us_per_kernel": first_us, "deferred_raised": d_raised,
                "what": "unified_wave_scaling(kernel, origin, dest, manager), the reference's "
                        "strategy signature (predictor.py:116-124): per call one "
                        "hbt_wave_scale_one, i.e. one launch on a pinned device-visible record "
                        "and a wait.  deferred_*: deferred_unified_wave_scaling in the same "
                        "loop, times read afterwards as run_time.py:50-58 does: one "
                        "hbt_wave_scale_host_records call for the whole set; first pass = "
                        "including the one-time packing of each kernel object's record"}

    attempt("scalar_strategy", scalar_section)

    # ---------------- records and results in HOST memory (PCIe inclusive) ----------------
    def host_records_section():
        import ctypes
        from habitat_amd.analysis.wave_scaling.deferred import RECORD_DTYPE
        host = np.zeros(args.records, RECORD_DTYPE)
        for src, dst in (("num_blocks", "num_blocks"), ("block_size", "block_size"),
                         ("dynamic_smem", "dynamic_smem"), ("static_smem", "static_smem"),
                         ("regs_per_thread", "regs"), ("run_time_ns", "run_time_ns"),
                         ("flop_sp_efficiency", "flop_sp_efficiency"),
                         ("dram_read_bytes", "dram_read_bytes"),
                         ("dram_write_bytes", "dram_write_bytes")):
            host[dst] = rec[src]
        host["dest_regs"], host["has_metrics"] = -1, 1
        t_ns, st = np.empty(args.records), np.empty(args.records, np.uint8)
        occ_o, occ_d = np.empty(args.records, np.int32), np.empty(args.records, np.int32)
        fn = _lib.lib().hbt_wave_scale_host_records
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

        def call(n):
            rc = fn(ctypes.byref(origin.spec), ctypes.byref(dest.spec), n,
                    ctypes.c_void_p(host.ctypes.data), ctypes.c_void_p(t_ns.ctypes.data),
                    ctypes.c_void_p(st.ctypes.data), ctypes.c_void_p(occ_o.ctypes.data),
                    ctypes.c_void_p(occ_d.ctypes.data), stream)
            if rc != 0:
                raise RuntimeError("hbt_wave_scale_host_records: %d" % rc)

        def rate(n, reps):
            call(n)
            best = float("inf")
            for _ in range(reps):
                t0 = time.perf_counter()
                call(n)
                best = min(best, time.perf_counter() - t0)
            return best
        small = rate(900, 200)
        whole = rate(args.records, 5)
        # the same records through the column kernel: results must be identical
        torch.cuda.synchronize()
        same = (np.array_equal(t_ns, out.time_ns[0].cpu().numpy(), equal_nan=True) and
                np.array_equal(occ_d, out.occ_dest[0].cpu().numpy()) and
                np.array_equal(occ_o, out.occ_origin.cpu().numpy()))
        return {"call_us_900_records": small * 1e6,
                "records_per_s_900": 900 / small,
                "records_per_s_%d" % args.records: args.records / whole,
                "GBps_host_in_plus_out": (64 + 17) * args.records / whole / 1e9,
                "equal_to_the_column_kernel": bool(same),
                "what": "hbt_wave_scale_host_records: 64-byte records in host memory in, "
                        "time + status + two occupancies in host memory out (17 bytes), "
                        "through the library's pinned staging block, host copies and the "
                        "wait included; best of 200 / 5 calls"}

    attempt("host_records", host_records_section)

    # ---------------- the same kernel beyond the last-level cache ----------------
    def large_section(n_records=None):
        big = KernelRecords.from_numpy(tile_records(rec, n_records or args.large_records))
        big_out = WaveScaleOutput(big.n, 1, big.device, waves=False, status=True)
        big_call = WaveScaleCall(big, origin, dest, big_out)
        # launch counts of this section's own, whatever --steps / --warmup say
        # (about 60 ms of launches at either size)
        steps = 80 if big.n > 32_000_000 else 300
        b_wall, b_launch = time_steps(big_call, steps, steps // 4)
        b_ach = BYTES_PER_RECORD * big.n / (b_launch * 1e-3) / 1e9
        return {"records": big.n, "steps": steps, "ms_per_step": b_wall,
                "value": big.n / (b_wall * 1e-3), "unit": "records/s",
                "roofline": {"bound": "hbm", "achieved": b_ach, "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": b_ach / HBM_PEAK_GBS,
                             "launch_us": b_launch * 1e3}}

    # ---------------- the same records for every other NVIDIA device of the table ------------
    def multi_dest_section():
        dests = [getattr(Device, name) for name in Device.names()
                 if name != origin.name and not name.startswith("MI355X")]
        m_out = WaveScaleOutput(records.n, len(dests), records.device, waves=False, status=True)
        m_call = WaveScaleCall(records, origin, dests, m_out)
        # launch counts of this section's own: a short run after a cold start
        # reads 60 % high (the kernel instantiation is loaded on first use)
        m_wall, m_launch = time_steps(m_call, 500, 200)
        # the record is read once and the origin occupancy written once per launch;
        # per destination: fp64 time + int32 occupancy + status byte
        per_record = 52 + 4 + 13 * len(dests)
        gbs = per_record * records.n / (m_launch * 1e-3) / 1e9
        return {"destinations": [d.name for d in dests], "launch_us": m_launch * 1e3,
                "us_per_destination": m_launch * 1e3 / len(dests),
                "value": records.n * len(dests) / (m_wall * 1e-3),
                "unit": "(record, destination) pairs/s",
                "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": gbs / HBM_PEAK_GBS, "bytes_per_record": per_record}}

    if not args.no_large:
        attempt("multi_destination", multi_dest_section)

    del call, records, out
    if not args.no_large and args.large_records > args.records:
        attempt("large", large_section)
        if "roofline" in result.get("large", {}):
            result["roofline"]["frac_beyond_cache"] = result["large"]["roofline"]["frac"]
            result["roofline"]["records_beyond_cache"] = result["large"]["records"]
        torch.cuda.empty_cache()
        # a size between the two: out of L2, within the last-level cache's reach
        if args.large_records > 16_000_000 > args.records:
            attempt("large_16M", lambda: large_section(16_000_000))
            torch.cuda.empty_cache()

    # ---------------- MLP, configs[2] ----------------
    if not args.no_mlp:
        attempt("mlp", lambda: mlp_bench(args))

    # ---------------- configs[4]: one trace, a sweep of destination devices ----------------
    if not args.no_sweep:
        attempt("sweep", lambda: sweep_bench(args, origin))

    # ---------------- what this box itself can do (ceilings under the published peaks) ----------
    def ceilings_section():
        from habitat_amd import device_info
        name, _ = device_info.local_device(0)
        m = device_info.measure()
        out = {"device": name, "copy_GBps_read_plus_write": m["copy_gbps"],
               "fp32_mfma_TFLOPs": m["fp32_mfma_gflops"] / 1e3,
               "fp32_vector_fma_TFLOPs": m["fp32_fma_gflops"] / 1e3}
        # yardstick for wave scaling: its loads and stores without the arithmetic
        out["record_stream_GBps_at_%d_records" % args.records] = device_info.record_stream_gbps(
            args.records, 500, 2000)
        out["record_stream_GBps_at_%d_records" % args.large_records] = (
            device_info.record_stream_gbps(args.large_records, 20, 40))
        # and for the launch with seven destinations (147 bytes per record)
        out["record_stream_GBps_seven_destinations_at_%d_records" % args.records] = (
            device_info.record_stream_multi_gbps(args.records, 7))
        # yardstick for the MLP: the vendor library's fp32 GEMM (+ bias) on one hidden
        # layer's shape, activations through HBM
        torch.backends.cuda.matmul.allow_tf32 = False
        rows = 262144
        a = torch.randn(rows, 1024, device="cuda")
        w = torch.randn(1024, 1024, device="cuda")
        b = torch.randn(1024, device="cuda")
        y = torch.empty(rows, 1024, device="cuda")
        _, g_ms = time_steps(lambda: torch.addmm(b, a, w.t(), out=y), 10, 3)
        out["vendor_fp32_gemm_one_layer_TFLOPs"] = 2.0 * rows * 1024 * 1024 / (g_ms * 1e-3) / 1e12
        return out

    if not args.no_ceilings:
        attempt("measured_ceilings", ceilings_section)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
