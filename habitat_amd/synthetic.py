"""Seeded synthetic inputs for the benchmark configurations: kernel records,
device sweeps and MLP feature matrices.  Everything is generated with numpy on
the host so that the same seed gives the same data on every machine.
"""
import ctypes

import numpy as np

from habitat_amd import _lib
from habitat_amd.device import DeviceProperties

BLOCK_SIZES = np.array([64, 128, 256, 512, 1024], dtype=np.int32)


def _draw_records(rng, n):
    total_smem = rng.integers(0, 65536, size=n, endpoint=True).astype(np.int32)
    static = (total_smem // 2).astype(np.int32)
    rec = {
        "num_blocks": np.clip(np.floor(2.0 ** rng.uniform(0, 20, n)), 1, 2**20).astype(np.int32),
        "block_size": rng.choice(BLOCK_SIZES, size=n).astype(np.int32),
        "regs_per_thread": rng.integers(16, 255, size=n, endpoint=True).astype(np.int32),
        "static_smem": static,
        "dynamic_smem": (total_smem - static).astype(np.int32),
        "run_time_ns": np.floor(10.0 ** rng.uniform(3, 7, n)),
        "dram_read_bytes": np.floor(10.0 ** rng.uniform(3, 10, n)),
        "dram_write_bytes": np.floor(10.0 ** rng.uniform(3, 10, n)),
        "flop_sp_efficiency": 10.0 ** rng.uniform(-2, 2, n),
    }
    return rec


def host_occupancy(device, rec, model32=False):
    """Occupancy of every record on `device` (host loop inside the library).
    `model32` evaluates the kernel's 32-bit formulation instead."""
    n = rec["block_size"].shape[0]
    out = np.empty(n, np.int32)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    cols = [np.ascontiguousarray(rec[k], np.int32)
            for k in ("block_size", "dynamic_smem", "static_smem", "regs_per_thread")]
    fn = (_lib.lib().hbt_occupancy_host_model32_batch if model32
          else _lib.lib().hbt_occupancy_host_batch)
    rc = fn(ctypes.byref(device.spec), n, *[p(c) for c in cols], p(out))
    _lib.check(rc, "hbt_occupancy_host_batch")
    return out


def kernel_records(n, origin, seed=0, metrics_fraction=1.0):
    """n records that can have run on `origin` (occupancy >= 1 there).

    num_blocks log-uniform in [1, 2^20]; block size in {64..1024}; 16..255
    registers per thread; 0..64 KiB of shared memory split evenly into static
    and dynamic; time log-uniform 1 us..10 ms (integer ns); DRAM bytes
    log-uniform 1e3..1e10; FLOP efficiency log-uniform 0.01..100 %.  Draws that
    could not have launched on the origin are rejected and redrawn.  Returns
    (columns, stats) where stats counts accepted and rejected draws.
    """
    rng = np.random.default_rng(seed)
    parts, have, drawn = [], 0, 0
    while have < n:
        m = max(1024, int((n - have) * 2.0))
        rec = _draw_records(rng, m)
        keep = host_occupancy(origin, rec) >= 1
        drawn += m
        parts.append({k: v[keep] for k, v in rec.items()})
        have += int(keep.sum())
    rec = {k: np.concatenate([p[k] for p in parts])[:n] for k in parts[0]}
    accepted_total = sum(p["num_blocks"].shape[0] for p in parts)
    if metrics_fraction < 1.0:
        rec["has_metrics"] = (rng.random(n) < metrics_fraction).astype(np.uint8)
    stats = {"seed": seed, "drawn": drawn, "accepted": accepted_total,
             "rejected": drawn - accepted_total, "used": n}
    return rec, stats


def device_sweep(count=256, seed=1, base=None):
    """`count` destination devices: 40..304 SMs, 500..8000 GB/s, 1.0..2.4 GHz,
    peak = SMs * clock * 128 / 1000 GFLOP/s, other limits as `base` (a
    DeviceProperties, default V100).  Also returns the MLP device features
    [mem, mem_bw, num_sm, single] per device."""
    from habitat_amd import Device
    base = base if base is not None else Device.V100
    rng = np.random.default_rng(seed)
    sms = rng.integers(40, 304, size=count, endpoint=True)
    bw = rng.integers(500, 8000, size=count, endpoint=True)
    clk = rng.integers(1000, 2400, size=count, endpoint=True)
    mem = rng.integers(8, 288, size=count, endpoint=True)
    devices, feats = [], np.empty((count, 4), np.float64)
    for i in range(count):
        kw = base.as_dict()
        kw["num_sms"] = int(sms[i])
        kw["mem_bandwidth_gb"] = int(bw[i])
        kw["base_clock_mhz"] = int(clk[i])
        kw["peak_gflops_per_second"] = int(sms[i]) * int(clk[i]) * 128 // 1000
        devices.append(DeviceProperties(name="sweep%03d" % i, **kw))
        feats[i] = (mem[i], bw[i], sms[i], kw["peak_gflops_per_second"] / 1000.0)
    return devices, feats


# Operation features per MLP, in the order the networks expect them
# (analyzer/habitat/analysis/mlp/mlp.py:38,57,76-77,97).
MLP_FEATURES = {
    "conv2d": ["bias", "batch", "image_size", "in_channels", "out_channels", "kernel_size",
               "stride", "padding"],
    "linear": ["bias", "batch", "in_features", "out_features"],
    "bmm": ["batch", "left", "middle", "right"],
    "lstm": ["bias", "bidirectional", "batch", "seq_len", "input_size", "hidden_size",
             "num_layers"],
}


# The six devices of the reference's MLP device table (analysis/mlp/devices.csv:2-7);
# a fixed list, so that seeded inputs do not depend on rows registered later.
REFERENCE_MLP_DEVICES = ("P100", "P4000", "RTX2070", "RTX2080Ti", "T4", "V100")


def mlp_features(kind, n, seed=2, device_features=None):
    """[n, F+4] float64 raw feature rows for one MLP kind: the operation
    features in MLP_FEATURES order, then [mem, mem_bw, num_sm, single] of a
    device drawn per row from `device_features` ([D, 4]; default: the six
    devices of mlp/devices.py).  Also returns (mu, sigma) = column mean and
    population standard deviation, as the reference's dataset does
    (analyzer/habitat/analysis/mlp/dataset.py:16-17)."""
    from habitat_amd.analysis.mlp.devices import DEVICE_FEATURES
    rng = np.random.default_rng(seed)
    u = lambda lo, hi: rng.integers(lo, hi, size=n, endpoint=True).astype(np.float64)
    pick = lambda vals: rng.choice(np.array(vals, np.float64), size=n)
    if kind == "conv2d":
        cols = dict(bias=u(0, 1), batch=u(1, 128), image_size=u(7, 224), in_channels=u(3, 2048),
                    out_channels=u(3, 2048), kernel_size=pick([1, 3, 5, 7]), stride=pick([1, 2]),
                    padding=u(0, 3))
    elif kind == "linear":
        cols = dict(bias=u(0, 1), batch=u(1, 3500), in_features=u(1, 32768),
                    out_features=u(1, 32768))
    elif kind == "bmm":
        cols = dict(batch=u(1, 128), left=u(1, 1024), middle=u(1, 1024), right=u(1, 1024))
    elif kind == "lstm":
        cols = dict(bias=u(0, 1), bidirectional=u(0, 1), batch=u(1, 128), seq_len=u(1, 512),
                    input_size=u(64, 4096), hidden_size=u(64, 4096), num_layers=u(1, 4))
    else:
        raise KeyError(kind)
    if device_features is None:
        device_features = np.array([DEVICE_FEATURES[k] for k in REFERENCE_MLP_DEVICES],
                                   np.float64)
    dev = device_features[rng.integers(0, device_features.shape[0], size=n)]
    x = np.concatenate([np.stack([cols[f] for f in MLP_FEATURES[kind]], axis=1), dev], axis=1)
    mu = np.mean(x, axis=0)
    sigma = np.std(x, axis=0)
    return np.ascontiguousarray(x), mu, sigma


def resnet50_trace(origin, batch=32, seed=3, metrics_fraction=0.3):
    """A ResNet-50-shaped training-iteration trace measured on `origin`: 53
    conv2d and 1 linear operation (MLP-predicted), and the batch-norm, ReLU,
    pooling, residual-add, loss and optimizer operations around them
    (wave-scaled; forward and backward kernels).  Shapes follow the torchvision
    layer table; times and metrics are synthetic but consistent with the shapes.
    About 180 operations and 900 kernel records."""
    from habitat_amd.analysis.arguments import Arguments
    from habitat_amd.analysis.kernels import KernelInstance, MeasuredKernel
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    from habitat_amd.analysis.trace import Trace

    rng = np.random.default_rng(seed)
    bw = origin.mem_bandwidth_gb * 1e9
    peak = origin.peak_gflops_per_second * 1e9
    ops = []

    def kernel(name, elements, bytes_per_el=8.0, block=256, regs=None):
        nblocks = max(1, int(np.ceil(elements / (block * 4))))
        t_ns = max(1500, int(elements * bytes_per_el / (bw * rng.uniform(0.45, 0.8)) * 1e9))
        k = KernelInstance(name, nblocks, block, 0, int(rng.choice([0, 0, 0, 2048, 4096])),
                           int(regs if regs is not None else rng.integers(16, 48)), t_ns)
        metrics = []
        if rng.random() < metrics_fraction:
            rd = elements * bytes_per_el * rng.uniform(0.4, 0.6)
            m = KernelInstance(name, nblocks, block, 0, 0, k.metadata["registers_per_thread"], t_ns, [
                ("dram__bytes_read.sum", float(int(rd))),
                ("dram__bytes_write.sum", float(int(elements * bytes_per_el - rd))),
                ("smsp__sass_thread_inst_executed_ops_fadd_fmul_ffma_pred_on.avg."
                 "pct_of_peak_sustained_elapsed", float(rng.uniform(0.5, 12.0)))])
            metrics = [m]
        return MeasuredKernel(k, metrics, origin)

    def scaled_op(name, elements, n_fwd, n_bwd):
        def one_pass(tag, count):
            ks = [kernel("%s_%s_%d" % (name, tag, i), elements) for i in range(count)]
            total_ms = sum(k.run_time_ns for k in ks) / 1e6 + rng.uniform(0.004, 0.02) * count
            return RunTimeMeasurement(total_ms, ks, origin)
        fwd = one_pass("fwd", n_fwd)
        bwd = one_pass("bwd", n_bwd) if n_bwd else None
        ops.append(MeasuredOperation(name, Arguments((), {}), fwd, bwd, origin))

    def conv(cin, cout, k, stride, hw_in, bias=False):
        pad = k // 2
        hw_out = (hw_in + 2 * pad - k) // stride + 1
        flops = 2.0 * batch * cout * hw_out * hw_out * cin * k * k
        fwd_ms = flops / (peak * rng.uniform(0.35, 0.7)) * 1e3 + 0.02
        args = ((batch, cin, hw_in, hw_in), (cout, cin, k, k), (cout,) if bias else None,
                (stride, stride), (pad, pad), (1, 1), 1)
        ops.append(MeasuredOperation(
            "conv2d", Arguments(args, {}), RunTimeMeasurement(fwd_ms, [], origin),
            RunTimeMeasurement(2.1 * fwd_ms, [], origin), origin))
        return hw_out

    def bn_relu(c, hw, relu=True):
        el = batch * c * hw * hw
        scaled_op("batch_norm", el, 3, 5)
        if relu:
            scaled_op("relu_", el, 1, 1)

    hw = conv(3, 64, 7, 2, 224)
    bn_relu(64, hw)
    scaled_op("max_pool2d", batch * 64 * hw * hw, 1, 1)
    hw = (hw + 2 - 3) // 2 + 1
    cin = 64
    for stage, (blocks, width) in enumerate(zip([3, 4, 6, 3], [64, 128, 256, 512])):
        for b in range(blocks):
            stride = 2 if (b == 0 and stage > 0) else 1
            conv(cin, width, 1, 1, hw)
            bn_relu(width, hw)
            hw2 = conv(width, width, 3, stride, hw)
            bn_relu(width, hw2)
            conv(width, width * 4, 1, 1, hw2)
            bn_relu(width * 4, hw2, relu=False)
            if b == 0:
                conv(cin, width * 4, 1, stride, hw)
                bn_relu(width * 4, hw2, relu=False)
            el = batch * width * 4 * hw2 * hw2
            scaled_op("add_", el, 1, 2)
            scaled_op("relu_", el, 1, 1)
            cin, hw = width * 4, hw2
    scaled_op("adaptive_avg_pool2d", batch * cin * hw * hw, 1, 1)
    fwd_ms = 2.0 * batch * 2048 * 1000 / (peak * 0.5) * 1e3 + 0.02
    ops.append(MeasuredOperation(
        "linear", Arguments(((batch, 2048), (1000, 2048), (1000,)), {}),
        RunTimeMeasurement(fwd_ms, [], origin), RunTimeMeasurement(2 * fwd_ms, [], origin), origin))
    scaled_op("log_softmax", batch * 1000, 1, 1)
    scaled_op("nll_loss", batch * 1000, 1, 1)
    # optimizer step: two small kernels per parameter tensor, no backward pass
    step = [kernel("sgd_%d" % i, int(rng.integers(64, 2_400_000)), 12.0) for i in range(322)]
    ops.append(MeasuredOperation(
        "_foreach_add_", Arguments((), {}),
        RunTimeMeasurement(sum(k.run_time_ns for k in step) / 1e6 * 1.1, step, origin), None,
        origin))
    return Trace(origin, ops)
