"""One-kernel wrappers around the batched HIP path.

The reference's strategies take one kernel object and return one
PredictedKernel; here that is a batch of one record.  The status the kernel
writes is turned back into the exception the reference raises at that point.
"""
import ctypes
import threading

import numpy as np
import torch

from habitat_amd import _lib
from habitat_amd.analysis.kernels import PredictedKernel
from habitat_amd.analysis.metrics import Metric

_METRICS = (Metric.SinglePrecisionFLOPEfficiency, Metric.DRAMReadBytes, Metric.DRAMWriteBytes)


def kernel_fields(kernel):
    """(num_blocks, block_size, dynamic_smem, static_smem, regs, run_time_ns)."""
    fast = getattr(kernel, "launch_fields", None)   # this package's kernel classes
    if fast is not None:
        return fast()
    md = kernel.metadata
    return (kernel.num_blocks, md["block_size"], md["dynamic_shared_memory"],
            md["static_shared_memory"], md["registers_per_thread"], kernel.run_time_ns)


def read_metrics(kernel):
    """(flop efficiency, read bytes, written bytes); AttributeError if one is absent."""
    return tuple(kernel.get_metric(m) for m in _METRICS)


def raise_for_status(status):
    if status == _lib.ST_OK:
        return
    if status == _lib.ST_BAD_GAMMA:
        raise AssertionError("gamma outside [0, 1]")
    if status == _lib.ST_ZERO_BLOCKS:
        raise ZeroDivisionError("division by zero")
    raise ZeroDivisionError("integer division or modulo by zero")


class _Lane:
    """Staging memory of the one-kernel call, per thread and GPU: a pinned host
    record and its device twin, a device result and its pinned host twin.  One
    call is then one host-to-device copy (64 bytes), one launch and one
    device-to-host copy (24 bytes) on the current stream, and one wait.

    Record layout (bytes): 0 run_time_ns, 8 flop efficiency, 16 read bytes,
    24 written bytes (fp64); 32 num_blocks, 36 block_size, 40 dynamic_smem,
    44 static_smem, 48 regs, 52 dest_regs (int32); 56 has_metrics (uint8).
    Result: 0 time (fp64); 8 origin occupancy, 12 destination occupancy
    (int32); 16 status (uint8)."""

    def __init__(self, device):
        self.device = device
        self.host_in = torch.zeros(64, dtype=torch.uint8, pin_memory=True)
        self.host_out = torch.zeros(24, dtype=torch.uint8, pin_memory=True)
        self.dev_in = torch.zeros(64, dtype=torch.uint8, device=device)
        self.dev_out = torch.zeros(24, dtype=torch.uint8, device=device)
        raw_in, raw_out = self.host_in.numpy(), self.host_out.numpy()
        self.f64_in = raw_in[0:32].view(np.float64)
        self.i32_in = raw_in[32:56].view(np.int32)
        self.u8_in = raw_in[56:57]
        self.time_out = raw_out[0:8].view(np.float64)
        self.status_out = raw_out[16:17]
        base, out = self.dev_in.data_ptr(), self.dev_out.data_ptr()
        p = ctypes.c_void_p
        # hbt_wave_scale's column and output pointers, in its argument order
        self.columns = (p(base + 32), p(base + 36), p(base + 40), p(base + 44), p(base + 48),
                        p(base + 52), p(base), p(base + 8), p(base + 16), p(base + 24),
                        p(base + 56))
        self.outputs = (p(out), p(out + 8), p(out + 12), None, None, p(out + 16))


_lanes = threading.local()


def _lane():
    device = torch.cuda.current_device()
    lanes = getattr(_lanes, "by_device", None)
    if lanes is None:
        lanes = _lanes.by_device = {}
    if device not in lanes:
        lanes[device] = _Lane(torch.device("cuda", device))
    return lanes[device]


def scale_one(kernel, origin_device, dest_device, metadata_manager, metrics, lookup_device=None):
    """metrics: (eff, rd, wr) for the roofline strategy, None for the
    no-metrics strategy.  `lookup_device`: the device the register table is
    asked about when that is not `dest_device` itself.  Returns a PredictedKernel.

    This is the reference's own plug point, one kernel per call
    (predictor.py:116-124), and it pays a launch and two small copies for a few
    hundred arithmetic operations: tens of microseconds where the batched call
    spends a hundredth of a nanosecond per record.  Callers with many kernels
    should hand them over together (Predictor.predict_operations)."""
    nb, block, dyn, stat, regs, t_ns = kernel_fields(kernel)
    dest_regs = metadata_manager.kernel_registers_for(kernel, lookup_device or dest_device)
    lane = _lane()
    eff, rd, wr = metrics if metrics is not None else (0.0, 0.0, 0.0)
    lane.f64_in[:] = (t_ns, eff, rd, wr)
    lane.i32_in[:] = (nb, block, dyn, stat, regs, -1 if dest_regs is None else dest_regs)
    lane.u8_in[0] = 1 if metrics is not None else 0
    stream = torch.cuda.current_stream(lane.device)     # the copies go to the current stream too
    lane.dev_in.copy_(lane.host_in, non_blocking=True)
    rc = _lib.lib().hbt_wave_scale(
        ctypes.byref(origin_device.spec), ctypes.byref(dest_device.spec), 1, 1,
        *lane.columns, *lane.outputs, ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_wave_scale")
    lane.host_out.copy_(lane.dev_out, non_blocking=True)
    stream.synchronize()
    raise_for_status(int(lane.status_out[0]))
    value = float(lane.time_out[0])
    if metrics is None and value == t_ns:
        value = kernel.run_time_ns  # the small-kernel branch returns the measured value as is
    return PredictedKernel(kernel, value)
