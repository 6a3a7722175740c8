"""One-kernel wrappers around the batched HIP path.

The reference's strategies take one kernel object and return one
PredictedKernel; here that is a batch of one record.  The status the kernel
writes is turned back into the exception the reference raises at that point.
"""
import ctypes
import threading

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


_state = threading.local()


def _call_state():
    """Per-thread ctypes objects of the one-kernel call, built once."""
    st = getattr(_state, "value", None)
    if st is None:
        record = _lib.KernelRecord()
        time_ns, status = ctypes.c_double(0.0), ctypes.c_uint8(0)
        st = _state.value = (record, time_ns, status, ctypes.byref(record),
                             ctypes.byref(time_ns), ctypes.byref(status))
    return st


def scale_one(kernel, origin_device, dest_device, metadata_manager, metrics, lookup_device=None):
    """metrics: (eff, rd, wr) for the roofline strategy, None for the
    no-metrics strategy.  `lookup_device`: the device the register table is
    asked about when that is not `dest_device` itself.  Returns a PredictedKernel.

    This is the reference's own plug point, one kernel per call
    (predictor.py:116-124): one hbt_wave_scale_one, i.e. one launch on a
    pinned, device-visible record and a wait, about ten microseconds for a few
    hundred arithmetic operations, where the batched call spends a hundredth of
    a nanosecond per record.  Callers with many kernels should hand them over
    together (Predictor.predict_operations), or keep this signature and use a
    deferred strategy (wave_scaling/deferred.py), which launches once per set
    of kernels."""
    nb, block, dyn, stat, regs, t_ns = kernel_fields(kernel)
    dest_regs = metadata_manager.kernel_registers_for(kernel, lookup_device or dest_device)
    record, time_ns, status, p_record, p_time, p_status = _call_state()
    record.num_blocks, record.block_size = nb, block
    record.dynamic_smem, record.static_smem, record.regs = dyn, stat, regs
    record.dest_regs = -1 if dest_regs is None else dest_regs
    record.run_time_ns = t_ns
    if metrics is not None:
        record.has_metrics = 1
        record.flop_sp_efficiency, record.dram_read_bytes, record.dram_write_bytes = metrics
    else:
        record.has_metrics = 0
        record.flop_sp_efficiency = record.dram_read_bytes = record.dram_write_bytes = 0.0
    stream = torch.cuda.current_stream()
    rc = _lib.lib().hbt_wave_scale_one(
        ctypes.byref(origin_device.spec), ctypes.byref(dest_device.spec), p_record, p_time, None,
        None, p_status, ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_wave_scale_one")
    raise_for_status(status.value)
    value = time_ns.value
    if metrics is None and value == t_ns:
        value = kernel.run_time_ns  # the small-kernel branch returns the measured value as is
    return PredictedKernel(kernel, value)
