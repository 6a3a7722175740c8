"""One-kernel wrappers around the batched HIP path.

The reference's strategies take one kernel object and return one
PredictedKernel; here that is a batch of one record.  The status the kernel
writes is turned back into the exception the reference raises at that point.
"""
import torch

from habitat_amd import _lib
from habitat_amd.analysis.kernels import PredictedKernel
from habitat_amd.analysis.metrics import Metric
from habitat_amd.analysis.wave_scaling.batch import KernelRecords, wave_scale

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


def scale_one(kernel, origin_device, dest_device, metadata_manager, metrics, lookup_device=None):
    """metrics: (eff, rd, wr) for the roofline strategy, None for the
    no-metrics strategy.  `lookup_device`: the device the register table is
    asked about when that is not `dest_device` itself.  Returns a PredictedKernel."""
    nb, block, dyn, stat, regs, t_ns = kernel_fields(kernel)
    dest_regs = metadata_manager.kernel_registers_for(kernel, lookup_device or dest_device)
    dev = torch.device("cuda", torch.cuda.current_device())
    i32 = lambda v: torch.tensor([v], dtype=torch.int32, device=dev)
    f64 = lambda v: torch.tensor([v], dtype=torch.float64, device=dev)
    eff, rd, wr = metrics if metrics is not None else (0.0, 0.0, 0.0)
    records = KernelRecords(
        {"num_blocks": i32(nb), "block_size": i32(block), "dynamic_smem": i32(dyn),
         "static_smem": i32(stat), "regs_per_thread": i32(regs), "run_time_ns": f64(t_ns),
         "flop_sp_efficiency": f64(eff), "dram_read_bytes": f64(rd), "dram_write_bytes": f64(wr)},
        dest_regs=None if dest_regs is None else i32(dest_regs),
        has_metrics=torch.tensor([1 if metrics is not None else 0], dtype=torch.uint8,
                                 device=dev))
    out = wave_scale(records, origin_device, [dest_device], waves=False)
    status = int(out.status[0, 0].item())
    raise_for_status(status)
    value = float(out.time_ns[0, 0].item())
    if metrics is None and value == t_ns:
        value = kernel.run_time_ns  # the small-kernel branch returns the measured value as is
    return PredictedKernel(kernel, value)
