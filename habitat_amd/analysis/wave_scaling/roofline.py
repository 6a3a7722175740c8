"""Roofline wave scaling of one kernel
(analyzer/habitat/analysis/wave_scaling/roofline.py:8-108), on the GPU."""
import math

import torch

from habitat_amd.analysis.wave_scaling import batch
from habitat_amd.analysis.wave_scaling.scalar import read_metrics, scale_one


def roofline_wave_scaling(kernel, origin_device, dest_device, metadata_manager):
    metrics = read_metrics(kernel)  # AttributeError when a metric is absent
    return scale_one(kernel, origin_device, dest_device, metadata_manager, metrics)


def _roofline_gamma(kernel, origin_device, dest_device):
    """The exponent that splits a kernel between the bandwidth ratio (gamma)
    and the clock / multiprocessor ratios (1 - gamma), roofline.py:68-104,
    from the kernel that also does the scaling (a batch of one record)."""
    eff, rd, wr = read_metrics(kernel)
    dev = torch.device("cuda", torch.cuda.current_device())
    f64 = lambda v: torch.tensor([v], dtype=torch.float64, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    records = batch.KernelRecords(
        {"num_blocks": zero, "block_size": zero, "dynamic_smem": zero, "static_smem": zero,
         "regs_per_thread": zero, "run_time_ns": f64(kernel.run_time_ns),
         "flop_sp_efficiency": f64(eff), "dram_read_bytes": f64(rd), "dram_write_bytes": f64(wr)})
    gamma = float(batch.roofline_gamma(records, origin_device, dest_device)[0].item())
    assert not math.isnan(gamma)      # roofline.py:103: assert gamma >= 0 and gamma <= 1
    return gamma


def _ridge_point(device):
    """GFLOP per GB at which the device's roofline bends (roofline.py:107-108)."""
    return device.peak_gflops_per_second / device.mem_bandwidth_gb
