"""Kernel objects of the data model.

`KernelInstance` is the record a profiler produces for one kernel launch: the
Python face of the reference's C++ class (cpp/src/cuda/kernel.h:64-151,
bindings cpp/src/frontend/model_bindings.cpp:57-82).  `MeasuredKernel` and
`PredictedKernel` follow analyzer/habitat/analysis/kernels.py:3-44.
"""
import struct

from habitat_amd.analysis.metrics import Metric

# hbt_kernel_record (include/habitat_mi.h): num_blocks, block_size, dynamic_smem,
# static_smem, regs, dest_regs, has_metrics, reserved; run_time_ns,
# flop_sp_efficiency, dram_read_bytes, dram_write_bytes.
RECORD_STRUCT = struct.Struct("<8i4d")
_ROOFLINE_METRICS = (Metric.SinglePrecisionFLOPEfficiency, Metric.DRAMReadBytes,
                     Metric.DRAMWriteBytes)


def pack_record(kernel):
    """(64-byte hbt_kernel_record of `kernel` with dest_regs = -1, has_metrics)
    for any object with the reference's kernel interface."""
    fast = getattr(kernel, "launch_fields", None)
    if fast is not None:
        nb, block, dyn, stat, regs, t_ns = fast()
    else:
        md = kernel.metadata
        nb, block, dyn, stat, regs, t_ns = (
            kernel.num_blocks, md["block_size"], md["dynamic_shared_memory"],
            md["static_shared_memory"], md["registers_per_thread"], kernel.run_time_ns)
    try:
        eff, rd, wr = [kernel.get_metric(m) for m in _ROOFLINE_METRICS]
        has = 1
    except AttributeError:
        eff = rd = wr = 0.0
        has = 0
    return RECORD_STRUCT.pack(nb, block, dyn, stat, regs, -1, has, 0, t_ns, eff, rd, wr), has


class KernelInstance:
    def __init__(self, name, num_blocks, block_size, dynamic_shared_memory,
                 static_shared_memory, registers_per_thread, run_time_ns, metrics=None):
        self._name = name
        self._num_blocks = int(num_blocks)
        self._block_size = int(block_size)
        self._dynamic_shared_memory = int(dynamic_shared_memory)
        self._static_shared_memory = int(static_shared_memory)
        self._registers_per_thread = int(registers_per_thread) & 0xFFFF  # uint16_t
        self._run_time_ns = int(run_time_ns)
        self._metrics = list(metrics) if metrics is not None else []

    @property
    def name(self):
        return self._name

    @property
    def run_time_ns(self):
        return self._run_time_ns

    @property
    def num_blocks(self):
        return self._num_blocks

    @property
    def metrics(self):
        """[(raw metric name, value)]"""
        return self._metrics

    def add_metric(self, name, value):
        self._metrics.append((name, float(value)))

    @property
    def metadata(self):
        return {
            "name": self._name,
            "num_blocks": self._num_blocks,
            "block_size": self._block_size,
            "static_shared_memory": self._static_shared_memory,
            "dynamic_shared_memory": self._dynamic_shared_memory,
            "registers_per_thread": self._registers_per_thread,
        }

    def launch_fields(self):
        """(num_blocks, block_size, dynamic_smem, static_smem, regs, run_time_ns):
        what `metadata`, `num_blocks` and `run_time_ns` hold, without the dict."""
        return (self._num_blocks, self._block_size, self._dynamic_shared_memory,
                self._static_shared_memory, self._registers_per_thread, self._run_time_ns)

    def thread_block_occupancy(self, device, registers_per_thread=-1):
        """Blocks per multiprocessor on `device`; a negative register count
        means this kernel's own (model_bindings.cpp:75-82)."""
        regs = self._registers_per_thread if registers_per_thread < 0 else registers_per_thread
        return device.thread_block_occupancy(
            self._block_size, self._dynamic_shared_memory, self._static_shared_memory, regs)


class MeasuredKernel:
    def __init__(self, time_kernel, metrics_kernels, device):
        self._c = time_kernel
        self._metrics_kernels = metrics_kernels
        self._device = device
        self._cached_metrics = {}
        self._packed = None

    def get_metric(self, metric_info, default=None):
        if metric_info in self._cached_metrics:
            return self._cached_metrics[metric_info]
        info = metric_info.value
        for metric_kernel in self._metrics_kernels:
            for raw_name, raw_value in metric_kernel.metrics:
                if raw_name == info.cupti_name or raw_name == info.legacy_cupti_name:
                    value = info.to_canonical_value(raw_value, self._device)
                    self._cached_metrics[metric_info] = value
                    return value
        if default is None:
            raise AttributeError("Unknown metric: {}".format(metric_info.name))
        return default

    # the attributes read per kernel on the prediction path, without the detour
    # through __getattr__
    name = property(lambda self: self._c.name)
    run_time_ns = property(lambda self: self._c.run_time_ns)
    num_blocks = property(lambda self: self._c.num_blocks)

    def launch_fields(self):
        return self._c.launch_fields()

    def packed_record(self):
        """(this kernel as a 64-byte hbt_kernel_record with dest_regs = -1, whether
        it has the three roofline metrics).  Built on first use and kept: the
        launch fields cannot change through this interface and a metric, once
        read, is cached for good (`_cached_metrics`, as in the reference); only
        a kernel found WITHOUT its metrics is looked at again when raw metrics
        have been added to its metric kernels since."""
        packed = self._packed
        if packed is not None:
            if packed[1] or packed[2] == sum(len(k.metrics) for k in self._metrics_kernels):
                return packed
        record, has = pack_record(self)
        self._packed = packed = (record, has,
                                 sum(len(k.metrics) for k in self._metrics_kernels))
        return packed

    def __getattr__(self, name):
        # Everything else comes from the underlying kernel instance.
        if name == "_c":
            raise AttributeError(name)
        return getattr(self._c, name)


class PredictedKernel:
    __slots__ = ("_measured_kernel", "_run_time_ns")

    def __init__(self, measured_kernel, run_time_ns):
        self._measured_kernel = measured_kernel
        self._run_time_ns = run_time_ns

    @property
    def run_time_ns(self):
        return self._run_time_ns

    @property
    def name(self):
        return self._measured_kernel.name
