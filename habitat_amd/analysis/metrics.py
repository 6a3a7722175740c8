"""Kernel metrics the wave-scaling strategies read, with the two CUPTI spellings
the reference's recordings use (analyzer/habitat/analysis/metrics.py:29-88)."""
from enum import Enum


class _MetricInfo:
    def __init__(self, cupti_name, legacy_cupti_name, legacy_to_canonical_fn):
        self._cupti_name = cupti_name
        self._legacy_cupti_name = legacy_cupti_name
        self._legacy_to_canonical_fn = legacy_to_canonical_fn

    @property
    def cupti_name(self):
        return self._cupti_name

    @property
    def legacy_cupti_name(self):
        return self._legacy_cupti_name

    def to_canonical_value(self, value, device):
        # Values recorded on compute capability >= 7 are already canonical.
        if device.compute_capability[0] >= 7:
            return value
        return self._legacy_to_canonical_fn(value)


def _same(value):
    return value


class Metric(Enum):
    DRAMUtilization = _MetricInfo(
        "dram__throughput.avg.pct_of_peak_sustained_elapsed", "dram_utilization",
        lambda value: value * 10)
    DRAMReadBytes = _MetricInfo("dram__bytes_read.sum", "dram_read_bytes", _same)
    DRAMWriteBytes = _MetricInfo("dram__bytes_write.sum", "dram_write_bytes", _same)
    SinglePrecisionFLOPEfficiency = _MetricInfo(
        "smsp__sass_thread_inst_executed_ops_fadd_fmul_ffma_pred_on.avg."
        "pct_of_peak_sustained_elapsed", "flop_sp_efficiency", _same)
    SinglePrecisionAddOps = _MetricInfo(
        "smsp__sass_thread_inst_executed_op_fadd_pred_on.sum", "flop_count_sp_add", _same)


def _get_metric_name(metric, device):
    if isinstance(metric, Metric):
        info = metric.value
        return info.cupti_name if device.compute_capability[0] >= 7 else info.legacy_cupti_name
    return metric


def resolve_metrics(metrics, device):
    """Metric enum values -> raw metric names for `device`; raw names pass through."""
    if metrics is None:
        return []
    if isinstance(metrics, (list, tuple)):
        return [_get_metric_name(m, device) for m in metrics]
    return [_get_metric_name(metrics, device)]
