"""Kernel metrics the wave-scaling strategies read.  Each has the name CUPTI
uses from compute capability 7.0 on and the name and unit of the older
spelling, as in the reference's recordings
(analyzer/habitat/analysis/metrics.py:29-88)."""
from enum import Enum


def _names_since_volta(device):
    return device.compute_capability[0] >= 7


class _MetricInfo:
    __slots__ = ("cupti_name", "legacy_cupti_name", "_legacy_scale")

    def __init__(self, cupti_name, legacy_cupti_name, legacy_scale=None):
        self.cupti_name = cupti_name
        self.legacy_cupti_name = legacy_cupti_name
        self._legacy_scale = legacy_scale    # canonical value = legacy value x this

    def to_canonical_value(self, value, device):
        if _names_since_volta(device) or self._legacy_scale is None:
            return value
        return value * self._legacy_scale


_PCT = ".pct_of_peak_sustained_elapsed"

Metric = Enum("Metric", {
    # the old DRAM utilisation is a level 0..10, the new one a percentage
    "DRAMUtilization": _MetricInfo("dram__throughput.avg" + _PCT, "dram_utilization", 10),
    "DRAMReadBytes": _MetricInfo("dram__bytes_read.sum", "dram_read_bytes"),
    "DRAMWriteBytes": _MetricInfo("dram__bytes_write.sum", "dram_write_bytes"),
    "SinglePrecisionFLOPEfficiency": _MetricInfo(
        "smsp__sass_thread_inst_executed_ops_fadd_fmul_ffma_pred_on.avg" + _PCT,
        "flop_sp_efficiency"),
    "SinglePrecisionAddOps": _MetricInfo(
        "smsp__sass_thread_inst_executed_op_fadd_pred_on.sum", "flop_count_sp_add"),
}, module=__name__)


def _get_metric_name(metric, device):
    if not isinstance(metric, Metric):
        return metric                        # already a raw name
    info = metric.value
    return info.cupti_name if _names_since_volta(device) else info.legacy_cupti_name


def resolve_metrics(metrics, device):
    """Raw metric names for `device` from Metric members (raw names pass
    through); one metric or a list or tuple of them; None gives []."""
    if metrics is None:
        return []
    if not isinstance(metrics, (list, tuple)):
        metrics = (metrics,)
    return [_get_metric_name(metric, device) for metric in metrics]
