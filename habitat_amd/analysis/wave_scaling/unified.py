"""Roofline scaling when the kernel has its three metrics, else the
bandwidth-ratio strategy (analyzer/habitat/analysis/wave_scaling/unified.py:8-35)."""
from habitat_amd.analysis.wave_scaling.scalar import read_metrics, scale_one


def unified_wave_scaling(kernel, origin_device, dest_device, metadata_manager):
    try:
        metrics = read_metrics(kernel)
    except AttributeError:
        metrics = None
    return scale_one(kernel, origin_device, dest_device, metadata_manager, metrics)
