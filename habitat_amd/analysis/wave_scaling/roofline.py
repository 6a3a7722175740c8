"""Roofline wave scaling of one kernel
(analyzer/habitat/analysis/wave_scaling/roofline.py:8-65), on the GPU."""
from habitat_amd.analysis.wave_scaling.scalar import read_metrics, scale_one


def roofline_wave_scaling(kernel, origin_device, dest_device, metadata_manager):
    metrics = read_metrics(kernel)  # AttributeError when a metric is absent
    return scale_one(kernel, origin_device, dest_device, metadata_manager, metrics)
