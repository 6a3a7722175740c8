"""Bandwidth-ratio wave scaling for kernels without metrics
(analyzer/habitat/analysis/wave_scaling/resimplified.py:7-40), on the GPU."""
from habitat_amd.analysis.wave_scaling.scalar import scale_one


def resimplified_wave_scaling(kernel, origin_device, dest_device, metadata_manager):
    return scale_one(kernel, origin_device, dest_device, metadata_manager, None)
