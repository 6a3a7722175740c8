"""Wave scaling with AMD's own occupancy rules for AMD devices.

An additional strategy for `Predictor(wave_scaling_strategy=...)`; the
reference has no counterpart (its occupancy routine models NVIDIA compute
capabilities 3.x to 7.x only, cpp/src/cuda/cuda_occupancy.h:573-694, so an AMD
destination has to be dressed up as one of those).  It is
unified_wave_scaling (analyzer/habitat/analysis/wave_scaling/unified.py:8-35)
with every AMD device replaced by its compute-unit description before the
occupancies are taken: work-groups per CU limited by VGPRs per SIMD, wave
slots, work-group slots and LDS (include/habitat_mi.h, HBT_COMPUTE_MAJOR_CDNA).
NVIDIA devices keep the reference's model, so NVIDIA -> NVIDIA predictions are
those of unified_wave_scaling.
"""
from habitat_amd.analysis.wave_scaling.scalar import read_metrics, scale_one
from habitat_amd.analysis import Device
from habitat_amd.device import DeviceProperties

CDNA_MAJOR = 109   # HBT_COMPUTE_MAJOR_CDNA
_HIP_GFX9_MAJOR = 9


def native_description(device):
    """The compute-unit description of an AMD device, or `device` itself.

    Accepted forms: a description that already carries compute_major 109; one
    with the compute capability HIP reports for gfx9 GPUs (9.x, e.g. from
    `habitat_amd.device_info.local_device`), whose fields already have the
    compute-unit meaning; or a table device `X` for which data/devices.yml has
    an `X_cdna` entry (MI355X)."""
    major, minor = device.compute_capability
    if major == CDNA_MAJOR:
        return device
    if major == _HIP_GFX9_MAJOR:
        props = device.as_dict()
        props["compute_major"] = CDNA_MAJOR
        # hipDeviceProp_t counts the 256 architectural VGPRs per lane and SIMD;
        # gfx942 and gfx950 (9.4, 9.5) allocate from a unified file of 512
        if minor >= 4 and props["regs_per_multiprocessor"] == 4 * 256 * props["warp_size"]:
            props["regs_per_multiprocessor"] *= 2
        return DeviceProperties(name=device.name, **props)
    if device.name + "_cdna" in Device.names():
        return getattr(Device, device.name + "_cdna")
    return device


def cdna_wave_scaling(kernel, origin_device, dest_device, metadata_manager):
    try:
        metrics = read_metrics(kernel)
    except AttributeError:
        metrics = None
    return scale_one(kernel, native_description(origin_device), native_description(dest_device),
                     metadata_manager, metrics, lookup_device=dest_device)
