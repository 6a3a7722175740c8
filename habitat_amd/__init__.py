"""habitat_amd — MI355X-native batched prediction behind Habitat's analysis API.

The compute lives in libhabitat_mi.so (hand-written HIP for gfx950, reached
through the C ABI of include/habitat_mi.h); this package is the host-side
mirror of the reference's `habitat.analysis` interface for that path
(analyzer/habitat/__init__.py:1-19 without the tracker).

    import habitat_amd as habitat
    trace.to_device(habitat.Device.MI355X)

`install_as_habitat()` registers the package under the name `habitat`, so that
code written against the reference (`import habitat.analysis.wave_scaling.unified`)
finds the same names.
"""
import importlib
import sys

from habitat_amd.analysis import Device
from habitat_amd.device import DeviceProperties

__version__ = "0.1.0"

_LAZY = {
    "Metric": ("habitat_amd.analysis.metrics", "Metric"),
    "Predictor": ("habitat_amd.analysis.predictor", "Predictor"),
    "Trace": ("habitat_amd.analysis.trace", "Trace"),
}

__all__ = ["Device", "DeviceProperties", "Metric", "Predictor", "Trace", "install_as_habitat"]


def __getattr__(name):
    # torch is only imported when prediction classes are first touched
    if name in _LAZY:
        module, attr = _LAZY[name]
        value = getattr(importlib.import_module(module), attr)
        globals()[name] = value
        return value
    if name == "OperationTracker":
        # analyzer/habitat/tracking/operation.py: measures operations with CUPTI on
        # an NVIDIA GPU; it produces this path's input and is not part of it
        raise AttributeError("habitat_amd has no OperationTracker: traces are measured with the "
                             "reference's tracker and handed over as habitat_amd.analysis objects")
    raise AttributeError("module 'habitat_amd' has no attribute %r" % name)


_SUBMODULES = [
    "analysis", "analysis.arguments", "analysis.device", "analysis.kernels", "analysis.metrics",
    "analysis.operation", "analysis.predictor", "analysis.run_time", "analysis.trace",
    "analysis.mlp", "analysis.mlp.devices", "analysis.mlp.mlp",
    "analysis.wave_scaling", "analysis.wave_scaling.common", "analysis.wave_scaling.metadata",
    "analysis.wave_scaling.resimplified", "analysis.wave_scaling.roofline",
    "analysis.wave_scaling.unified", "analysis.wave_scaling.batch", "analysis.wave_scaling.cdna",
    "analysis.wave_scaling.deferred", "analysis.wave_scaling.scalar",
    "analysis.report", "analysis.sweep", "data", "device", "utils",
]


def install_as_habitat():
    """Make `import habitat...` resolve to this package's modules."""
    sys.modules["habitat"] = sys.modules[__name__]
    for sub in _SUBMODULES:
        sys.modules["habitat." + sub] = importlib.import_module("habitat_amd." + sub)
    return sys.modules["habitat"]
