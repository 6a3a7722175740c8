"""habitat_amd — MI355X-native batched prediction behind Habitat's analysis API.

The compute lives in libhabitat_mi.so (hand-written HIP for gfx950, reached
through the C ABI of include/habitat_mi.h); this package is the host-side
mirror of the reference's `habitat.analysis` interface for that path.
"""
from habitat_amd.device import DeviceProperties, _Device

Device = _Device()

__version__ = "0.1.0"

__all__ = ["Device", "DeviceProperties"]
