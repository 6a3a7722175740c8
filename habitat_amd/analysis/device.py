"""`habitat.analysis.device` (analyzer/habitat/analysis/device.py:5-24): the
lazily loaded device table.  The implementation lives in habitat_amd.device."""
from habitat_amd.device import _Device  # noqa: F401
