"""Device descriptions: `DeviceProperties` and the lazily loaded `Device` table.

`DeviceProperties` takes the fifteen constructor arguments of the reference's
pybind class (cpp/src/frontend/model_bindings.cpp:17-55, fields
cpp/src/cuda/kernel.h:14-62) and exposes the same six read-only properties.
`Device.<NAME>` behaves like the reference's singleton
(analyzer/habitat/analysis/device.py:5-24), reading data/devices.yml on first
use.
"""
import ctypes

from habitat_amd import _lib

_FIELDS = (
    "compute_major", "compute_minor", "max_threads_per_block",
    "max_threads_per_multiprocessor", "regs_per_block", "regs_per_multiprocessor",
    "warp_size", "shared_mem_per_block", "shared_mem_per_multiprocessor", "num_sms",
    "shared_mem_per_block_optin", "mem_bandwidth_gb", "base_clock_mhz",
    "peak_gflops_per_second",
)
# The reference stores these as size_t: a negative value is a TypeError there.
_UNSIGNED = ("shared_mem_per_block", "shared_mem_per_multiprocessor",
             "shared_mem_per_block_optin", "base_clock_mhz", "peak_gflops_per_second")


class DeviceProperties:
    __slots__ = ("_name", "_v", "_spec")

    def __init__(self, name, compute_major, compute_minor, max_threads_per_block,
                 max_threads_per_multiprocessor, regs_per_block, regs_per_multiprocessor,
                 warp_size, shared_mem_per_block, shared_mem_per_multiprocessor, num_sms,
                 shared_mem_per_block_optin, mem_bandwidth_gb, base_clock_mhz,
                 peak_gflops_per_second):
        if not isinstance(name, str):
            raise TypeError("name must be a str")
        values = (compute_major, compute_minor, max_threads_per_block,
                  max_threads_per_multiprocessor, regs_per_block, regs_per_multiprocessor,
                  warp_size, shared_mem_per_block, shared_mem_per_multiprocessor, num_sms,
                  shared_mem_per_block_optin, mem_bandwidth_gb, base_clock_mhz,
                  peak_gflops_per_second)
        v = {}
        for key, val in zip(_FIELDS, values):
            if isinstance(val, bool) or not isinstance(val, int):
                raise TypeError("%s must be an int, got %r" % (key, val))
            if key in _UNSIGNED and val < 0:
                raise TypeError("%s must be non-negative" % key)
            if key not in _UNSIGNED and not -2**31 <= val < 2**31:
                raise TypeError("%s does not fit a 32-bit int" % key)
            v[key] = val
        self._name = name
        self._v = v
        self._spec = None

    def __repr__(self):
        return "DeviceProperties(name=" + self._name + ")"

    @property
    def name(self):
        return self._name

    @property
    def num_sms(self):
        return self._v["num_sms"]

    @property
    def mem_bandwidth_gb(self):
        return self._v["mem_bandwidth_gb"]

    @property
    def compute_capability(self):
        return (self._v["compute_major"], self._v["compute_minor"])

    @property
    def base_clock_mhz(self):
        return self._v["base_clock_mhz"]

    @property
    def peak_gflops_per_second(self):
        return self._v["peak_gflops_per_second"]

    # -- additions used by this package -------------------------------------
    def as_dict(self):
        """The fourteen numeric constructor arguments."""
        return dict(self._v)

    @property
    def spec(self):
        """The `hbt_device_spec` handed to the C ABI."""
        if self._spec is None:
            v = self._v
            s = _lib.DeviceSpec()
            s.compute_major, s.compute_minor = v["compute_major"], v["compute_minor"]
            s.max_threads_per_block = v["max_threads_per_block"]
            s.max_threads_per_sm = v["max_threads_per_multiprocessor"]
            s.regs_per_block, s.regs_per_sm = v["regs_per_block"], v["regs_per_multiprocessor"]
            s.warp_size, s.num_sms = v["warp_size"], v["num_sms"]
            # Values beyond int64 cannot occur in practice; clamp instead of wrapping.
            s.smem_per_block = min(v["shared_mem_per_block"], 2**62)
            s.smem_per_sm = min(v["shared_mem_per_multiprocessor"], 2**62)
            s.smem_per_block_optin = min(v["shared_mem_per_block_optin"], 2**62)
            s.mem_bandwidth_gb = float(v["mem_bandwidth_gb"])
            s.base_clock_mhz = float(v["base_clock_mhz"])
            s.peak_gflops = float(v["peak_gflops_per_second"])
            self._spec = s
        return self._spec

    def thread_block_occupancy(self, block_size, dynamic_shared_memory, static_shared_memory,
                               registers_per_thread):
        """Blocks per multiprocessor of one launch configuration on this device
        (host-side; the reference's KernelMetadata::threadBlockOccupancy,
        cpp/src/cuda/kernel.cpp:33-56)."""
        out = ctypes.c_uint32(0)
        rc = _lib.lib().hbt_occupancy_host(
            ctypes.byref(self.spec), block_size, dynamic_shared_memory, static_shared_memory,
            registers_per_thread & 0xFFFF, ctypes.byref(out))
        _lib.check(rc, "hbt_occupancy_host")
        return out.value


class _Device:
    """`Device.V100` etc.; the table is read on first attribute access."""

    def __init__(self):
        self._devices = None

    def __getattr__(self, device_name):
        if device_name.startswith("__"):
            raise AttributeError(device_name)
        if self._devices is None:
            self._load_devices()
        try:
            return self._devices[device_name]
        except KeyError:
            raise KeyError(device_name) from None

    def _load_devices(self):
        import yaml
        from habitat_amd.data import path_to_data
        with open(path_to_data("devices.yml")) as f:
            table = yaml.safe_load(f)
        # {columns: [...], devices: {name: row}}, a row being the values in column
        # order or a mapping; or the reference's layout, {name: mapping}
        columns = table.get("columns", _FIELDS) if "devices" in table else _FIELDS
        rows = table["devices"] if "devices" in table else table
        self._devices = {}
        for name, row in rows.items():
            props = row if isinstance(row, dict) else dict(zip(columns, row))
            self._devices[name] = DeviceProperties(name=name, **props)

    def names(self):
        if self._devices is None:
            self._load_devices()
        return list(self._devices)
