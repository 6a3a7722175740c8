"""ctypes binding of libhabitat_mi.so (the C ABI in include/habitat_mi.h).

The library is the only compute path: if it is missing this module raises, it
never falls back to CPU code.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libhabitat_mi.so")

ABI_VERSION = 103   # HBT_VERSION of include/habitat_mi.h this binding was written for

MLP_STATIC_MAX_ROWS = 1024   # HBT_MLP_STATIC_MAX_ROWS

HBT_OK, HBT_EINVAL, HBT_ESPEC, HBT_EHIP, HBT_ENOMEM, HBT_EALIGN, HBT_ESIZE = 0, -1, -2, -3, -4, -5, -6
ST_OK, ST_ORIGIN_WAVE_ZERO, ST_DEST_WAVE_ZERO, ST_BAD_GAMMA, ST_ZERO_BLOCKS = 0, 1, 2, 3, 4


class DeviceSpec(C.Structure):
    """hbt_device_spec."""
    _fields_ = [
        ("compute_major", C.c_int32), ("compute_minor", C.c_int32),
        ("max_threads_per_block", C.c_int32), ("max_threads_per_sm", C.c_int32),
        ("regs_per_block", C.c_int32), ("regs_per_sm", C.c_int32),
        ("warp_size", C.c_int32), ("num_sms", C.c_int32),
        ("smem_per_block", C.c_int64), ("smem_per_sm", C.c_int64),
        ("smem_per_block_optin", C.c_int64),
        ("mem_bandwidth_gb", C.c_double), ("base_clock_mhz", C.c_double),
        ("peak_gflops", C.c_double),
    ]


class KernelRecord(C.Structure):
    """hbt_kernel_record."""
    _fields_ = [
        ("num_blocks", C.c_int32), ("block_size", C.c_int32), ("dynamic_smem", C.c_int32),
        ("static_smem", C.c_int32), ("regs", C.c_int32), ("dest_regs", C.c_int32),
        ("has_metrics", C.c_int32), ("reserved", C.c_int32),
        ("run_time_ns", C.c_double), ("flop_sp_efficiency", C.c_double),
        ("dram_read_bytes", C.c_double), ("dram_write_bytes", C.c_double),
    ]


class HabitatLibraryError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s failed: %s (code %d)" % (what, strerror(code), code))


_lib = None

_P = C.c_void_p
_SIGNATURES = {
    "hbt_version": (C.c_int, []),
    "hbt_strerror": (C.c_char_p, [C.c_int]),
    "hbt_device_count": (C.c_int, []),
    "hbt_device_spec_check": (C.c_int, [C.POINTER(DeviceSpec)]),
    "hbt_occupancy_host": (C.c_int, [C.POINTER(DeviceSpec), C.c_int32, C.c_int32, C.c_int32,
                                     C.c_int32, C.POINTER(C.c_uint32)]),
    "hbt_occupancy_host_batch": (C.c_int, [C.POINTER(DeviceSpec), C.c_int64, _P, _P, _P, _P, _P]),
    "hbt_occupancy_host_model32_batch": (C.c_int, [C.POINTER(DeviceSpec), C.c_int64, _P, _P, _P, _P,
                                                   _P]),
    "hbt_wave_scale": (C.c_int, [C.POINTER(DeviceSpec), C.POINTER(DeviceSpec), C.c_int32,
                                 C.c_int64] + [_P] * 17 + [_P]),
    "hbt_wave_scale_one": (C.c_int, [C.POINTER(DeviceSpec), C.POINTER(DeviceSpec),
                                     C.POINTER(KernelRecord), C.POINTER(C.c_double),
                                     C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                     C.POINTER(C.c_uint8), _P]),
    "hbt_wave_scale_host_records": (C.c_int, [C.POINTER(DeviceSpec), C.POINTER(DeviceSpec),
                                              C.c_int64, _P, _P, _P, _P, _P, _P]),
    "hbt_device_table_create": (_P, [C.POINTER(DeviceSpec), C.POINTER(DeviceSpec), C.c_int32,
                                     C.POINTER(C.c_int)]),
    "hbt_device_table_size": (C.c_int32, [_P]),
    "hbt_device_table_destroy": (None, [_P]),
    "hbt_wave_scale_sum": (C.c_int, [_P, C.c_int64] + [_P] * 12 + [C.c_int32, _P, _P, _P]),
    "hbt_wave_scale_sum_ordered": (C.c_int, [_P, C.c_int64] + [_P] * 12 + [C.c_int32, _P, _P, _P,
                                                                            _P]),
    "hbt_roofline_gamma": (C.c_int, [C.POINTER(DeviceSpec), C.POINTER(DeviceSpec), C.c_int64,
                                     _P, _P, _P, _P, _P, _P]),
    "hbt_ratio_scale": (C.c_int, [_P, C.c_int32, C.c_int32, _P, C.c_int32, _P, _P, _P, _P, _P]),
    "hbt_mlp_create": (_P, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(_P), C.POINTER(_P), _P, _P,
                            C.POINTER(C.c_int)]),
    "hbt_mlp_forward": (C.c_int, [_P, _P, C.c_int64, _P, _P]),
    "hbt_mlp_destroy": (None, [_P]),
    "hbt_mlp_predict_one": (C.c_int, [_P, _P, C.POINTER(C.c_float), _P]),
    "hbt_mlp_forward_static": (C.c_int, [_P, _P, C.c_int64, _P, _P]),
    "hbt_local_device_spec": (C.c_int, [C.c_int, C.POINTER(DeviceSpec), C.c_char_p, C.c_size_t]),
    "hbt_measure_fp32_fma_gflops": (C.c_int, [C.c_int, C.POINTER(C.c_double)]),
    "hbt_measure_fp32_mfma_gflops": (C.c_int, [C.c_int, C.POINTER(C.c_double)]),
    "hbt_measure_copy_gbps": (C.c_int, [C.c_size_t, C.POINTER(C.c_double)]),
    "hbt_measure_record_stream_gbps": (C.c_int, [C.c_int64, C.c_int, C.c_int,
                                                 C.POINTER(C.c_double)]),
    "hbt_measure_record_stream_multi_gbps": (C.c_int, [C.c_int64, C.c_int32, C.c_int, C.c_int,
                                                       C.POINTER(C.c_double)]),
}

# Entry points added after the first release of the ABI; bound when present.
_OPTIONAL = {}


def exported_symbols():
    """Names include/habitat_mi.h declares."""
    return sorted(list(_SIGNATURES) + list(_OPTIONAL))


def lib():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "habitat_amd: %s is missing — build it with `python -m habitat_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        # The library and torch must share one HIP runtime: torch ships its own
        # libamdhip64, and whichever copy is loaded first serves both.  Import
        # torch first so that streams and device pointers it hands over belong
        # to the runtime the kernels are launched on.
        import torch  # noqa: F401
        handle = C.CDLL(LIB_PATH)
        handle.hbt_version.restype = C.c_int
        if handle.hbt_version() != ABI_VERSION:
            raise ImportError(
                "habitat_amd: %s implements ABI %d, this package binds ABI %d - rebuild it with "
                "`python -m habitat_amd.build`" % (LIB_PATH, handle.hbt_version(), ABI_VERSION))
        for name, (res, args) in list(_SIGNATURES.items()) + list(_OPTIONAL.items()):
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def strerror(code):
    return lib().hbt_strerror(code).decode()


def check(code, what):
    if code != HBT_OK:
        raise HabitatLibraryError(code, what)
