"""TEST INFRASTRUCTURE — ctypes loaders for the oracle's C code and for the
compiled reference occupancy routine (oracle/_ref), plus the build step."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "_build", "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libref_occupancy.so")


class Device(C.Structure):
    """Same field order as `orc_device` in occupancy.c (and as the reference's
    DeviceProperties, cpp/src/cuda/kernel.h:14-62, minus the name)."""
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


# Keyword names of the reference's DeviceProperties constructor
# (cpp/src/frontend/model_bindings.cpp:19-34) → struct fields.
_KW = {
    "compute_major": "compute_major", "compute_minor": "compute_minor",
    "max_threads_per_block": "max_threads_per_block",
    "max_threads_per_multiprocessor": "max_threads_per_sm",
    "regs_per_block": "regs_per_block", "regs_per_multiprocessor": "regs_per_sm",
    "warp_size": "warp_size", "shared_mem_per_block": "smem_per_block",
    "shared_mem_per_multiprocessor": "smem_per_sm", "num_sms": "num_sms",
    "shared_mem_per_block_optin": "smem_per_block_optin",
    "mem_bandwidth_gb": "mem_bandwidth_gb", "base_clock_mhz": "base_clock_mhz",
    "peak_gflops_per_second": "peak_gflops",
}


def make_device(**kwargs):
    d = Device()
    for k, v in kwargs.items():
        if k == "name":
            continue
        setattr(d, _KW[k], v)
    return d


def build(force=False):
    """Compile the oracle (and oracle/_ref where the reference is mounted)."""
    if force or not os.path.exists(ORACLE_SO) or (
            os.path.isdir("/root/reference") and not os.path.exists(REF_SO)):
        subprocess.check_call(["make", "-s", "-C", HERE] + (["-B"] if force else []))


_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")


class Limits(C.Structure):
    _fields_ = [("regs", C.c_int32), ("smem", C.c_int32), ("warps", C.c_int32),
                ("blocks", C.c_int32), ("error", C.c_int32)]


_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        build()
        lib = C.CDLL(ORACLE_SO)
        lib.orc_occupancy.restype = C.c_uint32
        lib.orc_occupancy.argtypes = [C.POINTER(Device)] + [C.c_int32] * 4
        lib.orc_occupancy_limits.restype = C.c_int
        lib.orc_occupancy_limits.argtypes = (
            [C.POINTER(Device)] + [C.c_int32] * 4 + [C.POINTER(Limits)])
        lib.orc_occupancy_batch.restype = None
        lib.orc_occupancy_batch.argtypes = (
            [C.POINTER(Device), C.c_int64] + [_i32p] * 4 + [C.c_void_p, _i32p])
        lib.orc_wave_scale.restype = None
        lib.orc_wave_scale.argtypes = (
            [C.POINTER(Device), C.POINTER(Device), C.c_int64] + [_i32p] * 5 +
            [C.c_void_p] + [_f64p] * 4 + [C.c_void_p] +
            [_f64p, _i32p, _i32p, _i32p, _i32p, _u8p, C.c_void_p])
        _oracle = lib
    return _oracle


def have_ref():
    if os.path.isdir("/root/reference"):
        build()
    return os.path.exists(REF_SO)


def ref():
    """The reference's own kernel.cpp behind a C face; None where it was never built."""
    global _ref
    if _ref is None:
        if not have_ref():
            return None
        lib = C.CDLL(REF_SO)
        lib.ref_occupancy.restype = C.c_uint32
        lib.ref_occupancy.argtypes = [C.POINTER(Device)] + [C.c_int32] * 5
        lib.ref_occupancy_batch.restype = None
        lib.ref_occupancy_batch.argtypes = (
            [C.POINTER(Device), C.c_int64] + [_i32p] * 4 + [C.c_void_p, _i32p])
        _ref = lib
    return _ref


def _opt(a, dtype):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    return a.ctypes.data_as(C.c_void_p), a


def occupancy(dev, block, dyn_smem, static_smem, regs):
    return int(oracle().orc_occupancy(C.byref(dev), block, dyn_smem, static_smem, regs))


def occupancy_limits(dev, block, dyn_smem, static_smem, regs):
    lim = Limits()
    occ = oracle().orc_occupancy_limits(C.byref(dev), block, dyn_smem, static_smem, regs,
                                        C.byref(lim))
    return occ, lim


def _batch(fn, dev, block, dyn_smem, static_smem, own_regs, registers=None):
    block = np.ascontiguousarray(block, np.int32)
    out = np.empty(block.shape[0], np.int32)
    r = _opt(registers, np.int32)
    fn(C.byref(dev), block.shape[0], block,
       np.ascontiguousarray(dyn_smem, np.int32), np.ascontiguousarray(static_smem, np.int32),
       np.ascontiguousarray(own_regs, np.int32), r[0] if r else None, out)
    return out


def occupancy_batch(dev, block, dyn_smem, static_smem, own_regs, registers=None):
    return _batch(oracle().orc_occupancy_batch, dev, block, dyn_smem, static_smem,
                  own_regs, registers)


def ref_occupancy_batch(dev, block, dyn_smem, static_smem, own_regs, registers=None):
    return _batch(ref().ref_occupancy_batch, dev, block, dyn_smem, static_smem,
                  own_regs, registers)


def wave_scale(origin, dest, rec, want_gamma=False):
    """Run the C restatement over a dict of numpy columns (see
    wave_scaling.c).  Returns a dict of numpy outputs."""
    n = int(rec["num_blocks"].shape[0])
    c = lambda k, t: np.ascontiguousarray(rec[k], t)
    out = {
        "time_ns": np.empty(n, np.float64), "occ_origin": np.empty(n, np.int32),
        "occ_dest": np.empty(n, np.int32), "wave_origin": np.empty(n, np.int32),
        "wave_dest": np.empty(n, np.int32), "status": np.empty(n, np.uint8),
    }
    gamma = np.empty(n, np.float64) if want_gamma else None
    dr = _opt(rec.get("dest_regs"), np.int32)
    hm = _opt(rec.get("has_metrics"), np.uint8)
    oracle().orc_wave_scale(
        C.byref(origin), C.byref(dest), n,
        c("num_blocks", np.int32), c("block_size", np.int32), c("dynamic_smem", np.int32),
        c("static_smem", np.int32), c("regs_per_thread", np.int32),
        dr[0] if dr else None,
        c("run_time_ns", np.float64), c("flop_sp_efficiency", np.float64),
        c("dram_read_bytes", np.float64), c("dram_write_bytes", np.float64),
        hm[0] if hm else None,
        out["time_ns"], out["occ_origin"], out["occ_dest"], out["wave_origin"],
        out["wave_dest"], out["status"],
        gamma.ctypes.data_as(C.c_void_p) if want_gamma else None)
    if want_gamma:
        out["gamma"] = gamma
    return out
