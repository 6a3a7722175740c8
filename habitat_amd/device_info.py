"""The local GPU in the device table's terms, and measured ceilings.

    python -m habitat_amd.device_info [--device 0] [--measure]

prints the keys of data/devices.yml for the GPU this process sees (the role of
the reference's `device_info` tool, cpp/src/device_info.cpp:9-33) and, with
--measure, the measured fp32 FMA and MFMA rates and the device-to-device copy
bandwidth (the role of tools/device-metadata/measure_peak_flops.py).
"""
import argparse
import ctypes

from habitat_amd import _lib


def local_device(device=0):
    """(name, dict with the keyword arguments of DeviceProperties) from
    hipDeviceProp_t.  The compute capability is HIP's (gfx950 reports 9.5), which
    the NVIDIA-rule occupancy model does not know: to use the GPU as a
    *destination* give it the rules of a known capability, as the MI355X entry
    of data/devices.yml does."""
    spec = _lib.DeviceSpec()
    name = ctypes.create_string_buffer(256)
    rc = _lib.lib().hbt_local_device_spec(device, ctypes.byref(spec), name, 256)
    _lib.check(rc, "hbt_local_device_spec")
    props = {
        "compute_major": spec.compute_major, "compute_minor": spec.compute_minor,
        "max_threads_per_block": spec.max_threads_per_block,
        "max_threads_per_multiprocessor": spec.max_threads_per_sm,
        "regs_per_block": spec.regs_per_block, "regs_per_multiprocessor": spec.regs_per_sm,
        "warp_size": spec.warp_size, "shared_mem_per_block": spec.smem_per_block,
        "shared_mem_per_multiprocessor": spec.smem_per_sm, "num_sms": spec.num_sms,
        "shared_mem_per_block_optin": spec.smem_per_block_optin,
        "mem_bandwidth_gb": int(round(spec.mem_bandwidth_gb)),
        "base_clock_mhz": int(round(spec.base_clock_mhz)),
        "peak_gflops_per_second": int(round(spec.peak_gflops)),
    }
    return name.value.decode(), props


def measure(iters=20000, copy_bytes=1 << 30):
    """{'fp32_fma_gflops', 'fp32_mfma_gflops', 'copy_gbps'} measured on the
    current device (allocates scratch memory, synchronises)."""
    L = _lib.lib()
    out = {}
    v = ctypes.c_double(0)
    _lib.check(L.hbt_measure_fp32_fma_gflops(iters, ctypes.byref(v)), "hbt_measure_fp32_fma_gflops")
    out["fp32_fma_gflops"] = v.value
    _lib.check(L.hbt_measure_fp32_mfma_gflops(iters, ctypes.byref(v)), "hbt_measure_fp32_mfma_gflops")
    out["fp32_mfma_gflops"] = v.value
    _lib.check(L.hbt_measure_copy_gbps(copy_bytes, ctypes.byref(v)), "hbt_measure_copy_gbps")
    out["copy_gbps"] = v.value
    return out


def record_stream_gbps(records, warmup=2000, launches=2000):
    """GB/s (68 bytes per record) of a kernel doing only the loads and stores of
    wave scaling on `records` records: the data-movement ceiling at that size."""
    v = ctypes.c_double(0)
    _lib.check(_lib.lib().hbt_measure_record_stream_gbps(records, warmup, launches,
                                                         ctypes.byref(v)),
               "hbt_measure_record_stream_gbps")
    return v.value


def record_stream_multi_gbps(records, n_dest, warmup=500, launches=500):
    """GB/s (52 + 4 + 13 x n_dest bytes per record) of a kernel doing only the
    loads and stores of wave scaling to `n_dest` destinations in one launch."""
    v = ctypes.c_double(0)
    _lib.check(_lib.lib().hbt_measure_record_stream_multi_gbps(records, n_dest, warmup, launches,
                                                               ctypes.byref(v)),
               "hbt_measure_record_stream_multi_gbps")
    return v.value


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--measure", action="store_true")
    args = ap.parse_args()
    name, props = local_device(args.device)
    print("# " + name)
    for k, v in props.items():
        print("%s: %s" % (k, v))
    if args.measure:
        for k, v in measure().items():
            print("# measured %s: %.1f" % (k, v))


if __name__ == "__main__":
    main()
