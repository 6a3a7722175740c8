"""TEST INFRASTRUCTURE — CPU oracle, not product code.

Wave scaling of ONE kernel record in pure Python, keeping the reference's
operation order and raising what the reference raises.  It exists to pin
oracle/wave_scaling.c (same numbers, bit for bit) and to define the exception
each batch status stands for.  Pure-Python loops: small cases only.

Follows, in the reference:
  analyzer/habitat/analysis/wave_scaling/unified.py:8-35       (metric probe, fallback)
  analyzer/habitat/analysis/wave_scaling/roofline.py:8-108     (gamma, two branches)
  analyzer/habitat/analysis/wave_scaling/resimplified.py:7-40  (no-metrics strategy)
  analyzer/habitat/analysis/wave_scaling/common.py:3-20        (wave sizes)

A record is a mapping with the keys of `KEYS`; a device is an oracle.lib.Device.
`occupancy` is injected so that tests can run this file over either the
oracle's C routine or the compiled reference routine.

pins: the hand-derived known answers in tests/golden/kat.json (gamma below and
above the ridge point, the small-kernel factor with ceilings 2 and 3, 4 and 6,
a register-table entry that changes the branch, the no-metrics strategy);
closed forms (same device both sides is the identity; flop efficiency 0 gives
t*bw_o/bw_d; zero bytes give t*(clk_o/clk_d)*(sms_o/sms_d); intensity equal to
the ridge point gives gamma 0.5 from either side).
"""
import math

from . import lib

KEYS = ("num_blocks", "block_size", "dynamic_smem", "static_smem", "regs_per_thread",
        "run_time_ns", "flop_sp_efficiency", "dram_read_bytes", "dram_write_bytes")


def _occ(dev, rec, regs):
    return lib.occupancy(dev, rec["block_size"], rec["dynamic_smem"], rec["static_smem"], regs)


def wave_info(rec, origin, dest, dest_regs=None, occupancy=_occ):
    """common.py:3-20.  `dest_regs` plays metadata_manager.kernel_registers_for()."""
    occ_o = occupancy(origin, rec, rec["regs_per_thread"])
    wave_o = origin.num_sms * occ_o
    if dest_regs is not None:
        occ_d = occupancy(dest, rec, dest_regs)
    else:
        occ_d = occupancy(dest, rec, rec["regs_per_thread"])
    wave_d = dest.num_sms * occ_d
    return wave_o, wave_d, occ_o, occ_d


def gamma(rec, origin, dest):
    """roofline.py:68-108."""
    eff = rec["flop_sp_efficiency"]
    total_gb = (rec["dram_read_bytes"] + rec["dram_write_bytes"]) / 1024 / 1024 / 1024
    gflops_per_second = eff / 100 * origin.peak_gflops
    num_gflops = gflops_per_second * rec["run_time_ns"] / 1e9
    if num_gflops < 1e-9:
        g = 1.
    elif total_gb == 0:
        g = 0.
    else:
        intensity = num_gflops / total_gb
        ridge = dest.peak_gflops / dest.mem_bandwidth_gb
        if intensity > ridge:
            g = 0.5 * ridge / intensity
        else:
            g = -0.5 / ridge * intensity + 1.
    assert g >= 0 and g <= 1
    return g


def _is_small(rec, wave_o, wave_d):
    # `//` raises ZeroDivisionError on a zero wave size; `and` short-circuits.
    return rec["num_blocks"] // wave_o == 0 and rec["num_blocks"] // wave_d == 0


def roofline(rec, origin, dest, dest_regs=None, occupancy=_occ):
    """roofline.py:8-65."""
    g = gamma(rec, origin, dest)
    g_compl = 1.0 - g
    wave_o, wave_d, _, _ = wave_info(rec, origin, dest, dest_regs, occupancy)
    t = rec["run_time_ns"]
    if _is_small(rec, wave_o, wave_d):
        o_max = math.ceil(rec["num_blocks"] / origin.num_sms)
        d_max = math.ceil(rec["num_blocks"] / dest.num_sms)
        factor = (origin.base_clock_mhz / dest.base_clock_mhz) * (d_max / o_max)
        return t * math.pow(factor, g_compl)
    bw = origin.mem_bandwidth_gb / dest.mem_bandwidth_gb
    clk = origin.base_clock_mhz / dest.base_clock_mhz
    sm = origin.num_sms / dest.num_sms
    return t * math.pow(bw, g) * math.pow(clk, g_compl) * math.pow(sm, g_compl)


def resimplified(rec, origin, dest, dest_regs=None, occupancy=_occ):
    """resimplified.py:7-40."""
    wave_o, wave_d, _, _ = wave_info(rec, origin, dest, dest_regs, occupancy)
    if _is_small(rec, wave_o, wave_d):
        return rec["run_time_ns"]
    return rec["run_time_ns"] * (origin.mem_bandwidth_gb / dest.mem_bandwidth_gb)


def unified(rec, origin, dest, dest_regs=None, has_metrics=True, occupancy=_occ):
    """unified.py:8-35: roofline when the three metrics exist, else resimplified."""
    if has_metrics:
        return roofline(rec, origin, dest, dest_regs, occupancy)
    return resimplified(rec, origin, dest, dest_regs, occupancy)


STATUS_EXCEPTION = {1: ZeroDivisionError, 2: ZeroDivisionError, 3: AssertionError,
                    4: ZeroDivisionError}


def unified_with_status(rec, origin, dest, dest_regs=None, has_metrics=True, occupancy=_occ):
    """(time, status) with the batch status codes of wave_scaling.c."""
    try:
        return float(unified(rec, origin, dest, dest_regs, has_metrics, occupancy)), 0
    except AssertionError:
        return math.nan, 3
    except ZeroDivisionError:
        wave_o, wave_d, _, _ = wave_info(rec, origin, dest, dest_regs, occupancy)
        if wave_o == 0:
            return math.nan, 1
        if wave_d == 0:
            return math.nan, 2
        return math.nan, 4
