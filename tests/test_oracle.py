"""CPU: pins the oracle (oracle/occupancy.c, wave_scaling.c, wave_scaling.py)
before anything is compared with it: reference-compiled golden vectors,
hand-derived known answers, the compiled reference itself where it was built,
closed forms and invariants."""
import json
import math
import os

import numpy as np
import pytest

from conftest import GOLDEN, oracle_device
from oracle import lib as olib
from oracle import wave_scaling as ows


def _devs():
    with open(os.path.join(GOLDEN, "occupancy_golden_devices.json")) as f:
        return json.load(f)


DEVS = _devs()


# ----------------------------------------------------------------- occupancy
def test_oracle_occupancy_matches_reference_golden(occupancy_golden):
    g, devices = occupancy_golden
    assert g["block"].shape[0] > 12000 and len(devices) >= 12
    for name, props in devices.items():
        d = oracle_device(props)
        own = olib.occupancy_batch(d, g["block"], g["dyn"], g["stat"], g["regs"])
        lut = olib.occupancy_batch(d, g["block"], g["dyn"], g["stat"], g["regs"], g["dregs"])
        assert np.array_equal(own, g["occ_own__" + name]), name
        assert np.array_equal(lut, g["occ_lut__" + name]), name


def test_oracle_occupancy_matches_compiled_reference_on_fresh_inputs():
    if olib.ref() is None:
        pytest.skip("oracle/_ref was not built (reference tree not mounted)")
    rng = np.random.default_rng(99)
    n = 50000
    block = rng.integers(1, 1100, n).astype(np.int32)
    dyn = rng.integers(0, 70000, n).astype(np.int32)
    stat = rng.integers(0, 50000, n).astype(np.int32)
    regs = rng.integers(0, 300, n).astype(np.int32)
    for name, props in DEVS.items():
        d = oracle_device(props)
        assert np.array_equal(olib.occupancy_batch(d, block, dyn, stat, regs),
                              olib.ref_occupancy_batch(d, block, dyn, stat, regs)), name


def test_oracle_occupancy_known_answers(kat):
    for dev, block, regs, stat, dyn, occ, wave in kat["occupancy"]:
        d = oracle_device(DEVS[dev])
        got = olib.occupancy(d, block, dyn, stat, regs)
        assert got == occ, (dev, block, regs, stat, dyn)
        if wave is not None:
            assert got * d.num_sms == wave
    for row in kat["occupancy_limits"]:
        d = oracle_device(DEVS[row["device"]])
        occ, lim = olib.occupancy_limits(d, row["block"], row["smem"], 0, row["regs"])
        assert (lim.regs, lim.warps, lim.blocks, lim.smem) == (
            row["reg"], row["warp"], row["block_slots"], row["smem_limit"]), row
        assert occ == min(lim.regs, lim.warps, lim.blocks, lim.smem)


def test_oracle_occupancy_invariants():
    rng = np.random.default_rng(5)
    d = oracle_device(DEVS["V100"])
    for _ in range(300):
        block = int(rng.integers(1, 1025))
        smem = int(rng.integers(0, 49152))
        regs = int(rng.integers(0, 200))
        occ, lim = olib.occupancy_limits(d, block, smem, 0, regs)
        assert occ == min(lim.regs, lim.warps, lim.blocks, lim.smem)
        # more registers or more shared memory never raise the occupancy
        assert olib.occupancy(d, block, smem, 0, regs + 8) <= occ
        assert olib.occupancy(d, block, smem + 1024, 0, regs) <= occ
        # nothing but warps and block slots limit a kernel without resources
        assert olib.occupancy(d, block, 0, 0, 0) == min(lim.warps, lim.blocks)
    # 16-bit narrowing of the register count (kernel.h:108)
    assert olib.occupancy(d, 256, 0, 0, 65536 + 32) == olib.occupancy(d, 256, 0, 0, 32)


# -------------------------------------------------------------- wave scaling
def _record(kat, num_blocks, **over):
    rec = dict(kat["scaling_record"], num_blocks=num_blocks)
    rec.update(over)
    return rec


def _cols(recs):
    return {k: np.array([r[k] for r in recs]) for k in recs[0]}


def _kat_case(kat, row):
    """(record, origin, dest, dest_regs, has_metrics) of one scaling known answer."""
    o, d = oracle_device(DEVS[row["origin"]]), oracle_device(DEVS[row["dest"]])
    rec = _record(kat, row["num_blocks"], **row.get("record", {}))
    return rec, o, d, row.get("dest_regs"), row.get("has_metrics", True)


def test_scaling_known_answers_python_and_c(kat):
    assert sum(r.get("above_ridge", False) for r in kat["scaling"]) >= 3
    assert any(r.get("origin_ceiling", 0) != r.get("dest_ceiling", 0) for r in kat["scaling"])
    for row in kat["scaling"]:
        rec, o, d, dest_regs, hm = _kat_case(kat, row)
        if hm:
            assert ows.gamma(rec, o, d) == pytest.approx(row["gamma"], rel=1e-15)
        assert ows.unified(rec, o, d, dest_regs, hm) == pytest.approx(row["time_ns"], rel=1e-14)
        cols = _cols([rec])
        cols["has_metrics"] = np.array([hm], np.uint8)
        if dest_regs is not None:
            cols["dest_regs"] = np.array([dest_regs], np.int32)
        c = olib.wave_scale(o, d, cols, want_gamma=True)
        assert c["status"][0] == 0
        assert c["time_ns"][0] == pytest.approx(row["time_ns"], rel=1e-14)
        if hm:
            assert c["gamma"][0] == pytest.approx(row["gamma"], rel=1e-15)
        wave_o, wave_d, occ_o, occ_d = ows.wave_info(rec, o, d, dest_regs)
        for key, got, got_c in (("occ_origin", occ_o, c["occ_origin"][0]),
                                ("occ_dest", occ_d, c["occ_dest"][0]),
                                ("wave_origin", wave_o, c["wave_origin"][0]),
                                ("wave_dest", wave_d, c["wave_dest"][0])):
            if key in row:
                assert got == row[key] == got_c, (key, row)
        small = row["num_blocks"] < wave_o and row["num_blocks"] < wave_d
        assert small == (row["branch"] == "small")


def test_scaling_closed_forms(kat):
    v100, p100 = oracle_device(DEVS["V100"]), oracle_device(DEVS["P100"])
    big = 1 << 16
    # same device on both sides: identity on both strategies and both branches
    for nb in (3, big):
        for hm in (True, False):
            t = ows.unified(_record(kat, nb), v100, v100, has_metrics=hm)
            assert t == pytest.approx(1e6, rel=1e-15)
    # no FLOPs: gamma = 1, pure bandwidth ratio
    t = ows.unified(_record(kat, big, flop_sp_efficiency=0.0), v100, p100)
    assert ows.gamma(_record(kat, big, flop_sp_efficiency=0.0), v100, p100) == 1.0
    assert t == pytest.approx(1e6 * 739 / 501, rel=1e-15)
    # no bytes but FLOPs: gamma = 0, clock ratio times SM ratio
    r = _record(kat, big, dram_read_bytes=0.0, dram_write_bytes=0.0)
    assert ows.gamma(r, v100, p100) == 0.0
    assert ows.unified(r, v100, p100) == pytest.approx(1e6 * (1312 / 1126) * (80 / 56), rel=1e-15)
    # intensity exactly at the ridge point: both formulas give 1/2
    ridge = 9504 / 501
    gflops = 50.0 / 100 * 6716 * 1e6 / 1e9
    nbytes = gflops / ridge * 1024 ** 3
    r_lo = _record(kat, big, dram_read_bytes=nbytes * (1 + 1e-9), dram_write_bytes=0.0)
    r_hi = _record(kat, big, dram_read_bytes=nbytes * (1 - 1e-9), dram_write_bytes=0.0)
    assert ows.gamma(r_lo, v100, p100) == pytest.approx(0.5, abs=1e-8)
    assert ows.gamma(r_hi, v100, p100) == pytest.approx(0.5, abs=1e-8)
    # The three factors are multiplied onto the time from left to right
    # (roofline.py:58-63), so a partial product may leave the range of fp64
    # where the whole product does not.  No bytes: gamma = 0, factors 1, clock
    # ratio, SM ratio.  RTX2070 -> V100: 1.7e308 * (1410/1312) overflows before
    # 36/80 brings it back.  (Nothing of the kind at the other end of the range:
    # a time small enough to underflow makes the FLOP count fall below 1e-9,
    # which forces gamma = 1 and leaves one factor.)
    no_bytes = dict(dram_read_bytes=0.0, dram_write_bytes=0.0)
    rtx2070 = oracle_device(DEVS["RTX2070"])
    for t_in, want in ((1.7e308, math.inf), (1e300, 1e300 * (1410 / 1312) * (36 / 80))):
        r = _record(kat, big, run_time_ns=t_in, **no_bytes)
        assert ows.gamma(r, rtx2070, v100) == 0.0
        assert ows.unified(r, rtx2070, v100) == pytest.approx(want, rel=1e-15)
        c = olib.wave_scale(rtx2070, v100, _cols([r]))
        assert c["status"][0] == 0 and c["time_ns"][0] == pytest.approx(want, rel=1e-15)
    tiny = _record(kat, big, run_time_ns=5e-324, **no_bytes)
    assert ows.gamma(tiny, oracle_device(DEVS["T4"]), oracle_device(DEVS["P4000"])) == 1.0
    # without metrics: small kernel unchanged, else bandwidth ratio
    assert ows.unified(_record(kat, 3), v100, p100, has_metrics=False) == 1000000
    assert ows.unified(_record(kat, big), v100, p100, has_metrics=False) == pytest.approx(
        1e6 * 739 / 501, rel=1e-15)
    # destination register count from the look-up table changes the wave size only
    r = _record(kat, 500)
    assert ows.wave_info(r, v100, p100, dest_regs=128)[3] == 2
    assert ows.wave_info(r, v100, p100)[3] == 8


def test_scaling_exceptions_and_statuses(kat):
    v100, p100, mi = (oracle_device(DEVS[k]) for k in ("V100", "P100", "MI355X"))
    cases = [
        # origin cannot hold the block at all
        (_record(kat, 100, regs_per_thread=255, block_size=1024), v100, p100, True, 1),
        # destination occupancy 0 and the kernel is small on the origin
        (_record(kat, 10, dynamic_smem=60000), mi, v100, True, 2),
        (_record(kat, 10, dynamic_smem=60000), mi, v100, False, 2),
        # ... but not evaluated when the origin test already fails (big kernel)
        (_record(kat, 1 << 16, dynamic_smem=60000), mi, v100, True, 0),
        (_record(kat, 1 << 16, dynamic_smem=60000), mi, v100, False, 0),
        # negative byte counts push gamma above 1
        (_record(kat, 100, dram_read_bytes=-3e8), v100, p100, True, 3),
        (_record(kat, 100, flop_sp_efficiency=float("nan")), v100, p100, True, 3),
        # a bad gamma is found before a zero wave size
        (_record(kat, 100, regs_per_thread=255, block_size=1024, dram_read_bytes=-3e8),
         v100, p100, True, 3),
        # num_blocks 0: ceil(0 / sms) = 0 divides
        (_record(kat, 0), v100, p100, True, 4),
        (_record(kat, 0), v100, p100, False, 0),
        # negative num_blocks is never "small" (floor division gives -1)
        (_record(kat, -5), v100, p100, True, 0),
    ]
    for rec, o, d, hm, want in cases:
        t, st = ows.unified_with_status(rec, o, d, has_metrics=hm)
        assert st == want, (rec, want)
        cols = _cols([rec])
        cols["has_metrics"] = np.array([1 if hm else 0], np.uint8)
        c = olib.wave_scale(o, d, cols)
        assert c["status"][0] == want
        if want:
            assert math.isnan(c["time_ns"][0]) and math.isnan(t)
            with pytest.raises(ows.STATUS_EXCEPTION[want]):
                ows.unified(rec, o, d, has_metrics=hm)
        else:
            assert c["time_ns"][0] == t


def test_c_restatement_equals_python_restatement_bit_for_bit():
    rng = np.random.default_rng(11)
    n = 3000
    recs = []
    for _ in range(n):
        total = int(rng.integers(0, 65537))
        recs.append(dict(
            num_blocks=int(2 ** rng.uniform(0, 20)), block_size=int(rng.choice([64, 128, 256, 512, 1024])),
            dynamic_smem=total - total // 2, static_smem=total // 2,
            regs_per_thread=int(rng.integers(16, 256)), run_time_ns=float(int(10 ** rng.uniform(3, 7))),
            flop_sp_efficiency=float(10 ** rng.uniform(-2, 2)),
            dram_read_bytes=float(int(10 ** rng.uniform(3, 10))),
            dram_write_bytes=float(int(10 ** rng.uniform(3, 10)))))
    cols = _cols(recs)
    hm = (rng.random(n) < 0.7).astype(np.uint8)
    dr = np.where(rng.random(n) < 0.3, rng.integers(16, 200, n), -1).astype(np.int32)
    cols["has_metrics"], cols["dest_regs"] = hm, dr
    for on, dn in (("V100", "MI355X"), ("MI355X", "V100"), ("P100", "T4"), ("T4", "P4000")):
        o, d = oracle_device(DEVS[on]), oracle_device(DEVS[dn])
        c = olib.wave_scale(o, d, cols)
        seen = set()
        for i, rec in enumerate(recs):
            t, st = ows.unified_with_status(rec, o, d, dest_regs=None if dr[i] < 0 else int(dr[i]),
                                            has_metrics=bool(hm[i]))
            assert st == c["status"][i]
            seen.add(st)
            if st == 0:
                assert t == c["time_ns"][i]  # identical doubles
            else:
                assert math.isnan(c["time_ns"][i])
        assert 0 in seen


def test_python_restatement_over_compiled_reference_occupancy(kat):
    """The wave-scaling restatement gives the same answers when its occupancy
    comes from the reference's own routine."""
    ref = olib.ref()
    if ref is None:
        pytest.skip("oracle/_ref was not built (reference tree not mounted)")
    import ctypes

    def ref_occ(dev, rec, regs):
        return int(ref.ref_occupancy(ctypes.byref(dev), rec["block_size"], rec["dynamic_smem"],
                                     rec["static_smem"], rec["regs_per_thread"], regs))
    for row in kat["scaling"]:
        rec, o, d, dest_regs, hm = _kat_case(kat, row)
        assert ows.unified(rec, o, d, dest_regs, hm, occupancy=ref_occ) == pytest.approx(
            row["time_ns"], rel=1e-14)


def test_predictor_arithmetic():
    """oracle/predictor.py against a three-operation, five-kernel trace worked
    by hand."""
    from oracle import predictor as opred
    # op 1: forward 2.0 ms with kernels 0.5 + 0.75 ms -> overhead 0.75 ms; the
    # kernels are predicted at 0.25 + 0.5 ms -> 1.5 ms.  Backward 1.0 ms with one
    # 1.5 ms kernel (longer than the pass: overhead clamps to 0) predicted 3.0 ms.
    fwd = opred.wave_scaled_pass_ms(2.0, [500000, 750000], [250000.0, 500000.0])
    bwd = opred.wave_scaled_pass_ms(1.0, [1500000], [3000000.0])
    assert fwd == 1.5 and bwd == 3.0
    # op 2: 4 ms measured, MLP predicts 0.02 on the destination, 0.05 on the origin
    assert opred.special_op_ms(4.0, 0.02, 0.05) == pytest.approx(1.6)
    # op 3: a negative prediction is clamped to zero
    assert opred.special_op_ms(4.0, -0.02, 0.05) == 0.0
    assert opred.trace_ms([fwd + bwd, 1.6, 0.0]) == pytest.approx(6.1)
    # a pass without kernels keeps its measured time
    assert opred.wave_scaled_pass_ms(0.7, [], []) == pytest.approx(0.7)


def random_device_specs(count, seed):
    """Device descriptions far from the shipped ones: every compute capability
    the routine distinguishes, odd warp sizes, limits from tiny to huge,
    occasional zeros and negatives."""
    rng = np.random.default_rng(seed)
    pick = lambda values: int(rng.choice(values))
    specs = []
    for _ in range(count):
        warp = pick([32, 32, 32, 64, 64, 16, 24, 48, 96, 128, 1, 1000])
        threads_block = pick([1024, 1024, 512, 2048, 1536, 100, 0, 65536])
        specs.append(dict(
            compute_major=pick([3, 5, 6, 6, 7, 7, 7, 8, 2, 9, 0]),
            compute_minor=pick([0, 0, 1, 2, 5, 7]),
            max_threads_per_block=threads_block,
            max_threads_per_multiprocessor=pick([2048, 1024, 1536, 4096, 768, 64, 0, 1 << 20]),
            regs_per_block=pick([65536, 32768, 131072, 65536, 4096, 0, 1 << 22, 100000]),
            regs_per_multiprocessor=pick([65536, 131072, 262144, 32768, 100000, 0, 1 << 22]),
            warp_size=warp,
            shared_mem_per_block=pick([49152, 65536, 98304, 16384, 163840, 1000, 0, 1 << 21]),
            shared_mem_per_multiprocessor=pick([65536, 98304, 102400, 163840, 49152, 32768, 8192,
                                                100, 0, 1 << 21]),
            num_sms=pick([1, 14, 80, 256, 1000]),
            shared_mem_per_block_optin=pick([0, 49152, 98304]),
            mem_bandwidth_gb=900, base_clock_mhz=1300, peak_gflops_per_second=14000))
    return specs


def test_random_device_specs_against_the_compiled_reference():
    """The oracle, the library's host routine and its 32-bit kernel model on 300
    random device descriptions x 400 launches (ordinary and out-of-range),
    against the reference's own routine compiled in place."""
    if olib.ref() is None:
        pytest.skip("oracle/_ref was not built (reference tree not mounted)")
    import ctypes
    from habitat_amd import DeviceProperties, _lib
    rng = np.random.default_rng(5)
    n = 400
    odd = np.array([0, -1, 1, 31, 33, 255, 256, 257, 1023, 1025, 65535, 65536, 65537, 1 << 20,
                    (1 << 31) - 1, -(1 << 31), -256, -510, -511])
    mix = lambda ordinary: np.where(rng.random(n) < 0.8, ordinary, rng.choice(odd, n)).astype(np.int32)
    accepted = model32_checked = 0
    for props in random_device_specs(300, 17):
        block = mix(rng.integers(1, 2100, n))
        dyn = mix(rng.integers(0, 120000, n))
        stat = mix(rng.integers(0, 60000, n))
        regs = mix(rng.integers(0, 300, n))
        d = oracle_device(props)
        want = olib.ref_occupancy_batch(d, block, dyn, stat, regs)
        assert np.array_equal(olib.occupancy_batch(d, block, dyn, stat, regs), want), props
        accepted += bool(want.any())
        dev = DeviceProperties(name="r", **props)
        for fn in ("hbt_occupancy_host_batch", "hbt_occupancy_host_model32_batch"):
            out = np.full(n, -9, np.int32)
            rc = getattr(_lib.lib(), fn)(
                ctypes.byref(dev.spec), n, *[a.ctypes.data_as(ctypes.c_void_p)
                                             for a in (block, dyn, stat, regs)],
                out.ctypes.data_as(ctypes.c_void_p))
            if fn.endswith("model32_batch") and rc == _lib.HBT_ESPEC:
                continue          # a limit of 2^20 or more: the kernel uses the 64-bit model
            assert rc == 0, (fn, rc, props)
            assert np.array_equal(out, want), (fn, props)
            model32_checked += fn.endswith("model32_batch")
    assert accepted > 60 and model32_checked > 150
