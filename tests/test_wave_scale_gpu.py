"""GPU: the HIP wave-scaling path (through the C ABI) against the CPU oracle.
Integers and statuses bit-exact; fp64 times within 1e-6 relative."""
import json
import math
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN, oracle_device
from habitat_amd import Device, DeviceProperties, synthetic
from habitat_amd.analysis.wave_scaling.batch import KernelRecords, WaveScaleOutput, wave_scale
from oracle import lib as olib

pytestmark = pytest.mark.gpu

TIME_RTOL = 1e-6   # tolerance for the fp64 scaled time


def odev(d):
    return oracle_device(d.as_dict())


def check(rec, origin, dests, out, rows=None):
    """Compare every output of `out` with the oracle."""
    n = rec["num_blocks"].shape[0]
    occ_o = out.occ_origin.cpu().numpy()
    for di, d in enumerate(dests):
        want = olib.wave_scale(odev(origin), odev(d), rec)
        assert np.array_equal(occ_o, want["occ_origin"])
        assert np.array_equal(out.occ_dest[di].cpu().numpy(), want["occ_dest"]), d.name
        if out.wave_origin is not None:
            assert np.array_equal(out.wave_origin.cpu().numpy(), want["wave_origin"])
            assert np.array_equal(out.wave_dest[di].cpu().numpy(), want["wave_dest"])
        st = out.status[di].cpu().numpy()
        assert np.array_equal(st, want["status"]), d.name
        t = out.time_ns[di].cpu().numpy()
        ok = want["status"] == 0
        assert np.all(np.isnan(t[~ok]))
        # atol: a subnormal result (a subnormal measured time, in the adversarial
        # sets) has no 1e-6 relative precision to meet; allow its last bits
        np.testing.assert_allclose(t[ok], want["time_ns"][ok], rtol=TIME_RTOL, atol=1e-320)
        normal = ok & (np.abs(want["time_ns"]) > 1e-300) & np.isfinite(want["time_ns"])
        if normal.any():
            worst = np.max(np.abs(t[normal] - want["time_ns"][normal]) / np.abs(want["time_ns"][normal]))
            print("wave scaling %s -> %s, %d records: max relative time error vs oracle %.3g "
                  "(bound %.0e); integers and statuses exact"
                  % (origin.name, d.name, n, float(worst), TIME_RTOL))
    return n


def test_config0_10k_records_v100_to_mi355x():
    rec, stats = synthetic.kernel_records(10_000, Device.V100, seed=0)
    out = wave_scale(KernelRecords.from_numpy(rec), Device.V100, [Device.MI355X])
    check(rec, Device.V100, [Device.MI355X], out)


def test_config1_1m_records():
    rec, _ = synthetic.kernel_records(1_000_000, Device.V100, seed=0)
    out = wave_scale(KernelRecords.from_numpy(rec), Device.V100, [Device.MI355X])
    check(rec, Device.V100, [Device.MI355X], out)
    # size-independent properties at the full size
    t = out.time_ns[0]
    assert bool(torch.all(t > 0)) and bool(torch.all(torch.isfinite(t)))
    # V100 -> MI355X: every factor favours the destination, so times shrink
    assert bool(torch.all(t < torch.from_numpy(rec["run_time_ns"]).cuda()))


def test_hand_worked_known_answers_through_the_batch_kernel(kat):
    """The kernel against the numbers worked by hand from roofline.py:8-104 and
    resimplified.py:7-40 (tests/golden/kat.json), without the oracle in between:
    gamma above and below the ridge point, unequal small-kernel ceilings, a
    register-table entry that changes the branch, records without metrics.
    All rows of one (origin, destination) pair go through one launch."""
    pairs = {}
    for row in kat["scaling"]:
        pairs.setdefault((row["origin"], row["dest"]), []).append(row)
    for (oname, dname), rows in pairs.items():
        recs = [dict(kat["scaling_record"], num_blocks=r["num_blocks"], **r.get("record", {}))
                for r in rows]
        rec = {k: np.array([r[k] for r in recs]) for k in recs[0]}
        rec = {k: v.astype(np.float64 if k in ("run_time_ns", "flop_sp_efficiency", "dram_read_bytes",
                                                "dram_write_bytes") else np.int32)
               for k, v in rec.items()}
        rec["dest_regs"] = np.array([r.get("dest_regs", -1) for r in rows], np.int32)
        rec["has_metrics"] = np.array([r.get("has_metrics", True) for r in rows], np.uint8)
        out = wave_scale(KernelRecords.from_numpy(rec), getattr(Device, oname),
                         [getattr(Device, dname)])
        assert not out.status[0].cpu().numpy().any()
        t = out.time_ns[0].cpu().numpy()
        for i, r in enumerate(rows):
            assert t[i] == pytest.approx(r["time_ns"], rel=TIME_RTOL), r
            for key, col in (("occ_origin", out.occ_origin), ("occ_dest", out.occ_dest[0]),
                             ("wave_origin", out.wave_origin), ("wave_dest", out.wave_dest[0])):
                if key in r:
                    assert int(col[i]) == r[key], (key, r)
        # gamma alone for the rows that have metrics
        from habitat_amd.analysis.wave_scaling.batch import roofline_gamma
        g = roofline_gamma(KernelRecords.from_numpy(rec), getattr(Device, oname),
                           getattr(Device, dname)).cpu().numpy()
        for i, r in enumerate(rows):
            if r.get("has_metrics", True):
                assert g[i] == pytest.approx(r["gamma"], rel=1e-12), r


def test_one_record_entry_point_through_the_c_abi(kat):
    """hbt_wave_scale_one (a host record in, time / occupancies / status out,
    synchronous) against the hand-worked known answers, against the batch entry
    point bit for bit on ordinary and adversarial records, and its argument
    checks."""
    import ctypes
    from habitat_amd import _lib
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def one(origin, dest, rec_fields):
        rec = _lib.KernelRecord(**rec_fields)
        t, st = ctypes.c_double(-1.0), ctypes.c_uint8(99)
        oo, od = ctypes.c_int32(-7), ctypes.c_int32(-7)
        rc = L.hbt_wave_scale_one(ctypes.byref(origin.spec), ctypes.byref(dest.spec),
                                  ctypes.byref(rec), ctypes.byref(t), ctypes.byref(oo),
                                  ctypes.byref(od), ctypes.byref(st), stream)
        assert rc == 0
        return t.value, oo.value, od.value, st.value

    base = kat["scaling_record"]
    for row in kat["scaling"]:
        over = row.get("record", {})
        fields = dict(num_blocks=row["num_blocks"], block_size=base["block_size"],
                      dynamic_smem=base["dynamic_smem"], static_smem=base["static_smem"],
                      regs=base["regs_per_thread"], dest_regs=row.get("dest_regs", -1),
                      has_metrics=int(row.get("has_metrics", True)),
                      run_time_ns=float(base["run_time_ns"]),
                      flop_sp_efficiency=over.get("flop_sp_efficiency", base["flop_sp_efficiency"]),
                      dram_read_bytes=base["dram_read_bytes"],
                      dram_write_bytes=base["dram_write_bytes"])
        t, oo, od, st = one(getattr(Device, row["origin"]), getattr(Device, row["dest"]), fields)
        assert st == 0 and t == pytest.approx(row["time_ns"], rel=TIME_RTOL), row
        if "occ_origin" in row:
            assert oo == row["occ_origin"]
        if "occ_dest" in row:
            assert od == row["occ_dest"]
    # the same kernel as the batch call: identical bits, record by record
    for rec in (synthetic.kernel_records(300, Device.V100, seed=31, metrics_fraction=0.7)[0],
                adversarial_records(300, 5)):
        out = wave_scale(KernelRecords.from_numpy(rec), Device.V100, [Device.T4])
        bt, bs = out.time_ns[0].cpu().numpy(), out.status[0].cpu().numpy()
        bo, bd = out.occ_origin.cpu().numpy(), out.occ_dest[0].cpu().numpy()
        for i in range(300):
            fields = dict(num_blocks=int(rec["num_blocks"][i]), block_size=int(rec["block_size"][i]),
                          dynamic_smem=int(rec["dynamic_smem"][i]),
                          static_smem=int(rec["static_smem"][i]), regs=int(rec["regs_per_thread"][i]),
                          dest_regs=int(rec["dest_regs"][i]) if "dest_regs" in rec else -1,
                          has_metrics=int(rec["has_metrics"][i]) if "has_metrics" in rec else 1,
                          run_time_ns=float(rec["run_time_ns"][i]),
                          flop_sp_efficiency=float(rec["flop_sp_efficiency"][i]),
                          dram_read_bytes=float(rec["dram_read_bytes"][i]),
                          dram_write_bytes=float(rec["dram_write_bytes"][i]))
            t, oo, od, st = one(Device.V100, Device.T4, fields)
            assert (st, oo, od) == (bs[i], bo[i], bd[i]), i
            assert t == bt[i] or (math.isnan(t) and math.isnan(bt[i])), i
    # argument checks
    rec = _lib.KernelRecord()
    t, st = ctypes.c_double(0), ctypes.c_uint8(0)
    v100 = ctypes.byref(Device.V100.spec)
    assert L.hbt_wave_scale_one(v100, v100, None, ctypes.byref(t), None, None, ctypes.byref(st),
                                stream) == _lib.HBT_EINVAL
    assert L.hbt_wave_scale_one(v100, v100, ctypes.byref(rec), None, None, None, ctypes.byref(st),
                                stream) == _lib.HBT_EINVAL
    bad = DeviceProperties(name="z", **dict(Device.V100.as_dict(), base_clock_mhz=0))
    assert L.hbt_wave_scale_one(v100, ctypes.byref(bad.spec), ctypes.byref(rec), ctypes.byref(t),
                                None, None, ctypes.byref(st), stream) == _lib.HBT_ESPEC


def test_identity_and_round_trip_properties():
    rec, _ = synthetic.kernel_records(200_000, Device.V100, seed=3, metrics_fraction=0.5)
    kr = KernelRecords.from_numpy(rec)
    same = wave_scale(kr, Device.V100, [Device.V100])
    t = same.time_ns[0].cpu().numpy()
    np.testing.assert_allclose(t, rec["run_time_ns"], rtol=1e-12)
    assert np.array_equal(same.occ_origin.cpu().numpy(), same.occ_dest[0].cpu().numpy())
    # linearity in the measured time: scaling 3t gives 3 * scale(t) unless gamma moves
    rec3 = dict(rec, flop_sp_efficiency=np.zeros_like(rec["flop_sp_efficiency"]))   # gamma = 1
    a = wave_scale(KernelRecords.from_numpy(rec3), Device.V100, [Device.T4]).time_ns[0].cpu().numpy()
    rec3["run_time_ns"] = rec3["run_time_ns"] * 3
    b = wave_scale(KernelRecords.from_numpy(rec3), Device.V100, [Device.T4]).time_ns[0].cpu().numpy()
    np.testing.assert_allclose(b, 3 * a, rtol=1e-12)


def test_every_device_pair_with_metrics_mix_and_register_table():
    rng = np.random.default_rng(4)
    names = ["P4000", "GTX1080Ti", "RTX2070", "RTX2080Ti", "P4", "T4", "V100", "P100", "MI355X"]
    for oname in ("V100", "P100", "T4", "MI355X", "P4000"):
        origin = getattr(Device, oname)
        rec, _ = synthetic.kernel_records(20_000, origin, seed=5, metrics_fraction=0.6)
        rec["dest_regs"] = np.where(rng.random(20_000) < 0.4, rng.integers(0, 300, 20_000),
                                    -1).astype(np.int32)
        dests = [getattr(Device, n) for n in names]          # 9 destinations: two launches
        out = wave_scale(KernelRecords.from_numpy(rec), origin, dests)
        check(rec, origin, dests, out)


def test_destinations_that_share_occupancy_constants():
    """A launch evaluates the occupancy model once per run of destinations with
    equal occupancy constants (the library puts equal ones next to each other):
    every destination's row must still be its own, whatever the order given,
    and equal what a launch for that destination alone writes."""
    origin = Device.V100
    rec, _ = synthetic.kernel_records(30_000, origin, seed=21, metrics_fraction=0.7)
    rng = np.random.default_rng(21)
    rec["dest_regs"] = np.where(rng.random(30_000) < 0.3, rng.integers(16, 256, 30_000),
                                -1).astype(np.int32)
    kr = KernelRecords.from_numpy(rec)
    sweep, _ = synthetic.device_sweep(6, seed=1)         # one class: only SMs, bandwidth, clock differ
    named = [getattr(Device, n) for n in ("T4", "P4000", "RTX2070", "P100", "GTX1080Ti", "P4",
                                          "RTX2080Ti", "MI355X")]
    mixed = [named[0], sweep[0], named[1], sweep[1], named[2], named[3], sweep[2], named[4],   # launch 1
             sweep[3], named[5], named[6], sweep[4], named[7], sweep[5]]                      # launch 2
    worst = 0.0
    # a warp size that is no power of two puts the launch on the general instantiation
    odd = DeviceProperties(name="odd", **dict(Device.V100.as_dict(), warp_size=48))
    odd2 = DeviceProperties(name="odd2", **dict(Device.V100.as_dict(), warp_size=48, num_sms=33,
                                                mem_bandwidth_gb=300))
    for dests in (mixed, sweep, [odd, named[0], odd2, sweep[0], named[2], sweep[1]]):
        out = wave_scale(kr, origin, dests)
        check(rec, origin, dests, out)
        for di, d in enumerate(dests):
            alone = wave_scale(kr, origin, [d])
            assert torch.equal(out.occ_dest[di], alone.occ_dest[0]), d.name
            assert torch.equal(out.wave_dest[di], alone.wave_dest[0]), d.name
            assert torch.equal(out.status[di], alone.status[0]), d.name
            a, b = out.time_ns[di].cpu().numpy(), alone.time_ns[0].cpu().numpy()
            ok = ~np.isnan(b)
            # gamma above the ridge is a product here and a quotient there: last bits
            np.testing.assert_allclose(a[ok], b[ok], rtol=1e-13)
            worst = max(worst, float(np.max(np.abs(a[ok] - b[ok]) / np.abs(b[ok]))))
    print("several destinations per launch vs one: max relative time difference %.3g" % worst)


def test_every_status_and_the_short_circuit(kat):
    base = dict(kat["scaling_record"])
    rows = [
        dict(base, num_blocks=100, regs_per_thread=255, block_size=1024),              # 1
        dict(base, num_blocks=10, dynamic_smem=60000),                                 # 2 (MI355X -> V100)
        dict(base, num_blocks=1 << 16, dynamic_smem=60000),                            # 0: not evaluated
        dict(base, num_blocks=100, dram_read_bytes=-3e8),                              # 3
        dict(base, num_blocks=100, flop_sp_efficiency=float("nan")),                   # 3
        dict(base, num_blocks=0),                                                      # 4 / 0 without metrics
        dict(base, num_blocks=-5),                                                     # 0
        dict(base, num_blocks=100, flop_sp_efficiency=float("inf")),                   # gamma 0+
        dict(base, num_blocks=100, dram_read_bytes=0.0, dram_write_bytes=0.0),         # gamma 0
        dict(base, num_blocks=100, flop_sp_efficiency=0.0),                            # gamma 1
    ]
    rec = {k: np.array([r[k] for r in rows]) for k in rows[0]}
    for hm in (1, 0):
        rec["has_metrics"] = np.full(len(rows), hm, np.uint8)
        for origin, dest in ((Device.MI355X, Device.V100), (Device.V100, Device.P100)):
            out = wave_scale(KernelRecords.from_numpy(rec), origin, [dest])
            check(rec, origin, [dest], out)
    rec["has_metrics"] = np.ones(len(rows), np.uint8)
    st = wave_scale(KernelRecords.from_numpy(rec), Device.MI355X, [Device.V100]).status[0].cpu().numpy()
    assert list(st[:7]) == [1, 2, 0, 3, 3, 4, 0]


def adversarial_records(n, seed):
    """Every field drawn from a pool that mixes ordinary values with the ones a
    formula mishandles first: zeros of both signs, subnormals, huge and tiny
    magnitudes, infinities, NaN, negative and out-of-range integers."""
    rng = np.random.default_rng(seed)
    floats = np.array([0.0, -0.0, 5e-324, 1e-310, 2.3e-308, 1e-300, 1e-30, 1e-9, 0.5, 1.0, 37.5,
                       100.0, 1e5, 1e9, 1e15, 1e100, 1e300, 1.7e308, np.inf, -np.inf, np.nan,
                       -1.0, -1e-300, -1e9])
    ints = np.array([0, 1, 2, 31, 32, 33, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4096,
                     49152, 49153, 65535, 65536, 65537, 98304, 1 << 20, (1 << 20) + 1, 1 << 24,
                     (1 << 31) - 1, -(1 << 31), -1, -255, -256, -510, -511, -512])
    pick_f = lambda ordinary: np.where(rng.random(n) < 0.6, ordinary, rng.choice(floats, n))
    pick_i = lambda ordinary: np.where(rng.random(n) < 0.7, ordinary,
                                       rng.choice(ints, n)).astype(np.int32)
    return {
        "num_blocks": pick_i(np.floor(2.0 ** rng.uniform(0, 20, n))),
        "block_size": pick_i(rng.choice([64, 128, 256, 512, 1024], n)),
        "dynamic_smem": pick_i(rng.integers(0, 30000, n)),
        "static_smem": pick_i(rng.integers(0, 30000, n)),
        "regs_per_thread": pick_i(rng.integers(16, 256, n)),
        "dest_regs": np.where(rng.random(n) < 0.5, -1, pick_i(rng.integers(0, 300, n))).astype(np.int32),
        "has_metrics": (rng.random(n) < 0.8).astype(np.uint8),
        "run_time_ns": pick_f(np.floor(10.0 ** rng.uniform(3, 7, n))),
        "flop_sp_efficiency": pick_f(10.0 ** rng.uniform(-2, 2, n)),
        "dram_read_bytes": pick_f(np.floor(10.0 ** rng.uniform(3, 10, n))),
        "dram_write_bytes": pick_f(np.floor(10.0 ** rng.uniform(3, 10, n))),
    }


def test_adversarial_field_values_agree_with_the_oracle_bit_for_bit_in_status():
    """Statuses and integers exactly; times exactly where the oracle's is zero,
    infinite or NaN, else within the tolerance."""
    rec = adversarial_records(60_000, 99)
    kr = KernelRecords.from_numpy(rec)
    pairs = ((Device.V100, Device.MI355X), (Device.MI355X, Device.T4), (Device.P100, Device.V100))
    for origin, dest in pairs:
        out = wave_scale(kr, origin, [dest])
        want = olib.wave_scale(odev(origin), odev(dest), rec)
        assert np.array_equal(out.occ_origin.cpu().numpy(), want["occ_origin"])
        assert np.array_equal(out.occ_dest[0].cpu().numpy(), want["occ_dest"])
        assert np.array_equal(out.wave_dest[0].cpu().numpy(), want["wave_dest"])
        st = out.status[0].cpu().numpy()
        bad = np.flatnonzero(st != want["status"])
        assert bad.size == 0, {k: v[bad[0]] for k, v in rec.items()}
        assert len(set(st.tolist())) == 5           # every status occurs
        t, w = out.time_ns[0].cpu().numpy(), want["time_ns"]
        ok = st == 0
        assert np.all(np.isnan(t[~ok]))
        special = ok & ~(np.isfinite(w) & (w != 0))
        assert special.sum() > 100
        assert np.array_equal(t[special], w[special], equal_nan=True)
        assert np.array_equal(np.signbit(t[special]), np.signbit(w[special]))
        plain = ok & ~special
        np.testing.assert_allclose(t[plain], w[plain], rtol=TIME_RTOL, atol=0)


def test_partial_products_overflow_as_in_the_reference():
    """The reference multiplies t by its three factors from left to right, so
    1.7e308 ns * 1.07 is already inf when 0.45 follows; the kernel's single
    combined power must not return the finite product there.  Huge and ordinary
    times, every device pair, single and multi-destination launches."""
    rng = np.random.default_rng(8)
    rec, _ = synthetic.kernel_records(30_000, Device.V100, seed=41, metrics_fraction=0.8)
    rec["run_time_ns"] = np.where(rng.random(30_000) < 0.5, rec["run_time_ns"],
                                  rng.choice([1.7e308, 1e308, 4e307, 1e305, 1e200, 3.3e150,
                                              1e151, np.inf], 30_000))
    rec["dram_read_bytes"] = np.where(rng.random(30_000) < 0.3, 0.0, rec["dram_read_bytes"])
    rec["dram_write_bytes"] = np.where(rng.random(30_000) < 0.5, 0.0, rec["dram_write_bytes"])
    kr = KernelRecords.from_numpy(rec)
    names = ["RTX2070", "V100", "T4", "P4000", "P100", "MI355X"]
    devices = [getattr(Device, n) for n in names]
    n_inf_where_product_is_finite = 0
    for origin in devices:
        multi = wave_scale(kr, origin, devices)
        for d, dest in enumerate(devices):
            want = olib.wave_scale(odev(origin), odev(dest), rec)
            single = wave_scale(kr, origin, [dest])
            for out, row in ((multi, d), (single, 0)):
                st = out.status[row].cpu().numpy()
                assert np.array_equal(st, want["status"])
                t, w = out.time_ns[row].cpu().numpy(), want["time_ns"]
                ok = st == 0
                assert np.array_equal(np.isinf(t[ok]), np.isinf(w[ok])), (origin.name, dest.name)
                fin = ok & np.isfinite(w)
                np.testing.assert_allclose(t[fin], w[fin], rtol=TIME_RTOL, atol=0)
            n_inf_where_product_is_finite += int(np.sum(
                (want["status"] == 0) & np.isinf(want["time_ns"]) & np.isfinite(rec["run_time_ns"])))
    assert n_inf_where_product_is_finite > 1000
    # the hand-checked case: no bytes, gamma = 0, RTX2070 -> V100
    one = {k: v[:1].copy() for k, v in rec.items()}
    one.update(num_blocks=np.array([1 << 16], np.int32), run_time_ns=np.array([1.7e308]),
               dram_read_bytes=np.array([0.0]), dram_write_bytes=np.array([0.0]),
               has_metrics=np.array([1], np.uint8), block_size=np.array([256], np.int32),
               regs_per_thread=np.array([32], np.int32), static_smem=np.array([0], np.int32),
               dynamic_smem=np.array([0], np.int32), flop_sp_efficiency=np.array([50.0]))
    out = wave_scale(KernelRecords.from_numpy(one), Device.RTX2070, [Device.V100])
    assert out.status[0].item() == 0 and out.time_ns[0].item() == math.inf


def test_more_than_2_to_28_records_take_64_bit_offsets():
    """Above 2^28 records byte offsets no longer fit 32 bits and the kernel's
    64-bit-offset instantiation runs.  Records are generated on the GPU (19 GB of
    columns); a sample from the start, the 32-bit boundary and the ragged end
    is checked against the oracle."""
    n = (1 << 28) + 12345
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * (1 << 30):
        pytest.skip("needs 40 GB of free device memory")
    g = torch.Generator(device="cuda").manual_seed(5)
    ri = lambda lo, hi: torch.randint(lo, hi, (n,), generator=g, device="cuda", dtype=torch.int32)
    cols = {
        "num_blocks": ri(1, 1 << 20),
        "block_size": ri(1, 9) * 128,
        "dynamic_smem": ri(0, 20000), "static_smem": ri(0, 20000),
        "regs_per_thread": ri(16, 129),
    }
    for name, lo, hi in (("run_time_ns", 3.0, 7.0), ("flop_sp_efficiency", -2.0, 2.0),
                         ("dram_read_bytes", 3.0, 10.0), ("dram_write_bytes", 3.0, 10.0)):
        u = torch.rand((n,), generator=g, device="cuda", dtype=torch.float64)
        cols[name] = torch.floor(10.0 ** (lo + (hi - lo) * u)) if name != "flop_sp_efficiency" \
            else 10.0 ** (lo + (hi - lo) * u)
        del u
    kr = KernelRecords(cols)
    out = WaveScaleOutput(n, 1, kr.device, waves=False, status=True)
    # poison the outputs so that a record the kernel skipped shows
    out.time_ns.fill_(-7.0)
    out.occ_dest.fill_(-7)
    wave_scale(kr, Device.V100, [Device.MI355X], out=out)
    torch.cuda.synchronize()
    boundary = 1 << 28
    idx = torch.cat([torch.arange(0, 2000), torch.arange(boundary - 2000, boundary + 2000),
                     torch.arange(n - 2000, n),
                     torch.randint(0, n, (20000,), generator=torch.Generator().manual_seed(6))]).cuda()
    rec = {k: v[idx].cpu().numpy() for k, v in cols.items()}
    want = olib.wave_scale(odev(Device.V100), odev(Device.MI355X), rec)
    assert np.array_equal(out.occ_origin[idx].cpu().numpy(), want["occ_origin"])
    assert np.array_equal(out.occ_dest[0][idx].cpu().numpy(), want["occ_dest"])
    st = out.status[0][idx].cpu().numpy()
    assert np.array_equal(st, want["status"])
    t = out.time_ns[0][idx].cpu().numpy()
    ok = st == 0
    assert ok.sum() > 10000
    np.testing.assert_allclose(t[ok], want["time_ns"][ok], rtol=TIME_RTOL, atol=0)
    # every record was written: no poison left anywhere
    assert int((out.occ_dest == -7).sum().item()) == 0
    assert int((out.time_ns == -7.0).sum().item()) == 0


def test_golden_launch_configurations_on_all_fixture_devices(occupancy_golden):
    g, devices = occupancy_golden
    n = g["block"].shape[0]
    rng = np.random.default_rng(8)
    rec = {"num_blocks": rng.integers(1, 5000, n).astype(np.int32), "block_size": g["block"],
           "dynamic_smem": g["dyn"], "static_smem": g["stat"], "regs_per_thread": g["regs"],
           "dest_regs": g["dregs"], "run_time_ns": np.full(n, 1e5),
           "flop_sp_efficiency": np.full(n, 20.0), "dram_read_bytes": np.full(n, 1e7),
           "dram_write_bytes": np.full(n, 1e6)}
    kr = KernelRecords.from_numpy(rec)
    names = list(devices)
    dests = [DeviceProperties(name=k, **devices[k]) for k in names]
    origin = dests[names.index("V100")]
    out = wave_scale(kr, origin, dests)
    for di, name in enumerate(names):
        # occupancies straight against the reference-compiled fixture
        assert np.array_equal(out.occ_dest[di].cpu().numpy(), g["occ_lut__" + name]), name
    assert np.array_equal(out.occ_origin.cpu().numpy(), g["occ_own__V100"])
    check(rec, origin, dests, out)


def test_slow_division_path_with_huge_device_and_record_values():
    big = DeviceProperties(name="big", **dict(
        Device.V100.as_dict(), max_threads_per_block=1 << 24, max_threads_per_multiprocessor=1 << 26,
        regs_per_block=1 << 30, regs_per_multiprocessor=1 << 30,
        shared_mem_per_block=1 << 28, shared_mem_per_multiprocessor=1 << 29, warp_size=48))
    rng = np.random.default_rng(10)
    n = 4096
    rec = {"num_blocks": rng.integers(1, 1 << 30, n).astype(np.int32),
           "block_size": rng.integers(1, 1 << 24, n).astype(np.int32),
           "dynamic_smem": rng.integers(0, 1 << 27, n).astype(np.int32),
           "static_smem": rng.integers(0, 1 << 27, n).astype(np.int32),
           "regs_per_thread": rng.integers(0, 256, n).astype(np.int32),
           "run_time_ns": np.floor(10.0 ** rng.uniform(3, 7, n)),
           "flop_sp_efficiency": 10.0 ** rng.uniform(-2, 2, n),
           "dram_read_bytes": np.floor(10.0 ** rng.uniform(3, 10, n)),
           "dram_write_bytes": np.floor(10.0 ** rng.uniform(3, 10, n))}
    # ordinary limits, but more SMs than the 32-bit model's float ceiling takes
    # (2^14): the general instantiation, with wave sizes up to 2^25
    wide = DeviceProperties(name="wide", **dict(Device.V100.as_dict(), num_sms=1 << 20))
    wide2 = DeviceProperties(name="wide2", **dict(Device.T4.as_dict(), num_sms=(1 << 17) + 3))
    for origin, dest in ((big, Device.V100), (Device.V100, big), (big, big), (wide2, big)):
        out = wave_scale(KernelRecords.from_numpy(rec), origin, [dest])
        check(rec, origin, [dest], out)
    # launches that run on such devices, with block counts on both sides of their waves
    ordinary, _ = synthetic.kernel_records(n, Device.V100, seed=12, metrics_fraction=0.8)
    ordinary["num_blocks"] = rng.integers(1, 1 << 26, n).astype(np.int32)
    for origin, dest in ((wide, Device.V100), (Device.V100, wide), (wide, wide2), (wide2, wide)):
        out = wave_scale(KernelRecords.from_numpy(ordinary), origin, [dest])
        check(ordinary, origin, [dest], out)
        assert int((out.status[0] == 0).sum()) > n // 2


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 130, 255, 256, 257, 258, 386, 1023, 1025, 2050])
def test_ragged_sizes_single_and_multi_destination(n):
    rec, _ = synthetic.kernel_records(n, Device.V100, seed=n)
    dests = [Device.MI355X, Device.T4, Device.P100]
    kr = KernelRecords.from_numpy(rec)
    check(rec, Device.V100, dests[:1], wave_scale(kr, Device.V100, dests[:1]))
    check(rec, Device.V100, dests, wave_scale(kr, Device.V100, dests))


def test_roofline_gamma_alone():
    """Row a-4 on its own: gamma of every record against the oracle's Python
    (bit-identical operation order), NaN exactly where the reference asserts."""
    from habitat_amd.analysis.wave_scaling.batch import roofline_gamma
    from oracle import wave_scaling as ows
    rec = adversarial_records(20_000, 23)
    kr = KernelRecords.from_numpy(rec)
    for origin, dest in ((Device.V100, Device.MI355X), (Device.T4, Device.P100)):
        got = roofline_gamma(kr, origin, dest).cpu().numpy()
        o, d = odev(origin), odev(dest)
        n_bad = n_mid = 0
        for i in range(got.shape[0]):
            row = {k: rec[k][i].item() for k in ("run_time_ns", "flop_sp_efficiency",
                                                 "dram_read_bytes", "dram_write_bytes")}
            try:
                want = ows.gamma(row, o, d)
            except AssertionError:
                assert math.isnan(got[i]), (i, row)
                n_bad += 1
                continue
            # abs: where the reference's intensity overflows to infinity (bytes in the
            # subnormal range) its gamma is exactly 0; the kernel's single division
            # gives the true quotient, some 1e-315
            assert got[i] == pytest.approx(want, rel=1e-12, abs=1e-290), (i, row, got[i], want)
            n_mid += 0 < want < 1
        assert n_bad > 100 and n_mid > 1000
    # the scalar face, and the ridge point
    from habitat_amd.analysis.wave_scaling.roofline import _ridge_point, _roofline_gamma
    from test_api_gpu import make_kernel
    row = {k: v[5].item() for k, v in synthetic.kernel_records(8, Device.V100, seed=1)[0].items()}
    k = make_kernel(Device.V100, t_ns=int(row["run_time_ns"]),
                    metrics=(row["flop_sp_efficiency"], row["dram_read_bytes"],
                             row["dram_write_bytes"]))
    assert _roofline_gamma(k, Device.V100, Device.T4) == pytest.approx(
        ows.gamma(row, odev(Device.V100), odev(Device.T4)), rel=1e-12)
    assert _ridge_point(Device.V100) == 6716 / 739


def test_random_device_descriptions_on_the_gpu():
    """Kernel occupancies on 60 random device descriptions (odd warp sizes, huge
    and zero limits, unknown architectures), as origins and destinations,
    against the oracle, which a CPU test pins to the compiled reference on the
    same descriptions."""
    from test_oracle import random_device_specs
    specs = random_device_specs(60, 17)
    devices = [DeviceProperties(name="r%d" % i, **p) for i, p in enumerate(specs)]
    rec = adversarial_records(4000, 31)
    kr = KernelRecords.from_numpy(rec)
    for origin in (devices[0], devices[7], Device.V100):
        out = wave_scale(kr, origin, devices)
        check(rec, origin, devices, out)


def test_wave_counts_are_the_reference_quotients():
    rec = adversarial_records(5000, 17)
    kr = KernelRecords.from_numpy(rec)
    dests = [Device.MI355X, Device.T4]
    out = wave_scale(kr, Device.V100, dests)
    count_o, count_d = out.wave_counts(kr.columns["num_blocks"])
    wave_o = out.wave_origin.cpu().numpy().astype(object)
    nb = rec["num_blocks"].astype(object)
    want_o = [int(b) // int(w) if w else -1 for b, w in zip(nb, wave_o)]
    assert count_o.cpu().tolist() == want_o
    for di in range(2):
        wave_d = out.wave_dest[di].cpu().numpy().astype(object)
        assert count_d[di].cpu().tolist() == [int(b) // int(w) if w else -1
                                              for b, w in zip(nb, wave_d)]


def test_empty_input_and_no_destinations():
    rec, _ = synthetic.kernel_records(8, Device.V100, seed=0)
    empty = {k: v[:0] for k, v in rec.items()}
    out = wave_scale(KernelRecords.from_numpy(empty), Device.V100, [Device.T4])
    assert out.time_ns.shape == (1, 0)
    out = wave_scale(KernelRecords.from_numpy(rec), Device.V100, [])
    assert out.time_ns.shape == (0, 8)


def test_unaligned_columns_take_the_element_wise_kernel():
    rec, _ = synthetic.kernel_records(1001, Device.V100, seed=12)
    shifted = {}
    for k, v in rec.items():
        t = torch.from_numpy(np.concatenate([v[:1], v])).cuda()
        shifted[k] = t[1:]                       # 4- or 8-byte aligned only
        assert shifted[k].data_ptr() % 16 != 0
    kr = KernelRecords(shifted)
    out = wave_scale(kr, Device.V100, [Device.MI355X, Device.P4])
    check(rec, Device.V100, [Device.MI355X, Device.P4], out)


def test_outputs_are_optional_and_buffers_reusable():
    rec, _ = synthetic.kernel_records(4096, Device.V100, seed=13)
    kr = KernelRecords.from_numpy(rec)
    full = wave_scale(kr, Device.V100, [Device.T4])
    bare = WaveScaleOutput(4096, 1, kr.device, waves=False, status=False)
    assert bare.wave_dest is None and bare.status is None
    for _ in range(2):
        wave_scale(kr, Device.V100, [Device.T4], out=bare)
    assert torch.equal(bare.time_ns, full.time_ns)
    assert torch.equal(bare.occ_dest, full.occ_dest)
    with pytest.raises(ValueError):
        wave_scale(kr, Device.V100, [Device.T4, Device.P4], out=bare)


def test_runs_on_a_side_stream():
    rec, _ = synthetic.kernel_records(50_000, Device.V100, seed=14)
    kr = KernelRecords.from_numpy(rec)
    want = wave_scale(kr, Device.V100, [Device.T4])
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        got = wave_scale(kr, Device.V100, [Device.T4])
    s.synchronize()
    assert torch.equal(got.time_ns, want.time_ns)


def test_bad_specs_are_rejected_not_launched():
    from habitat_amd import _lib
    rec, _ = synthetic.kernel_records(16, Device.V100, seed=0)
    kr = KernelRecords.from_numpy(rec)
    zero_bw = DeviceProperties(name="z", **dict(Device.V100.as_dict(), mem_bandwidth_gb=0))
    with pytest.raises(_lib.HabitatLibraryError) as e:
        wave_scale(kr, Device.V100, [zero_bw])
    assert e.value.code == _lib.HBT_ESPEC
