"""The AMD compute-unit occupancy model and the cdna_wave_scaling strategy.

The reference has nothing to compare these with (its occupancy routine answers
0 for any device that is not NVIDIA compute capability 3.x-7.x), so this is
not a parity test: the rules are restated below in plain Python from the
description in include/habitat_mi.h, worked by hand for a few launches, and the
library's three implementations (host, 32-bit model, HIP kernel) are checked
against that restatement and against each other.  Wave scaling on top of the
occupancies is the oracle's, with this occupancy function injected.
"""
import ctypes

import numpy as np
import pytest

from conftest import oracle_device
from habitat_amd import Device, DeviceProperties, _lib, synthetic

CDNA = 109


def cdna_occupancy(p, block, dyn, stat, regs):
    """Work-groups per CU; `p` is a dict of DeviceProperties arguments."""
    if p["compute_major"] != CDNA:
        raise ValueError("not a compute-unit description")
    limits = ("max_threads_per_block", "max_threads_per_multiprocessor", "regs_per_block",
              "regs_per_multiprocessor", "warp_size", "shared_mem_per_block",
              "shared_mem_per_multiprocessor", "num_sms")
    if any(p[k] <= 0 for k in limits):
        return 0
    regs &= 0xFFFF
    smem = (stat + dyn) & 0xFFFFFFFF
    smem = smem - (1 << 32) if smem >= (1 << 31) else smem
    wave = p["warp_size"]
    vgprs = p["regs_per_multiprocessor"] // 4 // wave
    if not (0 < block <= p["max_threads_per_block"] and regs <= vgprs
            and 0 <= smem <= p["shared_mem_per_block"]):
        return 0
    waves = -(-block // wave)
    slots = p["max_threads_per_multiprocessor"] // wave
    per_simd = min(slots // 4, vgprs // max(-(-regs // 8) * 8, 8))
    lim = min(4 * per_simd // waves, slots if waves == 1 else 16)
    granule = 1280 if p["compute_minor"] == 5 else 512
    lds = -(-smem // granule) * granule
    if lds > 0:
        lim = min(lim, p["shared_mem_per_multiprocessor"] // lds)
    return lim


def host_batch(dev, rec, fn="hbt_occupancy_host_batch"):
    n = rec["block_size"].shape[0]
    out = np.empty(n, np.int32)
    cols = [np.ascontiguousarray(rec[k], np.int32)
            for k in ("block_size", "dynamic_smem", "static_smem", "regs_per_thread")]
    rc = getattr(_lib.lib(), fn)(ctypes.byref(dev.spec), n,
                                 *[c.ctypes.data_as(ctypes.c_void_p) for c in cols],
                                 out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    return out


def launches(n, seed):
    rng = np.random.default_rng(seed)
    rec = {"block_size": rng.choice([1, 32, 63, 64, 65, 128, 192, 256, 320, 512, 1000, 1024, 1025,
                                     0, -5], n).astype(np.int32),
           "regs_per_thread": rng.integers(0, 600, n).astype(np.int32),
           "dynamic_smem": rng.choice([0, 0, 1, 511, 512, 1279, 1280, 1281, 40000, 65536, 100000,
                                       163840, 163841, -1], n).astype(np.int32),
           "static_smem": rng.choice([0, 0, 0, 256, 4096, 49152], n).astype(np.int32)}
    return rec


@pytest.mark.parametrize("block,regs,smem,want", [
    (256, 32, 0, 8),        # 4 waves; 8 wave slots per SIMD; 32 / 4
    (1024, 128, 0, 1),      # 16 waves; 512 / 128 = 4 per SIMD; 16 / 16
    (1024, 129, 0, 0),      # 136 allocated; 3 per SIMD; 12 / 16
    (64, 16, 65536, 2),     # one wave; LDS 66 560 after rounding to 1280; 163 840 / 66 560
    (128, 8, 0, 16),        # two waves: 32 / 2, capped by the 16 work-group slots
    (64, 8, 0, 32),         # one-wave work-groups may fill every wave slot
    (64, 0, 0, 32),         # no registers still allocates one granule
    (64, 512, 0, 4),        # one wave per SIMD
    (64, 513, 0, 0),
    (1025, 16, 0, 0),
    (0, 16, 0, 0),
    (256, 64, 163840, 1),
    (256, 64, 163841, 0),
])
def test_hand_worked_launches_on_mi355x_cdna(block, regs, smem, want):
    dev = Device.MI355X_cdna
    assert cdna_occupancy(dev.as_dict(), block, smem, 0, regs) == want
    assert dev.thread_block_occupancy(block, smem, 0, regs) == want


def test_host_and_32_bit_model_follow_the_restatement():
    rec = launches(20000, 7)
    variants = [Device.MI355X_cdna.as_dict()]
    variants.append(dict(variants[0], compute_minor=4, shared_mem_per_block=65536,
                         shared_mem_per_multiprocessor=65536, num_sms=304))      # MI300X-like
    variants.append(dict(variants[0], compute_minor=0, warp_size=48))            # non power of two
    variants.append(dict(variants[0], compute_minor=0, max_threads_per_multiprocessor=2560,
                         num_sms=120))                                # 10 waves per SIMD: 40 slots
    variants.append(dict(variants[0], regs_per_multiprocessor=0))                # rejected
    for props in variants:
        dev = DeviceProperties(name="v", **props)
        want = np.array([cdna_occupancy(props, int(b), int(d), int(s), int(r)) for b, d, s, r in
                         zip(rec["block_size"], rec["dynamic_smem"], rec["static_smem"],
                             rec["regs_per_thread"])], np.int32)
        assert np.array_equal(host_batch(dev, rec), want)
        assert np.array_equal(host_batch(dev, rec, "hbt_occupancy_host_model32_batch"), want)
    assert len(set(want.tolist())) == 1 and want[0] == 0


def test_plain_compute_capability_9_stays_unknown_as_in_the_reference():
    props = dict(Device.MI355X_cdna.as_dict(), compute_major=9)
    dev = DeviceProperties(name="gfx950-as-hip-reports-it", **props)
    assert dev.thread_block_occupancy(256, 0, 0, 32) == 0
    from habitat_amd.analysis.wave_scaling.cdna import native_description
    assert native_description(dev).compute_capability == (CDNA, 5)
    assert native_description(Device.MI355X) is Device.MI355X_cdna
    assert native_description(Device.V100) is Device.V100


def _oracle_occupancy(props_of):
    from oracle import lib as olib

    def occupancy(dev, rec, regs):
        p = props_of[id(dev)]
        if p["compute_major"] == CDNA:
            return cdna_occupancy(p, rec["block_size"], rec["dynamic_smem"], rec["static_smem"],
                                  regs)
        return olib.occupancy(dev, rec["block_size"], rec["dynamic_smem"], rec["static_smem"], regs)
    return occupancy


@pytest.mark.gpu
@pytest.mark.parametrize("origin_name,dest_name", [("V100", "MI355X_cdna"), ("MI355X_cdna", "V100"),
                                                   ("MI355X_cdna", "MI355X_cdna")])
def test_kernel_scales_with_compute_unit_occupancies(origin_name, dest_name):
    import torch
    from habitat_amd.analysis.wave_scaling.batch import KernelRecords, wave_scale
    from oracle import wave_scaling as ows
    origin, dest = getattr(Device, origin_name), getattr(Device, dest_name)
    rec, _ = synthetic.kernel_records(3000, Device.V100, seed=21, metrics_fraction=0.7)
    out = wave_scale(KernelRecords.from_numpy(rec), origin, [dest])
    o, d = oracle_device(origin.as_dict()), oracle_device(dest.as_dict())
    occupancy = _oracle_occupancy({id(o): origin.as_dict(), id(d): dest.as_dict()})
    assert np.array_equal(out.occ_origin.cpu().numpy(), host_batch(origin, rec))
    assert np.array_equal(out.occ_dest[0].cpu().numpy(), host_batch(dest, rec))
    t = out.time_ns[0].cpu().numpy()
    st = out.status[0].cpu().numpy()
    n_ok = 0
    for i in range(rec["num_blocks"].shape[0]):
        row = {k: v[i].item() for k, v in rec.items()}
        want, status = ows.unified_with_status(row, o, d, has_metrics=bool(rec["has_metrics"][i]),
                                               occupancy=occupancy)
        assert st[i] == status
        if status == 0:
            assert t[i] == pytest.approx(want, rel=1e-6)
            n_ok += 1
    assert n_ok > 1000


@pytest.mark.gpu
def test_small_kernels_on_a_compute_unit_with_forty_wave_slots():
    """A CU with 10 waves per SIMD holds 40 one-wave work-groups, so a kernel
    that fits one wave there can have ceil(num_blocks / CUs) anywhere in 1..40:
    the small-kernel factor's logarithms beyond 32 (NVIDIA's block-slot limit)
    are exercised on the origin and on the destination side, through the
    straight-line instantiations, the general one and the fused sums."""
    import torch
    from habitat_amd.analysis.wave_scaling.batch import (DeviceTable, KernelRecords, wave_scale,
                                                         wave_scale_sum)
    from oracle import wave_scaling as ows
    forty = DeviceProperties(name="forty", **dict(
        Device.MI355X_cdna.as_dict(), compute_minor=0, max_threads_per_multiprocessor=2560,
        num_sms=120, mem_bandwidth_gb=1200, base_clock_mhz=1500, peak_gflops_per_second=23000))
    assert forty.thread_block_occupancy(64, 0, 0, 32) == 40
    rng = np.random.default_rng(8)
    n = 6000
    rec = {"num_blocks": rng.integers(1, 41 * 120, n).astype(np.int32),
           "block_size": rng.choice([32, 64, 64, 64, 128], n).astype(np.int32),
           "dynamic_smem": np.zeros(n, np.int32), "static_smem": np.zeros(n, np.int32),
           "regs_per_thread": rng.integers(8, 56, n).astype(np.int32),
           "run_time_ns": np.floor(10.0 ** rng.uniform(3, 7, n)),
           "flop_sp_efficiency": 10.0 ** rng.uniform(-2, 2, n),
           "dram_read_bytes": np.floor(10.0 ** rng.uniform(3, 10, n)),
           "dram_write_bytes": np.floor(10.0 ** rng.uniform(3, 10, n)),
           "has_metrics": (rng.random(n) < 0.8).astype(np.uint8)}
    big = DeviceProperties(name="bigger", **dict(forty.as_dict(), num_sms=150))
    kr = KernelRecords.from_numpy(rec)
    for origin, dests in ((forty, [big]), (big, [forty]), (forty, [Device.MI355X_cdna]),
                          (Device.V100, [forty]), (forty, [big, Device.V100])):
        out = wave_scale(kr, origin, dests)
        o = oracle_device(origin.as_dict())
        ds = [oracle_device(d.as_dict()) for d in dests]
        props = {id(o): origin.as_dict()}
        props.update({id(d): dev.as_dict() for d, dev in zip(ds, dests)})
        occupancy = _oracle_occupancy(props)
        sums, bad = wave_scale_sum(kr, DeviceTable(origin, dests))
        for di, d in enumerate(ds):
            t = out.time_ns[di].cpu().numpy()
            st = out.status[di].cpu().numpy()
            beyond = total = 0
            for i in range(n):
                row = {k: v[i].item() for k, v in rec.items()}
                want, status = ows.unified_with_status(
                    row, o, d, has_metrics=bool(rec["has_metrics"][i]), occupancy=occupancy)
                assert st[i] == status
                if status == 0:
                    assert t[i] == pytest.approx(want, rel=1e-6), row
                    total += want
                    wave_o = origin.num_sms * occupancy(o, row, row["regs_per_thread"])
                    wave_d = dests[di].num_sms * occupancy(d, row, row["regs_per_thread"])
                    nb = row["num_blocks"]
                    if nb < wave_o and nb < wave_d and max(-(-nb // origin.num_sms),
                                                           -(-nb // dests[di].num_sms)) > 32:
                        beyond += 1
            if origin is not Device.V100 and dests[di] is not Device.V100:
                assert beyond > 50, (origin.name, dests[di].name)
            assert sums[di, 0].item() == pytest.approx(total, rel=1e-9)
            assert int(bad[di].item()) == int((st != 0).sum())


@pytest.mark.gpu
def test_strategy_and_sweep_use_the_compute_unit_model():
    import torch
    from habitat_amd.analysis.mlp.mlp import RuntimePredictor
    from habitat_amd.analysis.predictor import Predictor
    from habitat_amd.analysis.wave_scaling.cdna import cdna_wave_scaling
    from habitat_amd.analysis.wave_scaling.unified import unified_wave_scaling
    trace = synthetic.resnet50_trace(Device.V100, batch=32, seed=3)
    ops = [op for op in trace.operations if op.name not in ("conv2d", "linear")][:40]
    native = Predictor(wave_scaling_strategy=cdna_wave_scaling)
    dressed = Predictor(wave_scaling_strategy=unified_wave_scaling)
    got = native.predict_operations(ops, Device.MI355X)
    # the same thing, asked for explicitly
    want = dressed.predict_operations(ops, Device.MI355X_cdna)
    assert [o.run_time_ms for o in got] == [o.run_time_ms for o in want]
    # one kernel through the scalar strategy
    k = ops[0].forward.kernels[0]
    one = cdna_wave_scaling(k, Device.V100, Device.MI355X, native._kernel_metadata)
    assert one.run_time_ns == got[0].forward.kernels[0].run_time_ns
    # the deferred form of the strategy, through the reference's loop shape: one
    # call per kernel, times read afterwards
    from habitat_amd.analysis.wave_scaling.deferred import deferred_cdna_wave_scaling
    kernels = [k for op in ops for k in op.forward.kernels]
    noted = [deferred_cdna_wave_scaling(k, Device.V100, Device.MI355X, native._kernel_metadata)
             for k in kernels]
    assert [p.run_time_ns for p in noted] == [
        k.run_time_ns for o in got for k in o.forward.kernels]
    # NVIDIA to NVIDIA is untouched
    a = native.predict_operations(ops, Device.T4)
    b = dressed.predict_operations(ops, Device.T4)
    assert [o.run_time_ms for o in a] == [o.run_time_ms for o in b]


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["nvidia_to_amd", "amd_to_nvidia", "amd_to_amd", "with_p100",
                                  "from_p100"])
def test_lean_and_general_instantiations_agree_bit_for_bit(case):
    """A launch whose origin and destinations are each of one kind (NVIDIA-rule,
    with or without a P100 among them, or AMD description) runs a kernel
    instantiation without the model's uniform branches; destinations of mixed
    kinds force the general one.  Same records, same first destination: every
    integer output and status of that destination must be identical, on ordinary
    records and on field values at and beyond the limits, and the occupancies
    must be the host routine's.  Times agree to the last bits: NaN in the same
    places, and elsewhere within 1e-13 relative, because a lean launch with
    several destinations forms gamma above the ridge point as a product with
    the record's reciprocal intensity where the others divide."""
    import torch
    from test_wave_scale_gpu import adversarial_records
    from habitat_amd import DeviceProperties
    from habitat_amd.analysis.wave_scaling.batch import (DeviceTable, KernelRecords, wave_scale,
                                                         wave_scale_sum)
    amd = Device.MI355X_cdna
    # a second AMD description: gfx942-like (64 KiB LDS, 512-byte granules, 304 CUs)
    amd2 = DeviceProperties(name="other", **dict(
        amd.as_dict(), compute_minor=2, shared_mem_per_block=65536,
        shared_mem_per_multiprocessor=65536, num_sms=304, mem_bandwidth_gb=5300,
        base_clock_mhz=2100, peak_gflops_per_second=163400))
    origin, first, other, mixer = {"nvidia_to_amd": (Device.V100, amd, amd2, Device.P100),
                                   "amd_to_nvidia": (amd, Device.V100, Device.T4, Device.P100),
                                   "amd_to_amd": (amd2, amd, amd2, Device.P100),
                                   "with_p100": (Device.V100, Device.P100, Device.T4, amd),
                                   "from_p100": (Device.P100, Device.V100, Device.P100, amd)}[case]
    ordinary, _ = synthetic.kernel_records(50_001, Device.V100, seed=5, metrics_fraction=0.8)
    for rec in (ordinary, adversarial_records(40_003, 17)):
        kr = KernelRecords.from_numpy(rec)
        lean = wave_scale(kr, origin, [first, other], waves=True)
        general = wave_scale(kr, origin, [first, mixer], waves=True)
        single = wave_scale(kr, origin, [first], waves=True)
        for out in (lean, single):
            for name in ("occ_dest", "wave_dest", "status"):
                a = getattr(out, name)[0].cpu().numpy()
                b = getattr(general, name)[0].cpu().numpy()
                assert np.array_equal(a, b), name
            a, b = out.time_ns[0].cpu().numpy(), general.time_ns[0].cpu().numpy()
            assert np.array_equal(np.isnan(a), np.isnan(b))
            same = np.isfinite(b)
            assert np.array_equal(a[~same], b[~same], equal_nan=True)      # infinities, NaN
            np.testing.assert_allclose(a[same], b[same], rtol=1e-13, atol=1e-320)
            assert np.array_equal(out.occ_origin.cpu().numpy(), general.occ_origin.cpu().numpy())
        assert np.array_equal(lean.occ_origin.cpu().numpy(), host_batch(origin, rec))
        for d, dev in enumerate((first, other)):
            asked = dict(rec)
            if "dest_regs" in rec:
                asked["regs_per_thread"] = np.where(rec["dest_regs"] >= 0, rec["dest_regs"],
                                                    rec["regs_per_thread"])
            assert np.array_equal(lean.occ_dest[d].cpu().numpy(), host_batch(dev, asked))
        # the per-segment sums take the same instantiations
        seg = torch.arange(kr.n, dtype=torch.int32, device=kr.device) // 1000
        n_seg = (kr.n + 999) // 1000
        sums_lean, bad_lean = wave_scale_sum(kr, DeviceTable(origin, [first, other]), seg, n_seg)
        sums_gen, bad_gen = wave_scale_sum(kr, DeviceTable(origin, [first, mixer]), seg,
                                           n_seg)
        assert torch.equal(bad_lean[0], bad_gen[0])
        a, b = sums_lean[0].cpu().numpy(), sums_gen[0].cpu().numpy()
        finite = np.isfinite(b)
        assert np.array_equal(np.isfinite(a), finite)
        # sums of the same terms; atomics may add the runs in another order
        np.testing.assert_allclose(a[finite], b[finite], rtol=1e-12)
