"""CPU: the C-ABI library loads, exports every symbol include/habitat_mi.h
declares, and its host-side logic (device specs, host occupancy, argument
checks) behaves.  No GPU compute is attempted."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN, ROOT
from habitat_amd import Device, DeviceProperties, _lib, synthetic


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "habitat_mi.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(hbt_[a-z0-9_]+)\s*\(", header))
    assert {"hbt_wave_scale", "hbt_mlp_forward", "hbt_occupancy_host"} <= declared
    assert declared == set(_lib.exported_symbols())
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert _lib.lib().hbt_version() == _lib.ABI_VERSION
    assert _lib.strerror(0) == "ok" and "spec" in _lib.strerror(_lib.HBT_ESPEC)


def test_device_table_and_properties():
    v100 = Device.V100
    assert repr(v100) == "DeviceProperties(name=V100)"
    assert (v100.name, v100.num_sms, v100.mem_bandwidth_gb, v100.compute_capability,
            v100.base_clock_mhz, v100.peak_gflops_per_second) == ("V100", 80, 739, (7, 0), 1312, 6716)
    assert set(Device.names()) >= {"P4000", "GTX1080Ti", "RTX2070", "RTX2080Ti", "P4", "T4", "V100",
                                   "P100", "MI355X"}
    with pytest.raises(AttributeError):
        v100.num_sms = 3                      # read-only, as the pybind properties are
    with pytest.raises(KeyError):
        Device.NoSuchGPU
    kw = v100.as_dict()
    with pytest.raises(TypeError):
        DeviceProperties(name="x", **dict(kw, num_sms=80.5))
    with pytest.raises(TypeError):
        DeviceProperties(name="x", **dict(kw, shared_mem_per_block=-1))   # size_t in the reference
    with pytest.raises(TypeError):
        DeviceProperties(**kw)                # name is required


def test_host_occupancy_matches_reference_golden(occupancy_golden):
    g, devices = occupancy_golden
    rec = dict(block_size=g["block"], dynamic_smem=g["dyn"], static_smem=g["stat"],
               regs_per_thread=g["regs"])
    for name, props in devices.items():
        dev = DeviceProperties(name=name, **props)
        assert np.array_equal(synthetic.host_occupancy(dev, rec), g["occ_own__" + name]), name
        # the scalar entry, on a sample
        for i in range(0, g["block"].shape[0], 401):
            assert dev.thread_block_occupancy(int(g["block"][i]), int(g["dyn"][i]), int(g["stat"][i]),
                                              int(g["regs"][i])) == g["occ_own__" + name][i]


def test_kernel_32bit_occupancy_model_matches_reference_golden(occupancy_golden):
    """The formulation the HIP kernel runs (32-bit, closed forms for out-of-range
    fields), evaluated on the host, against the reference-compiled fixture and
    against random int32 garbage through the 64-bit host routine."""
    g, devices = occupancy_golden
    regs = np.where(g["dregs"] >= 0, g["dregs"], g["regs"]).astype(np.int32)
    rec = dict(block_size=g["block"], dynamic_smem=g["dyn"], static_smem=g["stat"],
               regs_per_thread=regs)
    rng = np.random.default_rng(17)
    n = 200_000
    wild = dict(block_size=rng.integers(-5, 3000, n).astype(np.int32),
                dynamic_smem=rng.integers(-70000, 200000, n).astype(np.int32),
                static_smem=rng.integers(-70000, 70000, n).astype(np.int32),
                regs_per_thread=rng.integers(0, 70000, n).astype(np.int32))
    wild["dynamic_smem"][::7] = rng.integers(-2**31, 2**31 - 1, wild["dynamic_smem"][::7].shape[0])
    wild["regs_per_thread"][::3] = rng.integers(0, 300, wild["regs_per_thread"][::3].shape[0])
    wild["dynamic_smem"][::2] = rng.integers(0, 50000, wild["dynamic_smem"][::2].shape[0])
    wild["static_smem"][::2] = 0
    # keep clear of the reference's signed overflow: (int)(static + dyn) + 255
    tot = ((wild["static_smem"].astype(np.int64) + wild["dynamic_smem"] + 2**31) % 2**32) - 2**31
    keep = tot <= 2**31 - 1 - 255
    wild = {k: v[keep] for k, v in wild.items()}
    for name, props in devices.items():
        dev = DeviceProperties(name=name, **props)
        assert np.array_equal(synthetic.host_occupancy(dev, rec, model32=True),
                              g["occ_lut__" + name]), name
        a = synthetic.host_occupancy(dev, wild, model32=True)
        b = synthetic.host_occupancy(dev, wild)
        assert np.array_equal(a, b), name
        assert name in ("A100like_cc80", "zero_optin_smem_block0") or (a > 0).mean() > 0.01
    huge = DeviceProperties(name="huge", **dict(Device.V100.as_dict(), regs_per_multiprocessor=1 << 30))
    with pytest.raises(_lib.HabitatLibraryError):
        synthetic.host_occupancy(huge, rec, model32=True)


def test_kernel_instance_occupancy_known_answers(kat):
    from habitat_amd.analysis.kernels import KernelInstance
    for dev, block, regs, stat, dyn, occ, _ in kat["occupancy"]:
        k = KernelInstance("k", 1, block, dyn, stat, regs, 1000)
        assert k.thread_block_occupancy(getattr(Device, dev)) == occ
    k = KernelInstance("k", 1, 256, 0, 0, 32, 1000)
    assert k.thread_block_occupancy(Device.V100, 128) == 2     # explicit register count
    assert k.thread_block_occupancy(Device.V100, -1) == 8      # negative = own
    assert k.metadata == {"name": "k", "num_blocks": 1, "block_size": 256,
                          "static_shared_memory": 0, "dynamic_shared_memory": 0,
                          "registers_per_thread": 32}


def test_spec_check_and_argument_errors():
    L = _lib.lib()
    ok = Device.V100.spec
    assert L.hbt_device_spec_check(ctypes.byref(ok)) == 0
    assert L.hbt_device_spec_check(None) == _lib.HBT_EINVAL
    for field, value in (("mem_bandwidth_gb", 0.0), ("base_clock_mhz", float("nan")),
                         ("peak_gflops", -1.0), ("warp_size", 1 << 16), ("smem_per_sm", -1),
                         ("num_sms", 1 << 27), ("num_sms", (1 << 20) + 1)):
        s = _lib.DeviceSpec.from_buffer_copy(ok)
        setattr(s, field, value)
        assert L.hbt_device_spec_check(ctypes.byref(s)) == _lib.HBT_ESPEC, field
    s = _lib.DeviceSpec.from_buffer_copy(ok)
    s.num_sms = 1 << 20
    assert L.hbt_device_spec_check(ctypes.byref(s)) == 0
    # an AMD compute-unit description may have up to 63 wave slots per CU
    amd = Device.MI355X_cdna.spec
    for slots, want in ((32, 0), (40, 0), (63, 0), (64, _lib.HBT_ESPEC)):
        s = _lib.DeviceSpec.from_buffer_copy(amd)
        s.max_threads_per_sm = slots * s.warp_size
        assert L.hbt_device_spec_check(ctypes.byref(s)) == want, slots
    # a device the occupancy model rejects is still a valid spec: occupancy 0
    s = _lib.DeviceSpec.from_buffer_copy(ok)
    s.compute_major = 8
    assert L.hbt_device_spec_check(ctypes.byref(s)) == 0
    out = ctypes.c_uint32(7)
    assert L.hbt_occupancy_host(ctypes.byref(s), 256, 0, 0, 32, ctypes.byref(out)) == 0
    assert out.value == 0
    assert L.hbt_occupancy_host(None, 256, 0, 0, 32, ctypes.byref(out)) == _lib.HBT_EINVAL
    # wave scaling: argument checks come before any GPU work
    z = None
    rc = L.hbt_wave_scale(ctypes.byref(ok), ctypes.byref(ok), 1, -1, *([z] * 17), None)
    assert rc == _lib.HBT_EINVAL
    rc = L.hbt_wave_scale(ctypes.byref(ok), ctypes.byref(ok), 1, 0, *([z] * 17), None)
    assert rc == 0                                            # nothing to do
    rc = L.hbt_wave_scale(ctypes.byref(ok), ctypes.byref(ok), 1, 4, *([z] * 17), None)
    assert rc == _lib.HBT_EINVAL                              # null columns
    err = ctypes.c_int(0)
    assert not L.hbt_mlp_create(12, 1024, 8, None, None, None, None, ctypes.byref(err))
    assert err.value == _lib.HBT_EINVAL


def test_compute_entry_fails_loudly_without_gpu():
    L = _lib.lib()
    if L.hbt_device_count() > 0:
        pytest.skip("a GPU is present")
    ok = Device.V100.spec
    buf = (ctypes.c_double * 8)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = L.hbt_wave_scale(ctypes.byref(ok), ctypes.byref(ok), 1, 1, p, p, p, p, p, None, p, p, p, p,
                          None, p, None, None, None, None, None, None)
    assert rc == _lib.HBT_EHIP


def test_synthetic_generators_are_seeded_and_respect_the_origin():
    rec, stats = synthetic.kernel_records(5000, Device.V100, seed=0)
    rec2, _ = synthetic.kernel_records(5000, Device.V100, seed=0)
    assert all(np.array_equal(rec[k], rec2[k]) for k in rec)
    assert stats["used"] == 5000 and stats["rejected"] > 0
    assert synthetic.host_occupancy(Device.V100, rec).min() >= 1
    assert rec["num_blocks"].min() >= 1 and rec["num_blocks"].max() <= 2 ** 20
    assert set(np.unique(rec["block_size"])) <= {64, 128, 256, 512, 1024}
    assert rec["run_time_ns"].min() >= 1e3 and rec["run_time_ns"].max() <= 1e7
    assert np.all(rec["run_time_ns"] == np.floor(rec["run_time_ns"]))
    devs, feats = synthetic.device_sweep(16, seed=1)
    assert len(devs) == 16 and feats.shape == (16, 4)
    assert all(40 <= d.num_sms <= 304 and 500 <= d.mem_bandwidth_gb <= 8000 for d in devs)
    for kind, f in (("conv2d", 12), ("linear", 8), ("bmm", 8), ("lstm", 11)):
        x, mu, sigma = synthetic.mlp_features(kind, 256, seed=2)
        assert x.shape == (256, f) and mu.shape == (f,) and np.all(sigma > 0)


def test_mlp_device_features_table():
    from habitat_amd.analysis.mlp import devices as md
    assert md.get_device_features("V100", ["mem", "mem_bw", "num_sm", "single"]) == [16, 900, 80, 14.028]
    assert md.get_device_features("P4000", ["single"]) == [5.3]
    with pytest.raises(IndexError):
        md.get_device_features("nope", ["mem"])
    assert set(md.get_all_devices(["mem"])) >= {"P100", "P4000", "RTX2070", "RTX2080Ti", "T4", "V100"}


def test_metrics_and_measured_kernel():
    from habitat_amd.analysis.kernels import KernelInstance, MeasuredKernel
    from habitat_amd.analysis.metrics import Metric, resolve_metrics
    k = KernelInstance("k", 10, 128, 0, 0, 32, 5000)
    m = KernelInstance("k", 10, 128, 0, 0, 32, 5000, metrics=[("dram_read_bytes", 1e6)])
    m2 = KernelInstance("k", 10, 128, 0, 0, 32, 5000, metrics=[("dram_utilization", 3.0)])
    mk = MeasuredKernel(k, [m, m2], Device.P100)
    assert mk.get_metric(Metric.DRAMReadBytes) == 1e6
    assert mk.get_metric(Metric.DRAMUtilization) == 30.0          # legacy scale on cc < 7
    assert mk.get_metric(Metric.DRAMWriteBytes, default=5.0) == 5.0
    with pytest.raises(AttributeError, match="Unknown metric: DRAMWriteBytes"):
        mk.get_metric(Metric.DRAMWriteBytes)
    assert (mk.name, mk.num_blocks, mk.run_time_ns) == ("k", 10, 5000)   # delegated
    assert resolve_metrics(Metric.DRAMReadBytes, Device.V100) == ["dram__bytes_read.sum"]
    assert resolve_metrics([Metric.DRAMReadBytes, "raw"], Device.P100) == ["dram_read_bytes", "raw"]


def test_habitat_alias_imports():
    import habitat_amd
    habitat_amd.install_as_habitat()
    from habitat.analysis.wave_scaling.common import calculate_wave_info
    from habitat.analysis.wave_scaling.metadata import MetadataManager  # noqa: F401
    from habitat.analysis.wave_scaling.resimplified import resimplified_wave_scaling  # noqa: F401
    from habitat.analysis.wave_scaling.roofline import roofline_wave_scaling  # noqa: F401
    from habitat.analysis.wave_scaling.unified import unified_wave_scaling  # noqa: F401
    from habitat.analysis.wave_scaling.deferred import deferred_unified_wave_scaling  # noqa: F401
    from habitat.analysis.mlp.mlp import RuntimePredictor, LinearMLP, LSTMMLP, Conv2DMLP, BMMMLP  # noqa: F401
    from habitat.analysis.predictor import Predictor  # noqa: F401
    from habitat.analysis.kernels import MeasuredKernel, PredictedKernel, KernelInstance
    from habitat.analysis.metrics import Metric  # noqa: F401
    from habitat.analysis.wave_scaling.metadata import NullMetadataManager
    from habitat.analysis.device import _Device  # noqa: F401
    from habitat.analysis.wave_scaling.roofline import _ridge_point
    from habitat.analysis.trace import Trace  # noqa: F401  (no data files needed to import)
    from habitat.utils import ms_to_ns, name_all_arguments, ns_to_ms
    import habitat
    assert ns_to_ms(ms_to_ns(2.5)) == 2.5
    assert name_all_arguments(["a", "b", "c"], (1, 2), {"c": 3}) == {"a": 1, "b": 2, "c": 3}
    assert _ridge_point(habitat.Device.T4) == 1804 / 239
    assert habitat.Device.V100.num_sms == 80
    k = KernelInstance("k", 4096, 256, 0, 0, 32, 1000000)
    assert calculate_wave_info(k, habitat.Device.V100, habitat.Device.P100,
                               NullMetadataManager()) == (640, 448, 8, 8)
    assert RuntimePredictor("conv2d", 8, 1024).model.features == [
        "bias", "batch", "image_size", "in_channels", "out_channels", "kernel_size", "stride",
        "padding"]


def test_metadata_manager_sqlite(tmp_path):
    import sqlite3
    from habitat_amd.analysis.kernels import KernelInstance
    from habitat_amd.analysis.wave_scaling.metadata import MetadataManager
    path = str(tmp_path / "kernels.sqlite")
    con = sqlite3.connect(path)
    con.execute("CREATE TABLE kernels (name TEXT, arch INTEGER, registers_per_thread INTEGER)")
    con.executemany("INSERT INTO kernels VALUES (?, ?, ?)",
                    [("gemm", 60, 96), ("gemm", 70, 128), ("relu", 75, 16)])
    con.commit()
    con.close()
    mm = MetadataManager(path)
    gemm = KernelInstance("gemm", 1, 256, 0, 0, 64, 1)
    relu = KernelInstance("relu", 1, 256, 0, 0, 64, 1)
    assert mm.kernel_registers_for(gemm, Device.V100) == 128
    assert mm.kernel_registers_for(gemm, Device.P4000) == 96      # nearest arch below 61
    assert mm.kernel_registers_for(gemm, Device.T4) == 128        # 70 <= 75
    assert mm.kernel_registers_for(relu, Device.V100) is None     # only a newer arch listed
    assert mm.registers_for_names(["gemm", "relu", "x"], Device.T4) == [128, 16, -1]


def test_csv_reports(tmp_path):
    import csv
    from habitat_amd.analysis import report
    from habitat_amd.analysis.arguments import Arguments
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    from habitat_amd.analysis.trace import Trace
    v100 = Device.V100
    ops = [MeasuredOperation("relu_", Arguments((), {}), RunTimeMeasurement(1.5, [], v100),
                             RunTimeMeasurement(0.25, [], v100), v100),
           MeasuredOperation("conv2d", Arguments((), {}), RunTimeMeasurement(4.0, [], v100), None, v100)]
    trace = Trace(v100, ops)
    assert trace.run_time_ms == 5.75
    p = report.record_breakdown("resnet50+16", v100, Device.T4, trace, str(tmp_path))
    assert p.endswith("resnet50+16-V100-T4-breakdown.csv")
    assert list(csv.reader(open(p))) == [["operation", "run_time_ms"], ["relu_", "1.75"], ["conv2d", "4.0"]]
    p = report.record_sweep("resnet50+16", trace, [Device.T4, Device.P100], [9.5, 7.25], str(tmp_path))
    assert p.endswith("resnet50+16-V100-e2e.csv")
    assert list(csv.reader(open(p))) == [["device", "run_time_ms"], ["V100", "5.75"], ["T4", "9.5"],
                                         ["P100", "7.25"]]


def test_bench_refuses_more_than_one_gpu():
    """One GPU per box: `bench.py --gpus N` with N above 1 exits with a message."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_nothing_in_the_product_imports_the_oracle():
    """The oracle is test infrastructure: the package must not reach for it."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    offenders = []
    for base, _, files in os.walk(os.path.join(root, "habitat_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                if "oracle" in text.replace("oracle's", ""):
                    offenders.append(os.path.join(base, f))
    assert offenders == []


def test_device_table_is_read_in_both_layouts(tmp_path, monkeypatch):
    """The shipped table is columnar; a table in the reference's layout (device
    names at the top level, one mapping each: analyzer/habitat/data/devices.yml)
    and rows written as mappings are read the same way."""
    import yaml
    import habitat_amd.data
    from habitat_amd.device import _Device, _FIELDS
    v100 = {f: getattr(Device.V100, f) for f in ("num_sms", "mem_bandwidth_gb")}
    as_mapping = dict(Device.V100.as_dict())
    assert list(as_mapping) == list(_FIELDS)
    for layout in ({"V100": as_mapping},
                   {"columns": list(_FIELDS), "devices": {"V100": as_mapping}},
                   {"columns": list(_FIELDS), "devices": {"V100": list(as_mapping.values())}}):
        path = tmp_path / "devices.yml"
        path.write_text(yaml.safe_dump(layout))
        monkeypatch.setattr(habitat_amd.data, "path_to_data", lambda name: str(path))
        table = _Device()
        assert table.names() == ["V100"]
        assert {f: getattr(table.V100, f) for f in v100} == v100
        assert table.V100.as_dict() == as_mapping


def test_prediction_from_times_matches_one_from_kernels():
    """A pass made from bare times reads like one made from PredictedKernels."""
    from habitat_amd.analysis.kernels import KernelInstance, MeasuredKernel, PredictedKernel
    from habitat_amd.analysis.run_time import RunTimePrediction
    dev = Device.V100
    measured = [MeasuredKernel(KernelInstance("k%d" % i, 10, 64, 0, 0, 32, 1000 + i), [], dev)
                for i in range(3)]
    times = [1500.25, 1001, 7.5]
    lazy = RunTimePrediction.from_times(250.5, measured, times, dev)
    eager = RunTimePrediction(250.5, [PredictedKernel(k, t) for k, t in zip(measured, times)], dev)
    assert lazy.run_time_ms == eager.run_time_ms == (250.5 + 1500.25 + 1001 + 7.5) / 1e6
    assert lazy.ktime_ns == eager.ktime_ns
    assert [k.run_time_ns for k in lazy.kernels] == times
    assert [k.name for k in lazy.kernels] == ["k0", "k1", "k2"]
    assert lazy.kernels is lazy.kernels and lazy.ktime_ns == eager.ktime_ns
    assert lazy.device is dev


def test_feature_extraction_known_answers():
    """Recorded call shapes -> MLP feature rows, against lists written by hand
    from the reference's four scalers (tests/arguments_kat.py): conv2d with
    tuple / int / keyword arguments, linear with 2, 3 and 4 input dimensions,
    bmm, both lstm overloads."""
    from arguments_kat import CASES, FEATURE_ORDER, arguments_of
    from habitat_amd.analysis import predictor as P
    from habitat_amd.analysis.mlp import mlp as M
    from habitat_amd.analysis.operation import MeasuredOperation
    from habitat_amd.analysis.run_time import RunTimeMeasurement
    classes = {"conv2d": M.Conv2DMLP, "linear": M.LinearMLP, "bmm": M.BMMMLP, "lstm": M.LSTMMLP}
    for kind, cls in classes.items():
        assert list(cls(1, 8).features) == FEATURE_ORDER[kind]
    seen = set()
    for case in CASES:
        kind, label, _, _, _, want = case
        op = MeasuredOperation(kind, arguments_of(case),
                               RunTimeMeasurement(1.0, [], Device.V100), None, Device.V100)
        named = P._ARGUMENTS[kind](op)
        assert sorted(named) == sorted(FEATURE_ORDER[kind]), label
        got = [named[x] for x in FEATURE_ORDER[kind]]
        assert got == want, (kind, label, got)
        assert all(type(v) is int for v in got), (kind, label)
        seen.add(kind)
    assert seen == set(classes)


def test_record_cache_fingerprint_sees_in_place_changes():
    """The cached record columns of a pass are reused only while nothing they
    were built from has changed: any launch field, any time, the order of the
    kernels, metrics recorded since."""
    from habitat_amd.analysis.kernels import KernelInstance
    from habitat_amd.analysis.predictor import _fingerprint
    trace = synthetic.resnet50_trace(Device.V100, batch=8, seed=3)
    passes = [rt for op in trace.operations if op.name not in ("conv2d", "linear")
              for rt in (op.forward, op.backward) if rt is not None][:12]
    base = _fingerprint(passes)
    assert _fingerprint(passes) == base
    k0, k1 = passes[0].kernels[0], passes[3].kernels[0]
    for field in ("_registers_per_thread", "_block_size", "_static_shared_memory",
                  "_dynamic_shared_memory", "_num_blocks", "_run_time_ns"):
        old = getattr(k0._c, field)
        setattr(k0._c, field, old + 1)
        assert _fingerprint(passes) != base, field
        setattr(k0._c, field, old)
        assert _fingerprint(passes) == base
    # two kernels exchange their times: every sum stays, the columns do not
    t0, t1 = k0._c._run_time_ns, k1._c._run_time_ns
    assert t0 != t1
    k0._c._run_time_ns, k1._c._run_time_ns = t1, t0
    assert _fingerprint(passes) != base
    k0._c._run_time_ns, k1._c._run_time_ns = t0, t1
    # metrics recorded after the columns were built
    k0._metrics_kernels.append(KernelInstance("m", 1, 64, 0, 0, 16, 1000, [("dram_read_bytes", 1.0)]))
    assert _fingerprint(passes) != base
    k0._metrics_kernels.pop()
    assert _fingerprint(passes) == base
    # a kernel moved from one pass to the next one
    moved = passes[0].kernels.pop()
    passes[1].kernels.insert(0, moved)
    assert _fingerprint(passes)[1] == base[1]       # the same kernels in the same order ...
    assert _fingerprint(passes) != base             # ... but other passes
    passes[1].kernels.pop(0)
    passes[0].kernels.append(moved)
    assert _fingerprint(passes) == base


def test_the_c_abi_from_plain_c99(tmp_path, built_library):
    """include/habitat_mi.h is C: a C99 program compiled with -pedantic -Werror
    links against the library and gets the host-side answers without Python."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    lib_dir = os.path.dirname(built_library)
    exe = str(tmp_path / "abi_c99")
    cmd = [gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror",
           "-I", os.path.join(ROOT, "include"), "-o", exe,
           os.path.join(ROOT, "tests", "native", "abi_c99.c"),
           "-L", lib_dir, "-lhabitat_mi", "-Wl,-rpath," + lib_dir]
    built = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert built.returncode == 0, built.stdout
    import torch
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.pathsep.join(
        [torch_lib, "/opt/rocm/lib", env.get("LD_LIBRARY_PATH", "")])
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         env=env, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout)
    assert run.stdout.startswith("ok:"), run.stdout


def test_gpu_selftest_library_builds_and_exports_its_checkers():
    """tests/native/device_arith.hip (the brute-force checkers of
    tests/test_device_arith_gpu.py) cross-compiles for gfx950 and exports every
    entry the GPU test binds; nothing is launched here."""
    import ctypes
    import subprocess
    native = os.path.join(ROOT, "tests", "native")
    subprocess.check_call(["make", "-s", "-C", native])
    lib = ctypes.CDLL(os.path.join(native, "_build", "libdevice_arith.so"))
    for name in ("arith_fast_div", "arith_ceil_div", "arith_div_const", "arith_exp2",
                 "arith_exp2_at", "arith_occupancy_lattice"):
        assert hasattr(lib, name), name
