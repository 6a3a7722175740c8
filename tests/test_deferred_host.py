"""CPU: the host side of the deferred strategies — how kernels are packed into
hbt_kernel_record, when pending sets begin and end, and that handing a set over
fails loudly without a GPU (there is no CPU path behind it)."""
import ctypes

import numpy as np
import pytest

from habitat_amd import Device, _lib
from habitat_amd.analysis.kernels import (RECORD_STRUCT, KernelInstance, MeasuredKernel,
                                          pack_record)
from habitat_amd.analysis.wave_scaling import deferred
from habitat_amd.analysis.wave_scaling.deferred import (
    RECORD_DTYPE, deferred_resimplified_wave_scaling, deferred_roofline_wave_scaling,
    deferred_unified_wave_scaling)
from habitat_amd.analysis.wave_scaling.metadata import NullMetadataManager


def kernel(metrics=True, name="k", regs=40, t_ns=123456):
    k = KernelInstance(name, 777, 256, 1024, 2048, regs, t_ns)
    mk = []
    if metrics:
        mk = [KernelInstance(name, 777, 256, 1024, 2048, regs, t_ns, [
            ("flop_sp_efficiency", 12.5), ("dram_read_bytes", 3e6), ("dram_write_bytes", 5e6)])]
    return MeasuredKernel(k, mk, Device.P100)


def test_packed_record_is_the_c_structure():
    assert RECORD_STRUCT.size == ctypes.sizeof(_lib.KernelRecord) == RECORD_DTYPE.itemsize == 64
    record, has = kernel().packed_record()[:2]
    c = _lib.KernelRecord.from_buffer_copy(record)
    assert has == 1
    assert (c.num_blocks, c.block_size, c.dynamic_smem, c.static_smem, c.regs, c.dest_regs,
            c.has_metrics) == (777, 256, 1024, 2048, 40, -1, 1)
    assert (c.run_time_ns, c.flop_sp_efficiency, c.dram_read_bytes, c.dram_write_bytes) == (
        123456.0, 12.5, 3e6, 5e6)
    as_numpy = np.frombuffer(record, RECORD_DTYPE)[0]
    for field, _ in _lib.KernelRecord._fields_:
        assert as_numpy[field] == getattr(c, field), field
    record, has = kernel(metrics=False).packed_record()[:2]
    c = _lib.KernelRecord.from_buffer_copy(record)
    assert has == 0 and c.has_metrics == 0 and c.flop_sp_efficiency == 0.0
    # a kernel object of another implementation, through the reference's interface only
    class Foreign:
        name, num_blocks, run_time_ns = "f", 9, 4000
        metadata = {"block_size": 64, "dynamic_shared_memory": 0, "static_shared_memory": 16,
                    "registers_per_thread": 20}

        def get_metric(self, metric, default=None):
            raise AttributeError("Unknown metric")
    c = _lib.KernelRecord.from_buffer_copy(pack_record(Foreign())[0])
    assert (c.num_blocks, c.block_size, c.static_smem, c.regs, c.has_metrics, c.run_time_ns) == (
        9, 64, 16, 20, 0, 4000.0)


def test_packed_record_is_kept_and_notices_metrics_added_later():
    mk = kernel(metrics=False)
    first = mk.packed_record()
    assert mk.packed_record() is first and first[1] == 0
    mk._metrics_kernels.append(KernelInstance("k", 777, 256, 1024, 2048, 40, 123456, [
        ("flop_sp_efficiency", 1.0), ("dram_read_bytes", 2.0), ("dram_write_bytes", 3.0)]))
    again = mk.packed_record()
    assert again[1] == 1 and _lib.KernelRecord.from_buffer_copy(again[0]).dram_write_bytes == 3.0
    assert mk.packed_record() is again


def test_pending_sets_begin_and_end_with_their_key():
    mm, other_mm = NullMetadataManager(), NullMetadataManager()
    v100, p100, t4 = Device.V100, Device.P100, Device.T4
    a = deferred_unified_wave_scaling(kernel(), v100, p100, mm)
    b = deferred_unified_wave_scaling(kernel(metrics=False), v100, p100, mm)
    assert a._set is b._set and (a._index, b._index) == (0, 1) and deferred.pending_kernels() == 2
    c = deferred_unified_wave_scaling(kernel(), v100, t4, mm)             # another destination
    d = deferred_unified_wave_scaling(kernel(), v100, t4, other_mm)       # another manager
    e = deferred_resimplified_wave_scaling(kernel(), v100, t4, other_mm)  # another strategy
    assert len({id(x._set) for x in (a, c, d, e)}) == 4
    assert deferred.pending_kernels() == 1
    # what a set hands over: call order, the strategy's view of the metrics
    rec = a._set.records()
    assert rec.shape == (2,) and list(rec["has_metrics"]) == [1, 0] and list(rec["dest_regs"]) == [-1, -1]
    assert list(e._set.records()["has_metrics"]) == [0]
    assert a.name == "k"
    with pytest.raises(AttributeError, match="Unknown metric"):
        deferred_roofline_wave_scaling(kernel(metrics=False), v100, p100, mm)

    class Table:
        def kernel_registers_for(self, k, device):
            return 99 if k.name == "gemm" else None
    t = Table()
    f = deferred_unified_wave_scaling(kernel(name="gemm"), v100, p100, t)
    deferred_unified_wave_scaling(kernel(name="other"), v100, p100, t)
    assert list(f._set.records()["dest_regs"]) == [99, -1]


def test_handing_over_fails_loudly_without_a_gpu():
    if _lib.lib().hbt_device_count() > 0:
        pytest.skip("a GPU is present")
    p = deferred_unified_wave_scaling(kernel(), Device.V100, Device.P100, NullMetadataManager())
    with pytest.raises(RuntimeError):     # torch (no HIP GPUs) or the library (HBT_EHIP)
        p.run_time_ns


def test_a_pending_set_is_closed_at_its_size_limit(monkeypatch):
    """A caller that never reads its results must not make the thread's set
    grow for ever: at MAX_PENDING kernels the set is closed and the next call
    opens another (the closed one lives as long as its results do)."""
    monkeypatch.setattr(deferred, "MAX_PENDING", 5)
    mm = NullMetadataManager()
    k = kernel()
    results = [deferred_unified_wave_scaling(k, Device.V100, Device.P100, mm) for _ in range(12)]
    sets = []
    for r in results:
        if not sets or sets[-1] is not r._set:
            sets.append(r._set)
    assert [len(s) for s in sets] == [5, 5, 2]
    assert [r._index for r in results] == [0, 1, 2, 3, 4] * 2 + [0, 1]
    assert deferred.pending_kernels() == 2
