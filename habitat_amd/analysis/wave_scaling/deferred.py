"""Wave-scaling strategies with the reference's signature that cost one GPU
launch per trace instead of one per kernel.

The reference calls its strategy once per kernel
(analyzer/habitat/analysis/predictor.py:116-124) and reads the result's
`run_time_ns` only later, when a pass's time is summed
(analysis/run_time.py:50-58).  A deferred strategy uses that gap: the call
only notes the kernel in the calling thread's pending set and returns a
`DeferredPredictedKernel`; the first read of any `run_time_ns` of the set
hands the whole set to the GPU in ONE hbt_wave_scale_host_records call and
every kernel of the set has its time from then on.

    Predictor(wave_scaling_strategy=deferred_unified_wave_scaling)

(likewise deferred_roofline_, deferred_resimplified_ and deferred_cdna_wave_scaling).

What shifts against the eager strategies: the exceptions the reference raises
inside the strategy call for a kernel that cannot be scaled
(ZeroDivisionError, AssertionError) are raised by that kernel's `run_time_ns`
instead, on every read; a sum over a pass's kernels therefore stops at the same
kernel with the same exception as the reference's loop.  A missing metric
under `deferred_roofline_wave_scaling` still raises AttributeError in the call
itself.  Kernels are read when the set is handed over, not when the strategy
is called.  A pending set belongs to the thread whose calls made it: reading
its results from another thread while that thread is still adding to it is a
race.
"""
import ctypes
import threading

import numpy as np
import torch

from habitat_amd import _lib
from habitat_amd.analysis.kernels import PredictedKernel, pack_record
from habitat_amd.analysis.wave_scaling.cdna import native_description
from habitat_amd.analysis.wave_scaling.metadata import NullMetadataManager
from habitat_amd.analysis.wave_scaling.scalar import raise_for_status, read_metrics

RECORD_DTYPE = np.dtype([
    ("num_blocks", "<i4"), ("block_size", "<i4"), ("dynamic_smem", "<i4"),
    ("static_smem", "<i4"), ("regs", "<i4"), ("dest_regs", "<i4"), ("has_metrics", "<i4"),
    ("reserved", "<i4"), ("run_time_ns", "<f8"), ("flop_sp_efficiency", "<f8"),
    ("dram_read_bytes", "<f8"), ("dram_write_bytes", "<f8")])
assert RECORD_DTYPE.itemsize == ctypes.sizeof(_lib.KernelRecord) == 64

_UNIFIED, _ROOFLINE, _RESIMPLIFIED, _CDNA = "unified", "roofline", "resimplified", "cdna"
# A pending set is closed at this many kernels and the next call opens another.
MAX_PENDING = 65536


class PendingSet:
    """Kernels noted by a deferred strategy for one (origin, destination,
    metadata manager, strategy), in call order; `times` is None until the set
    has been handed to the GPU."""
    __slots__ = ("origin", "dest", "manager", "mode", "kernels", "times", "failed",
                 "model_origin", "model_dest")

    def __init__(self, origin, dest, manager, mode):
        self.origin, self.dest, self.manager, self.mode = origin, dest, manager, mode
        # the descriptions whose occupancy rules apply: under the cdna strategy an
        # AMD device's compute-unit description (the register table is still
        # asked about the device the caller named)
        self.model_origin = native_description(origin) if mode is _CDNA else origin
        self.model_dest = native_description(dest) if mode is _CDNA else dest
        self.kernels = []
        self.times = None
        self.failed = None    # {index: status} of the kernels the reference raises for

    def __len__(self):
        return len(self.kernels)

    def records(self):
        """The set as a numpy array of hbt_kernel_record."""
        kernels = self.kernels
        try:
            packed = [k.packed_record() for k in kernels]     # this package's MeasuredKernel
        except AttributeError:
            packed = [k.packed_record() if hasattr(k, "packed_record") else pack_record(k)
                      for k in kernels]
        rec = np.frombuffer(bytearray(b"".join([p[0] for p in packed])), dtype=RECORD_DTYPE)
        if self.mode == _RESIMPLIFIED:
            rec["has_metrics"] = 0
        manager = self.manager
        if not isinstance(manager, NullMetadataManager):
            if hasattr(manager, "registers_for_names"):
                regs = manager.registers_for_names([k.name for k in kernels], self.dest)
            else:
                looked = [manager.kernel_registers_for(k, self.dest) for k in kernels]
                regs = [-1 if r is None else r for r in looked]
            rec["dest_regs"] = regs
        return rec

    def flush(self):
        """Scale every kernel of the set in one call (a wait for the GPU)."""
        if self.times is not None:
            return
        n = len(self.kernels)
        rec = self.records()
        times = np.empty(n, np.float64)
        status = np.empty(n, np.uint8)
        stream = torch.cuda.current_stream()
        rc = _lib.lib().hbt_wave_scale_host_records(
            ctypes.byref(self.model_origin.spec), ctypes.byref(self.model_dest.spec), n,
            ctypes.c_void_p(rec.ctypes.data), ctypes.c_void_p(times.ctypes.data),
            ctypes.c_void_p(status.ctypes.data), None, None,
            ctypes.c_void_p(stream.cuda_stream))
        _lib.check(rc, "hbt_wave_scale_host_records")
        out = times.tolist()
        # the no-metrics strategy returns a one-wave kernel's measured time as it
        # is, an int (resimplified.py:27-31)
        for i in np.flatnonzero((rec["has_metrics"] == 0) & (times == rec["run_time_ns"])).tolist():
            out[i] = self.kernels[i].run_time_ns
        bad = np.flatnonzero(status)
        self.failed = {int(i): int(status[i]) for i in bad} if bad.size else None
        self.times = out
        if _state.pending is self:
            _state.pending = None


class DeferredPredictedKernel(PredictedKernel):
    """A PredictedKernel whose time is formed with its whole pending set on the
    first read.  Raises what the reference's strategy call raises for this
    kernel, if it does."""
    __slots__ = ("_set", "_index")

    def __init__(self, measured_kernel, pending, index):
        self._measured_kernel = measured_kernel
        self._set = pending
        self._index = index

    @property
    def run_time_ns(self):
        pending = self._set
        if pending.times is None:
            pending.flush()
        if pending.failed is not None and self._index in pending.failed:
            raise_for_status(pending.failed[self._index])
        return pending.times[self._index]


class _State(threading.local):
    pending = None


_state = _State()


def _strategy(mode, name, doc, needs_metrics=False):
    """A strategy function of the reference's signature that notes the kernel
    in the calling thread's pending set."""

    def strategy(kernel, origin_device, dest_device, metadata_manager):
        if needs_metrics:
            packed = (kernel.packed_record() if hasattr(kernel, "packed_record")
                      else pack_record(kernel))
            if not packed[1]:
                read_metrics(kernel)     # raises the reference's AttributeError
        pending = _state.pending
        if (pending is None or pending.times is not None or pending.dest is not dest_device
                or pending.origin is not origin_device or pending.manager is not metadata_manager
                or pending.mode is not mode or len(pending.kernels) >= MAX_PENDING):
            # another set begins; the one before is handed over when one of its
            # kernels is read (and is garbage once its results are dropped: a
            # caller that never reads leaves at most MAX_PENDING kernels behind)
            pending = _state.pending = PendingSet(origin_device, dest_device, metadata_manager,
                                                  mode)
        kernels = pending.kernels
        kernels.append(kernel)
        return DeferredPredictedKernel(kernel, pending, len(kernels) - 1)

    strategy.__name__ = strategy.__qualname__ = name
    strategy.__doc__ = doc
    return strategy


deferred_unified_wave_scaling = _strategy(
    _UNIFIED, "deferred_unified_wave_scaling",
    "unified_wave_scaling (wave_scaling/unified.py:8-35), deferred.")
deferred_resimplified_wave_scaling = _strategy(
    _RESIMPLIFIED, "deferred_resimplified_wave_scaling",
    "resimplified_wave_scaling (wave_scaling/resimplified.py:7-40), deferred.")
deferred_roofline_wave_scaling = _strategy(
    _ROOFLINE, "deferred_roofline_wave_scaling",
    "roofline_wave_scaling (wave_scaling/roofline.py:8-65), deferred.  A kernel without its "
    "metrics raises AttributeError in the call, as there.", needs_metrics=True)


deferred_cdna_wave_scaling = _strategy(
    _CDNA, "deferred_cdna_wave_scaling",
    "cdna_wave_scaling (unified wave scaling with AMD devices judged by the compute-unit "
    "occupancy rules; no counterpart in the reference), deferred.")


def pending_kernels():
    """Kernels noted by this thread and not yet handed to the GPU."""
    pending = _state.pending
    return len(pending) if pending is not None and pending.times is None else 0


def flush():
    """Hand this thread's pending set to the GPU now (reads do that by
    themselves; this is for callers that want the wait at a chosen point)."""
    pending = _state.pending
    if pending is not None and pending.times is None and len(pending):
        pending.flush()
