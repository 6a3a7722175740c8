"""Batched wave scaling: structure-of-arrays kernel records in HBM, one HIP
launch per (origin, up to 8 destinations).

This is the entry the scalar strategies (roofline.py, resimplified.py,
unified.py in this package) are thin wrappers of.  It stands in for the
reference's per-kernel loop (analyzer/habitat/analysis/predictor.py:116-124).
torch is used only to own device memory and to name the stream.
"""
import ctypes

import numpy as np
import torch

from habitat_amd import _lib

INT_COLUMNS = ("num_blocks", "block_size", "dynamic_smem", "static_smem", "regs_per_thread")
F64_COLUMNS = ("run_time_ns", "flop_sp_efficiency", "dram_read_bytes", "dram_write_bytes")


class KernelRecords:
    """Kernel records as columns on one GPU.

    Columns (length n): the launch geometry and resource use of
    cpp/src/cuda/kernel.h:64-151 as int32 (`num_blocks` = grid x*y*z), the
    measured time and the three metrics of wave_scaling/roofline.py:69-71 as
    float64.  Optional: `dest_regs` (int32, < 0 = no entry in the register
    table for the destination architecture) and `has_metrics` (uint8).
    """

    def __init__(self, columns, dest_regs=None, has_metrics=None):
        n = None
        self.columns = {}
        for name in INT_COLUMNS + F64_COLUMNS:
            t = columns[name]
            want = torch.int32 if name in INT_COLUMNS else torch.float64
            if not isinstance(t, torch.Tensor) or t.dtype != want or t.dim() != 1:
                raise TypeError("column %s must be a 1-D %s tensor" % (name, want))
            if not t.is_cuda:
                raise ValueError("column %s must live on the GPU" % name)
            t = t.contiguous()
            n = t.shape[0] if n is None else n
            if t.shape[0] != n:
                raise ValueError("column %s has length %d, expected %d" % (name, t.shape[0], n))
            self.columns[name] = t
        self.n = int(n)
        self.device = self.columns["num_blocks"].device
        self.dest_regs = self._optional(dest_regs, torch.int32, "dest_regs")
        self.has_metrics = self._optional(has_metrics, torch.uint8, "has_metrics")

    def _optional(self, t, dtype, name):
        if t is None:
            return None
        if t.dtype != dtype or t.dim() != 1 or t.shape[0] != self.n or not t.is_cuda:
            raise TypeError("%s must be a 1-D %s GPU tensor of length %d" % (name, dtype, self.n))
        return t.contiguous()

    def __len__(self):
        return self.n

    @classmethod
    def from_numpy(cls, rec, device="cuda"):
        """Upload a dict of numpy columns (synchronous copy)."""
        cols = {}
        for name in INT_COLUMNS:
            cols[name] = torch.from_numpy(np.ascontiguousarray(rec[name], np.int32)).to(device)
        for name in F64_COLUMNS:
            cols[name] = torch.from_numpy(np.ascontiguousarray(rec[name], np.float64)).to(device)
        dr = rec.get("dest_regs")
        hm = rec.get("has_metrics")
        if dr is not None:
            dr = torch.from_numpy(np.ascontiguousarray(dr, np.int32)).to(device)
        if hm is not None:
            hm = torch.from_numpy(np.ascontiguousarray(hm, np.uint8)).to(device)
        return cls(cols, dr, hm)


class WaveScaleOutput:
    """Preallocated outputs of one `wave_scale` call (all on the GPU).

    time_ns, occ_dest, wave_dest, status: [n_dest, n]; occ_origin, wave_origin: [n].
    """

    def __init__(self, n, n_dest, device, waves=True, status=True):
        self.n, self.n_dest = n, n_dest
        self.time_ns = torch.empty((n_dest, n), dtype=torch.float64, device=device)
        self.occ_origin = torch.empty((n,), dtype=torch.int32, device=device)
        self.occ_dest = torch.empty((n_dest, n), dtype=torch.int32, device=device)
        self.wave_origin = torch.empty((n,), dtype=torch.int32, device=device) if waves else None
        self.wave_dest = (torch.empty((n_dest, n), dtype=torch.int32, device=device)
                          if waves else None)
        self.status = torch.empty((n_dest, n), dtype=torch.uint8, device=device) if status else None

    def wave_counts(self, num_blocks):
        """(origin [n], destination [n_dest, n]) int64 tensors of
        `num_blocks // wave_size`, the quotient the reference compares with zero
        to tell a kernel that fits one wave (wave_scaling/roofline.py:29-30),
        with Python's floor semantics; -1 where the wave size is 0 (the
        reference raises ZeroDivisionError there).  Needs the wave-size outputs."""
        if self.wave_origin is None:
            raise ValueError("allocate the output with waves=True")
        nb = num_blocks.to(torch.int64)

        def quotient(wave):
            wave = wave.to(torch.int64)
            safe = torch.where(wave == 0, torch.ones_like(wave), wave)
            q = torch.div(nb.expand_as(wave), safe, rounding_mode="floor")
            return torch.where(wave == 0, torch.full_like(q, -1), q)

        return quotient(self.wave_origin), quotient(self.wave_dest)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def wave_scale(records, origin, dests, out=None, stream=None, waves=True, status=True):
    """Scale every record from `origin` to each device in `dests`.

    `origin` and the items of `dests` are DeviceProperties.  Returns a
    WaveScaleOutput (the one passed in `out`, if any); the work is enqueued on
    `stream` (default: torch's current stream) and not synchronised.
    """
    if not isinstance(dests, (list, tuple)):
        dests = [dests]
    n_dest = len(dests)
    if out is None:
        out = WaveScaleOutput(records.n, n_dest, records.device, waves=waves, status=status)
    elif out.n != records.n or out.n_dest != n_dest:
        raise ValueError("output buffers were allocated for another shape")
    specs = (_lib.DeviceSpec * max(n_dest, 1))(*[d.spec for d in dests])
    if stream is None:
        stream = torch.cuda.current_stream(records.device)
    c = records.columns
    with torch.cuda.device(records.device):
        rc = _lib.lib().hbt_wave_scale(
            ctypes.byref(origin.spec), specs, n_dest, records.n,
            _ptr(c["num_blocks"]), _ptr(c["block_size"]), _ptr(c["dynamic_smem"]),
            _ptr(c["static_smem"]), _ptr(c["regs_per_thread"]), _ptr(records.dest_regs),
            _ptr(c["run_time_ns"]), _ptr(c["flop_sp_efficiency"]), _ptr(c["dram_read_bytes"]),
            _ptr(c["dram_write_bytes"]), _ptr(records.has_metrics),
            _ptr(out.time_ns), _ptr(out.occ_origin), _ptr(out.occ_dest), _ptr(out.wave_origin),
            _ptr(out.wave_dest), _ptr(out.status), ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_wave_scale")
    return out


class DeviceTable:
    """A sweep of destination devices resident on the GPU (`hbt_device_table`)."""

    def __init__(self, origin, dests):
        self.origin = origin
        self.dests = list(dests)
        if not self.dests:
            raise ValueError("a device table needs at least one destination")
        specs = (_lib.DeviceSpec * len(self.dests))(*[d.spec for d in self.dests])
        err = ctypes.c_int(0)
        self.torch_device = torch.device("cuda", torch.cuda.current_device())
        self.handle = _lib.lib().hbt_device_table_create(
            ctypes.byref(origin.spec), specs, len(self.dests), ctypes.byref(err))
        if not self.handle:
            raise _lib.HabitatLibraryError(err.value, "hbt_device_table_create")

    def __len__(self):
        return len(self.dests)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.lib().hbt_device_table_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def wave_scale_sum(records, table, segment=None, n_segments=1, stream=None, segment_start=None,
                   workspace=None):
    """Per destination of `table` and per segment, the sum of the scaled times
    of `records` (see hbt_wave_scale_sum).  `segment`: int32 GPU tensor [n] or
    None.  Or `segment_start`: int64 GPU tensor [n_segments + 1] when segment s
    is the run of records [segment_start[s], segment_start[s + 1]): the times
    are then added in the records' order, as the reference adds a pass's
    kernels, without floating-point atomics (hbt_wave_scale_sum_ordered; the
    scaled times pass through `workspace`, a float64 GPU tensor of n_dest x n
    elements, allocated here when not given).
    Returns (sums [n_dest, n_segments] float64, bad [n_dest] int32), both GPU
    tensors, not synchronised."""
    if records.device != table.torch_device:
        raise ValueError("records and device table live on different GPUs")
    if segment_start is not None:
        if segment is not None:
            raise ValueError("give segment or segment_start, not both")
        if (segment_start.dtype != torch.int64 or segment_start.shape != (n_segments + 1,)
                or segment_start.device != records.device):
            raise TypeError("segment_start must be an int64 GPU tensor of length %d"
                            % (n_segments + 1))
        n_dest = len(table)
        sums = torch.empty((n_dest, n_segments), dtype=torch.float64, device=records.device)
        bad = torch.empty((n_dest,), dtype=torch.int32, device=records.device)
        if workspace is None:
            workspace = torch.empty((n_dest, max(records.n, 1)), dtype=torch.float64,
                                    device=records.device)
        elif (workspace.dtype != torch.float64 or workspace.numel() < n_dest * records.n
              or workspace.device != records.device or not workspace.is_contiguous()):
            raise TypeError("workspace must be a contiguous float64 GPU tensor of at least "
                            "%d elements" % (n_dest * records.n))
        if stream is None:
            stream = torch.cuda.current_stream(records.device)
        c = records.columns
        with torch.cuda.device(records.device):
            rc = _lib.lib().hbt_wave_scale_sum_ordered(
                table.handle, records.n,
                _ptr(c["num_blocks"]), _ptr(c["block_size"]), _ptr(c["dynamic_smem"]),
                _ptr(c["static_smem"]), _ptr(c["regs_per_thread"]), _ptr(records.dest_regs),
                _ptr(c["run_time_ns"]), _ptr(c["flop_sp_efficiency"]),
                _ptr(c["dram_read_bytes"]), _ptr(c["dram_write_bytes"]),
                _ptr(records.has_metrics), _ptr(segment_start.contiguous()), n_segments,
                _ptr(workspace), _ptr(sums), _ptr(bad), ctypes.c_void_p(stream.cuda_stream))
        _lib.check(rc, "hbt_wave_scale_sum_ordered")
        return sums, bad
    if segment is not None and (segment.dtype != torch.int32 or segment.shape != (records.n,)
                                or segment.device != records.device):
        raise TypeError("segment must be an int32 GPU tensor of length %d" % records.n)
    n_dest = len(table)
    sums = torch.empty((n_dest, n_segments), dtype=torch.float64, device=records.device)
    bad = torch.empty((n_dest,), dtype=torch.int32, device=records.device)
    if stream is None:
        stream = torch.cuda.current_stream(records.device)
    c = records.columns
    with torch.cuda.device(records.device):
        rc = _lib.lib().hbt_wave_scale_sum(
            table.handle, records.n,
            _ptr(c["num_blocks"]), _ptr(c["block_size"]), _ptr(c["dynamic_smem"]),
            _ptr(c["static_smem"]), _ptr(c["regs_per_thread"]), _ptr(records.dest_regs),
            _ptr(c["run_time_ns"]), _ptr(c["flop_sp_efficiency"]), _ptr(c["dram_read_bytes"]),
            _ptr(c["dram_write_bytes"]), _ptr(records.has_metrics),
            _ptr(segment.contiguous() if segment is not None else None), n_segments,
            _ptr(sums), _ptr(bad), ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_wave_scale_sum")
    return sums, bad


def ratio_scale(pred, run_time_ms, n_dest, totals=None, want_ms=True, stream=None, op_row=None,
                clamped=None):
    """MLP-predicted operations on a sweep (see hbt_ratio_scale).  pred: float32
    GPU tensor [(n_dest + 1), n_rows] whose last row is the origin; run_time_ms:
    float64 GPU tensor [n_ops]; op_row: int32 GPU tensor [n_ops] naming each
    operation's column of pred (None: column o, n_rows == n_ops).  Returns ms
    [n_dest, n_ops] (or None), adds the per-destination sums to `totals`
    ([n_dest] float64) and the number of negative predictions replaced by 0 to
    `clamped` ([n_dest] int32) if given."""
    n_ops = run_time_ms.shape[0]
    n_rows = pred.shape[1] if pred.dim() == 2 else -1
    if pred.dtype != torch.float32 or pred.dim() != 2 or pred.shape[0] != n_dest + 1 or (
            op_row is None and n_rows != n_ops):
        raise TypeError("pred must be float32 [%d, %d]" % (n_dest + 1, n_ops))
    if op_row is not None and (op_row.dtype != torch.int32 or op_row.shape != (n_ops,)):
        raise TypeError("op_row must be int32 [%d]" % n_ops)
    if run_time_ms.dtype != torch.float64 or (totals is not None and (
            totals.dtype != torch.float64 or totals.shape != (n_dest,))):
        raise TypeError("run_time_ms and totals must be float64")
    if clamped is not None and (clamped.dtype != torch.int32 or clamped.shape != (n_dest,)):
        raise TypeError("clamped must be int32 [%d]" % n_dest)
    pred = pred.contiguous()
    out = (torch.empty((n_dest, n_ops), dtype=torch.float64, device=pred.device)
           if want_ms else None)
    if stream is None:
        stream = torch.cuda.current_stream(pred.device)
    with torch.cuda.device(pred.device):
        rc = _lib.lib().hbt_ratio_scale(
            _ptr(pred), n_dest, n_rows, _ptr(op_row.contiguous() if op_row is not None else None),
            n_ops, _ptr(run_time_ms.contiguous()), _ptr(out), _ptr(totals), _ptr(clamped),
            ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_ratio_scale")
    return out


def roofline_gamma(records, origin, dest, stream=None):
    """The roofline exponent of every record (see hbt_roofline_gamma): a float64
    GPU tensor [n], NaN where the reference's assertion on gamma fails.  Every
    record is taken to have its metrics."""
    out = torch.empty((records.n,), dtype=torch.float64, device=records.device)
    if stream is None:
        stream = torch.cuda.current_stream(records.device)
    c = records.columns
    with torch.cuda.device(records.device):
        rc = _lib.lib().hbt_roofline_gamma(
            ctypes.byref(origin.spec), ctypes.byref(dest.spec), records.n,
            _ptr(c["run_time_ns"]), _ptr(c["flop_sp_efficiency"]), _ptr(c["dram_read_bytes"]),
            _ptr(c["dram_write_bytes"]), _ptr(out), ctypes.c_void_p(stream.cuda_stream))
    _lib.check(rc, "hbt_roofline_gamma")
    return out
