"""Whole-trace prediction for a sweep of destination devices.

For every destination d the reference would compute (analysis/trace.py:27-36,
analysis/run_time.py:50-58, analysis/predictor.py:111-148)

    total_ms(d) = sum over wave-scaled passes p of (overhead_p + sum_k t'_k(d)) / 1e6
                + sum over MLP operations o of max(0, ms_o * pred(o, d) / pred(o, origin))
                + sum over pass-through operations of their measured time

`overhead_p = max(0, ms_p * 1e6 - sum_k t_k)` depends on the origin only, so it
is computed once on the host.  The per-destination parts run on the GPU: one
hbt_wave_scale_sum_ordered launch over all kernel records of the trace (scaled
times are summed per pass on the fly, in the kernels' order, and never written
out), one MLP launch per
operation kind over (destinations + origin) x distinct feature rows (a network
repeats layer shapes: ResNet-50's 53 convolutions have 23 distinct rows), and
hbt_ratio_scale for the ratio, clamp and sum.
"""
import logging

import numpy as np
import torch

from habitat_amd.analysis import SPECIAL_OPERATIONS
from habitat_amd.analysis.mlp.devices import get_device_features
from habitat_amd.analysis.run_time import ms_to_ns
from habitat_amd.analysis.wave_scaling.batch import DeviceTable, ratio_scale, wave_scale_sum

logger = logging.getLogger(__name__)


class TraceSweep:
    """Per-destination results of one trace: `total_ms` [D], and the pieces it
    is made of (GPU tensors unless noted)."""

    def __init__(self):
        self.total_ms = None        # float64 [D]
        self.pass_kernel_ns = None  # float64 [D, n_passes]: scaled kernel time per pass
        self.pass_overhead_ns = None  # numpy float64 [n_passes]
        self.pass_owner = None      # list of (operation index, 'forward' | 'backward')
        self.special_ms = {}        # kind -> float64 [D, n_ops of that kind]
        self.special_owner = {}     # kind -> list of operation indices
        self.bad_records = None     # int32 [D]: records on which the reference would raise
        self.clamped_ops = None     # int32 [D]: MLP operations predicted negative, counted as 0

    def warn_if_clamped(self):
        """The reference warns once per operation whose MLP prediction is
        negative (predictor.py:135-141); a sweep counts them on the GPU and this
        logs one line for the whole sweep.  Reads the counter back (synchronises).
        Returns the counts as a list."""
        counts = self.clamped_ops.cpu().tolist() if self.clamped_ops is not None else []
        if any(counts):
            logger.warning(
                "%d MLP-predicted operation(s) had a negative predicted run time on %d of %d "
                "devices and count as 0 ms", sum(counts), sum(1 for c in counts if c), len(counts))
        return counts


class TracePlan:
    """What a sweep needs of one trace, independent of the destinations and
    resident on the GPU: the kernel records of every wave-scaled pass with their
    pass numbers, the pass overheads, and per MLP kind the operation features
    and measured times.  Build once per trace, then `run` (or `prepare` +
    `launch`) per set of destinations."""

    def __init__(self, predictor, trace):
        from habitat_amd.analysis import predictor as P
        self.predictor = predictor
        self.origin = trace.device
        self.mode = P._BUILTIN.get(predictor._wave_scaling_strategy)
        if self.mode is None:
            raise ValueError("device sweeps need one of the built-in wave-scaling strategies")
        self.gpu = torch.device("cuda", torch.cuda.current_device())
        kernels, segment, overheads, owners = [], [], [], []
        const_ms = 0.0
        special = {}
        for idx, op in enumerate(trace.operations):
            if op.name not in SPECIAL_OPERATIONS:
                for which, rt in (("forward", op.forward), ("backward", op.backward)):
                    if rt is None:
                        continue
                    overhead = ms_to_ns(rt.run_time_ms) - sum(k.run_time_ns for k in rt.kernels)
                    overhead = 0 if overhead < 0 else overhead
                    const_ms += overhead / 1e6
                    segment.extend([len(owners)] * len(rt.kernels))
                    kernels.extend(rt.kernels)
                    overheads.append(overhead)
                    owners.append((idx, which))
            elif op.name in P._ARGUMENTS:
                special.setdefault(op.name, []).append(idx)
            else:
                const_ms += op.run_time_ms
        self.const_ms = const_ms
        self.kernels = kernels
        self.pass_overhead_ns = np.asarray(overheads, np.float64)
        self.pass_owner = owners
        self.n_seg = max(len(owners), 1)
        self.segment = (torch.tensor(segment, dtype=torch.int32, device=self.gpu)
                        if kernels else None)
        # a pass's kernels are consecutive records: pass p is the run
        # [segment_start[p], segment_start[p + 1]), summed in that order
        counts = np.bincount(np.asarray(segment, np.int64), minlength=self.n_seg)
        self.segment_start = torch.tensor(np.concatenate([[0], np.cumsum(counts)]),
                                          dtype=torch.int64, device=self.gpu)
        self._records = {}
        self.special = {}
        for kind, idxs in special.items():
            pred = predictor._mlp(kind)
            ops = [trace.operations[i] for i in idxs]
            feats = []
            for op in ops:
                a = P._ARGUMENTS[kind](op)
                feats.append([a[x] for x in pred.model.features])
            # operations with equal features share one MLP row
            uniq, op_row = np.unique(np.asarray(feats, np.float64), axis=0, return_inverse=True)
            self.special[kind] = (
                idxs, pred,
                torch.tensor(uniq, device=self.gpu),                                   # [U, F]
                torch.tensor([op.run_time_ms for op in ops], dtype=torch.float64, device=self.gpu),
                torch.tensor(op_row.reshape(-1), dtype=torch.int32, device=self.gpu))  # [O]

    def _records_for(self, dest):
        """Kernel records with the register column resolved for `dest`'s
        architecture (the look-up depends on nothing else of the destination)."""
        from habitat_amd.analysis import predictor as P
        from habitat_amd.analysis.wave_scaling.metadata import NullMetadataManager
        meta = self.predictor._kernel_metadata
        key = None if isinstance(meta, NullMetadataManager) else dest.compute_capability
        if key not in self._records:
            self._records[key] = P.records_from_kernels(self.kernels, dest, meta, self.mode)
        return self._records[key]

    def prepare(self, dest_devices, device_features=None):
        """Everything that allocates or copies for one set of destinations: the
        device-resident destination tables and the MLP device-feature rows.
        Returns a SweepCall whose `launch()` only enqueues kernels."""
        return SweepCall(self, list(dest_devices), device_features)

    def run(self, dest_devices, device_features=None):
        return self.prepare(dest_devices, device_features).launch()


class SweepCall:
    """A prepared sweep: `launch()` enqueues its kernels on the current stream
    and returns a TraceSweep of GPU tensors, without synchronising and without
    reading anything back, so it can be repeated or captured in a HIP graph.
    Launches of ONE prepared sweep must follow each other on one stream (or be
    ordered otherwise): they share the workspace the scaled times pass through
    and the side streams the networks run on."""

    def __init__(self, plan, dests, device_features):
        from habitat_amd.analysis import predictor as P
        self.plan = plan
        self.dests = dests

        def feats_of(dev):
            if device_features is not None and dev.name in device_features:
                return list(device_features[dev.name])
            return get_device_features(dev.name, ["mem", "mem_bw", "num_sm", "single"])

        self.groups = []
        if plan.kernels:
            by_arch = {}
            for i, d in enumerate(dests):
                by_arch.setdefault(d.compute_capability, []).append(i)
            whole = len(by_arch) == 1
            for idxs in by_arch.values():
                rec = plan._records_for(dests[idxs[0]])
                table = DeviceTable(P.occupancy_device(plan.origin, plan.mode),
                                    [P.occupancy_device(dests[i], plan.mode) for i in idxs])
                at = None if whole else torch.tensor(idxs, device=plan.gpu)
                # where the scaled times pass through on their way to the ordered sums
                work = torch.empty((len(idxs), max(rec.n, 1)), dtype=torch.float64,
                                   device=plan.gpu)
                self.groups.append((rec, table, at, work))
        self.streams = [torch.cuda.Stream(plan.gpu) for _ in plan.special]   # default priority
        # The MLP input rows of every kind, (destinations + origin) x distinct
        # operation rows: they depend on the plan and the destinations only, so
        # they are laid out here, once, and `launch` just runs the networks.
        self.rows = {}
        if plan.special:
            D = len(dests)
            dev_feats = torch.tensor(
                np.asarray([feats_of(d) for d in dests] + [feats_of(plan.origin)], np.float64),
                device=plan.gpu)                                                      # [D + 1, 4]
            for kind, (idxs, pred, op_feats, ms, op_row) in plan.special.items():
                U = op_feats.shape[0]
                self.rows[kind] = torch.cat(
                    [op_feats.unsqueeze(0).expand(D + 1, U, -1),
                     dev_feats.unsqueeze(1).expand(D + 1, U, 4)], dim=2).reshape((D + 1) * U, -1)

    def launch(self):
        plan, D = self.plan, len(self.dests)
        res = TraceSweep()
        res.pass_overhead_ns = plan.pass_overhead_ns
        res.pass_owner = plan.pass_owner
        # One MLP forward per kind, each on a stream of its own and enqueued
        # first: a kind with few operations fills a fraction of the GPU, so the
        # kinds run side by side, and the wave-scaling sums of the main stream
        # run beside them instead of in front of them.
        main = torch.cuda.current_stream(plan.gpu)
        preds = {}
        for (kind, (idxs, pred, op_feats, ms, op_row)), side in zip(plan.special.items(),
                                                                    self.streams):
            U = op_feats.shape[0]
            side.wait_stream(main)
            with torch.cuda.stream(side):
                y = pred.predict_batch(self.rows[kind]).view(D + 1, U)
            y.record_stream(main)
            preds[kind] = y
        total = torch.full((D,), plan.const_ms, dtype=torch.float64, device=plan.gpu)
        if self.groups:
            if len(self.groups) == 1 and self.groups[0][2] is None:
                rec, table, _, work = self.groups[0]
                res.pass_kernel_ns, res.bad_records = wave_scale_sum(
                    rec, table, n_segments=plan.n_seg, segment_start=plan.segment_start,
                    workspace=work)
            else:
                res.pass_kernel_ns = torch.zeros((D, plan.n_seg), dtype=torch.float64,
                                                 device=plan.gpu)
                res.bad_records = torch.zeros((D,), dtype=torch.int32, device=plan.gpu)
                for rec, table, at, work in self.groups:
                    sums, bad = wave_scale_sum(rec, table, n_segments=plan.n_seg,
                                               segment_start=plan.segment_start, workspace=work)
                    res.pass_kernel_ns[at] = sums
                    res.bad_records[at] = bad
            total += res.pass_kernel_ns.sum(dim=1) / 1e6
            total = torch.where(res.bad_records > 0, torch.full_like(total, float("nan")), total)
        else:
            res.pass_kernel_ns = torch.zeros((D, plan.n_seg), dtype=torch.float64, device=plan.gpu)
            res.bad_records = torch.zeros((D,), dtype=torch.int32, device=plan.gpu)
        res.clamped_ops = torch.zeros((D,), dtype=torch.int32, device=plan.gpu)
        for side in self.streams:
            main.wait_stream(side)
        for kind, (idxs, pred, op_feats, ms, op_row) in plan.special.items():
            res.special_ms[kind] = ratio_scale(preds[kind], ms, D, totals=total, op_row=op_row,
                                               clamped=res.clamped_ops)
            res.special_owner[kind] = idxs
        res.total_ms = total
        return res


def predict_trace_sweep(predictor, trace, dest_devices, device_features=None):
    return TracePlan(predictor, trace).run(dest_devices, device_features)


def predict_trace_times(predictor, trace, dest_devices, device_features=None):
    """[total_ms per destination] as a list of floats.  `device_features`
    optionally maps a device name to its four MLP features (default: the table
    of mlp/devices.py).  A destination on which the reference would raise yields
    NaN."""
    sweep = predict_trace_sweep(predictor, trace, dest_devices, device_features)
    totals = sweep.total_ms.cpu().tolist()
    sweep.warn_if_clamped()
    return totals
