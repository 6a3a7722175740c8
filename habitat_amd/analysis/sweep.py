"""Whole-trace prediction for a sweep of destination devices.

For every destination d the reference would compute (analysis/trace.py:27-36,
analysis/run_time.py:50-58, analysis/predictor.py:111-148)

    total_ms(d) = sum over wave-scaled passes p of (overhead_p + sum_k t'_k(d)) / 1e6
                + sum over MLP operations o of max(0, ms_o * pred(o, d) / pred(o, origin))
                + sum over pass-through operations of their measured time

`overhead_p = max(0, ms_p * 1e6 - sum_k t_k)` depends on the origin only, so it
is computed once on the host.  The per-destination parts run on the GPU: one
hbt_wave_scale_sum launch over all kernel records of the trace (scaled times
are summed per pass on the fly and never written out), one MLP launch per
operation kind over (destinations + origin) x operations rows, and
hbt_ratio_scale for the ratio, clamp and sum.
"""
import numpy as np
import torch

from habitat_amd.analysis import SPECIAL_OPERATIONS
from habitat_amd.analysis.mlp.devices import get_device_features
from habitat_amd.analysis.run_time import ms_to_ns
from habitat_amd.analysis.wave_scaling.batch import DeviceTable, ratio_scale, wave_scale_sum


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


def predict_trace_sweep(predictor, trace, dest_devices, device_features=None):
    from habitat_amd.analysis import predictor as P
    dests = list(dest_devices)
    D = len(dests)
    origin = trace.device
    mode = P._BUILTIN.get(predictor._wave_scaling_strategy)
    if mode is None:
        raise ValueError("device sweeps need one of the built-in wave-scaling strategies")

    def feats_of(dev):
        if device_features is not None and dev.name in device_features:
            return list(device_features[dev.name])
        return get_device_features(dev.name, ["mem", "mem_bw", "num_sm", "single"])

    res = TraceSweep()
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
    res.pass_overhead_ns = np.asarray(overheads, np.float64)
    res.pass_owner = owners

    gpu = torch.device("cuda", torch.cuda.current_device())
    total = torch.full((D,), const_ms, dtype=torch.float64, device=gpu)
    res.bad_records = torch.zeros((D,), dtype=torch.int32, device=gpu)
    n_seg = max(len(owners), 1)
    res.pass_kernel_ns = torch.zeros((D, n_seg), dtype=torch.float64, device=gpu)
    if kernels:
        seg = torch.tensor(segment, dtype=torch.int32, device=gpu)
        # The register look-up depends on the destination's architecture: one
        # launch per group of destinations that share it (one group without a table).
        groups = {}
        for i, d in enumerate(dests):
            groups.setdefault(d.compute_capability, []).append(i)
        for idxs in groups.values():
            rec = P.records_from_kernels(kernels, dests[idxs[0]], predictor._kernel_metadata, mode)
            table = DeviceTable(origin, [dests[i] for i in idxs])
            sums, bad = wave_scale_sum(rec, table, seg, n_seg)
            at = torch.tensor(idxs, device=gpu)
            res.pass_kernel_ns[at] = sums
            res.bad_records[at] = bad
        total += res.pass_kernel_ns.sum(dim=1) / 1e6
        total = torch.where(res.bad_records > 0, torch.full_like(total, float("nan")), total)

    for kind, idxs in special.items():
        pred = predictor._mlp(kind)
        ops = [trace.operations[i] for i in idxs]
        op_feats = []
        for op in ops:
            a = P._ARGUMENTS[kind](op)
            op_feats.append([a[x] for x in pred.model.features])
        op_feats = np.asarray(op_feats, np.float64)                        # [O, F]
        dev_feats = np.asarray([feats_of(d) for d in dests] + [feats_of(origin)], np.float64)
        O = op_feats.shape[0]
        rows = np.concatenate([np.repeat(op_feats[None], D + 1, axis=0),
                               np.repeat(dev_feats[:, None], O, axis=1)], axis=2)
        y = pred.predict_batch(rows.reshape((D + 1) * O, -1)).view(D + 1, O)
        ms = torch.tensor([op.run_time_ms for op in ops], dtype=torch.float64, device=gpu)
        res.special_ms[kind] = ratio_scale(y, ms, D, totals=total)
        res.special_owner[kind] = idxs
    res.total_ms = total
    return res


def predict_trace_times(predictor, trace, dest_devices, device_features=None):
    """[total_ms per destination] as a list of floats.  `device_features`
    optionally maps a device name to its four MLP features (default: the table
    of mlp/devices.py).  A destination on which the reference would raise yields
    NaN."""
    return predict_trace_sweep(predictor, trace, dest_devices, device_features).total_ms.cpu().tolist()
