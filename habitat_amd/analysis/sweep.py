"""Whole-trace prediction for a sweep of destination devices.

For every destination d the reference would compute (analysis/trace.py:27-36,
analysis/run_time.py:50-58, analysis/predictor.py:111-148)

    total_ms(d) = sum over wave-scaled passes p of (overhead_p + sum_k t'_k(d)) / 1e6
                + sum over MLP operations o of max(0, ms_o * pred(o, d) / pred(o, origin))
                + sum over pass-through operations of their measured time

`overhead_p = max(0, ms_p * 1e6 - sum_k t_k)` depends on the origin only, so it
is computed once on the host; the per-destination parts run on the GPU: one
multi-destination wave-scaling call over all kernel records of the trace, and
one MLP call per operation kind over (operations x destinations) rows.
"""
import numpy as np
import torch

from habitat_amd.analysis import SPECIAL_OPERATIONS
from habitat_amd.analysis.mlp.devices import get_device_features
from habitat_amd.analysis.run_time import ms_to_ns
from habitat_amd.analysis.wave_scaling.batch import wave_scale


def predict_trace_times(predictor, trace, dest_devices, device_features=None):
    """[total_ms per destination].  `device_features` optionally maps a device
    name to its four MLP features (default: the table of mlp/devices.py).  A
    destination on which the reference would raise yields NaN."""
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

    kernels, const_ms = [], 0.0
    special = {}
    for op in trace.operations:
        if op.name not in SPECIAL_OPERATIONS:
            for rt in (op.forward, op.backward):
                if rt is None:
                    continue
                overhead = ms_to_ns(rt.run_time_ms) - sum(k.run_time_ns for k in rt.kernels)
                const_ms += (0 if overhead < 0 else overhead) / 1e6
                kernels.extend(rt.kernels)
        elif op.name in P._ARGUMENTS:
            special.setdefault(op.name, []).append(op)
        else:
            const_ms += op.run_time_ms

    gpu = torch.device("cuda", torch.cuda.current_device())
    total = torch.full((D,), const_ms, dtype=torch.float64, device=gpu)
    if kernels:
        # dest_regs depends on the destination architecture: group destinations
        # whose register look-up agrees (all of them when there is no table).
        groups = {}
        for i, d in enumerate(dests):
            groups.setdefault(d.compute_capability, []).append(i)
        for idxs in groups.values():
            rec = P.records_from_kernels(kernels, dests[idxs[0]], predictor._kernel_metadata, mode)
            res = wave_scale(rec, origin, [dests[i] for i in idxs], waves=False)
            t = torch.where(res.status == 0, res.time_ns,
                            torch.full_like(res.time_ns, float("nan")))
            total[torch.tensor(idxs, device=gpu)] += t.sum(dim=1) / 1e6

    for kind, ops in special.items():
        pred = predictor._mlp(kind)
        op_feats = []
        for op in ops:
            a = P._ARGUMENTS[kind](op)
            op_feats.append([a[x] for x in pred.model.features])
        op_feats = np.asarray(op_feats, np.float64)                       # [O, F]
        dev_feats = np.asarray([feats_of(d) for d in dests] + [feats_of(origin)], np.float64)
        O = op_feats.shape[0]
        rows = np.concatenate([np.repeat(op_feats[None], D + 1, axis=0),
                               np.repeat(dev_feats[:, None], O, axis=1)], axis=2)
        y = pred.predict_batch(rows.reshape((D + 1) * O, -1)).to(torch.float64).view(D + 1, O)
        ms = torch.tensor([op.run_time_ms for op in ops], dtype=torch.float64, device=gpu)
        scaled = ms[None, :] * y[:D] / y[D:D + 1]
        total += torch.clamp(scaled, min=0.0).sum(dim=1)
    return total.cpu().tolist()
