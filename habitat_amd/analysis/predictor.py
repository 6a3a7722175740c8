"""Routes each operation of a trace to wave scaling or to an MLP and assembles
the predicted run times (analyzer/habitat/analysis/predictor.py:53-283).

The reference predicts one kernel and one operation at a time.  Here
`predict_operation` keeps that interface, while `predict_operations` and
`predict_trace_times` gather every kernel record (resp. every MLP feature row)
of a trace and hand them to the GPU in one call each.
"""
import collections
import functools
import itertools
import logging
import operator
import os

import numpy as np
import torch

from habitat_amd.analysis import SPECIAL_OPERATIONS
from habitat_amd.analysis.metrics import Metric
from habitat_amd.analysis.mlp.devices import get_device_features
from habitat_amd.analysis.mlp.mlp import RuntimePredictor
from habitat_amd.analysis.operation import PredictedOperation
from habitat_amd.analysis.run_time import (RunTimePrediction, RunTimePurePrediction, ms_to_ns)
from habitat_amd.analysis.wave_scaling.batch import KernelRecords, wave_scale
from habitat_amd.analysis.wave_scaling.cdna import cdna_wave_scaling, native_description
from habitat_amd.analysis.wave_scaling.metadata import MetadataManager, NullMetadataManager
from habitat_amd.analysis.wave_scaling.resimplified import resimplified_wave_scaling
from habitat_amd.analysis.wave_scaling.roofline import roofline_wave_scaling
from habitat_amd.analysis.wave_scaling.scalar import kernel_fields, raise_for_status
from habitat_amd.analysis.wave_scaling.unified import unified_wave_scaling
from habitat_amd.data import path_to_data

logger = logging.getLogger(__name__)

# Positional parameter names of the torch callables whose arguments were recorded.
CONV2D_PARAMS = ["input", "weight", "bias", "stride", "padding", "dilation", "groups"]
LINEAR_PARAMS = ["input", "weight", "bias"]
BMM_PARAMS = ["input", "mat2", "out"]
MATMUL_PARAMS = ["input", "other", "out"]   # defined and unused in the reference too (predictor.py:50)
LSTM_PARAMS_NO_BATCH_SIZES = ["input", "hx", "flat_weights", "bias", "num_layers", "dropout",
                              "training", "bidirectional", "batch_first"]
LSTM_PARAMS = ["input", "batch_sizes", "hx", "flat_weights", "bias", "num_layers", "dropout",
               "training", "bidirectional"]

_METRICS = (Metric.SinglePrecisionFLOPEfficiency, Metric.DRAMReadBytes, Metric.DRAMWriteBytes)
_MLP_KINDS = ("conv2d", "lstm", "linear", "bmm")


def name_all_arguments(all_parameters, args, kwargs):
    """Positional and keyword arguments merged under the declared parameter
    names (analyzer/habitat/utils.py:54-63)."""
    merged = dict(kwargs)
    for arg_name, arg in zip(all_parameters, args):
        merged[arg_name] = arg
    return merged


def _first(value):
    return value[0] if isinstance(value, tuple) else value


def conv2d_arguments(operation):
    """predictor.py:150-173"""
    m = name_all_arguments(CONV2D_PARAMS, operation.arguments.args, operation.arguments.kwargs)
    return dict(batch=m["input"][0], image_size=m["input"][2], in_channels=m["input"][1],
                out_channels=m["weight"][0], kernel_size=m["weight"][2],
                stride=_first(m["stride"]), padding=_first(m["padding"]),
                bias=(1 if m["bias"] is not None else 0))


def linear_arguments(operation):
    """predictor.py:184-211: the batch is the product of all leading dimensions."""
    m = name_all_arguments(LINEAR_PARAMS, operation.arguments.args, operation.arguments.kwargs)
    return dict(batch=functools.reduce(operator.mul, m["input"][:-1]),
                in_features=m["weight"][1], out_features=m["weight"][0],
                bias=(1 if m["bias"] is not None else 0))


def bmm_arguments(operation):
    """predictor.py:220-232"""
    m = name_all_arguments(BMM_PARAMS, operation.arguments.args, operation.arguments.kwargs)
    return dict(batch=m["input"][0], left=m["input"][1], middle=m["input"][2],
                right=m["mat2"][2])


def lstm_arguments(operation):
    """predictor.py:240-276: the packed-sequence overload has a bool in position 4."""
    args = operation.arguments.args
    if not isinstance(args[4], bool):
        m = name_all_arguments(LSTM_PARAMS_NO_BATCH_SIZES, args, operation.arguments.kwargs)
        batch, seq_len, input_size = m["input"][1], m["input"][0], m["input"][2]
    else:
        m = name_all_arguments(LSTM_PARAMS, args, operation.arguments.kwargs)
        batch = max(operation.arguments.special["batch_sizes"])
        seq_len, input_size = m["input"][0] // batch, m["input"][1]
    return dict(bias=(1 if m["bias"] is not None else 0),
                bidirectional=(1 if m["bidirectional"] else 0), batch=batch, seq_len=seq_len,
                input_size=input_size, hidden_size=m["hx"][0][2], num_layers=m["num_layers"])


_ARGUMENTS = {"conv2d": conv2d_arguments, "linear": linear_arguments, "bmm": bmm_arguments,
              "lstm": lstm_arguments}

_BUILTIN = {unified_wave_scaling: "unified", roofline_wave_scaling: "roofline",
            resimplified_wave_scaling: "resimplified", cdna_wave_scaling: "cdna"}


def occupancy_device(device, mode):
    """The description whose occupancy rules `mode` applies to `device`."""
    return native_description(device) if mode == "cdna" else device


def records_from_kernels(kernels, dest_device, metadata_manager, mode="unified", device=None):
    """Python kernel objects -> KernelRecords on the GPU (one upload)."""
    n = len(kernels)
    fields = list(zip(*[kernel_fields(k) for k in kernels])) if n else [()] * 6
    metrics = [(0.0, 0.0, 0.0)] * n
    has = [0] * n
    if mode != "resimplified":
        for i, k in enumerate(kernels):
            try:
                metrics[i] = [k.get_metric(m) for m in _METRICS]
                has[i] = 1
            except AttributeError:
                if mode == "roofline":
                    raise
    ints = [np.array(fields[j], np.int32) for j in range(5)]
    f64 = [np.array(fields[5], np.float64)] + [
        np.array(col, np.float64) for col in (zip(*metrics) if n else [(), (), ()])]
    has = np.array(has, np.uint8)
    if hasattr(metadata_manager, "registers_for_names"):
        dest_regs = metadata_manager.registers_for_names([k.name for k in kernels], dest_device)
    else:
        looked = [metadata_manager.kernel_registers_for(k, dest_device) for k in kernels]
        dest_regs = [-1 if r is None else r for r in looked]
    rec = {"num_blocks": ints[0], "block_size": ints[1], "dynamic_smem": ints[2],
           "static_smem": ints[3], "regs_per_thread": ints[4], "run_time_ns": f64[0],
           "flop_sp_efficiency": f64[1], "dram_read_bytes": f64[2], "dram_write_bytes": f64[3],
           "dest_regs": np.asarray(dest_regs, np.int32), "has_metrics": has}
    return KernelRecords.from_numpy(rec, device=device or "cuda")


# a MeasuredKernel's launch_fields() without the two Python calls: one C-level
# getter per kernel (kernel objects of another implementation lack these
# names and take the AttributeError path of _fingerprint)
_LAUNCH_FIELDS = operator.attrgetter(
    "_c._num_blocks", "_c._block_size", "_c._dynamic_shared_memory", "_c._static_shared_memory",
    "_c._registers_per_thread", "_c._run_time_ns")
_RAW_METRICS = operator.attrgetter("_metrics_kernels")


def _fingerprint(passes):
    """What the cached record columns of `passes` were built from: every
    kernel's launch fields and measured time (a hash over the tuples, so a
    changed block size, register count, shared-memory size, block count or time
    is seen, and so is a swap of two kernels), how many kernels each pass
    holds (a kernel moved to a neighbouring pass changes both overheads), the number of raw metric entries
    behind each kernel (metrics recorded since are seen; a metric already read
    is cached by the kernel object for good, as in the reference, so its value
    cannot change under the cache) and the passes' own times.  About 0.3 ms for
    900 kernels, a fraction of what converting and uploading them takes."""
    kernels = list(itertools.chain.from_iterable(p.kernels for p in passes))
    try:
        fields = hash(tuple(map(_LAUNCH_FIELDS, kernels)))
        metrics = sum(len(m.metrics) for ms in map(_RAW_METRICS, kernels) for m in ms)
    except AttributeError:       # kernel objects of another implementation
        fields = hash(tuple(kernel_fields(k) for k in kernels))
        metrics = -1
    return (tuple(len(p.kernels) for p in passes), fields, metrics,
            sum(p.run_time_ms for p in passes))


class Predictor:
    _RECORD_CACHE_SETS = 8

    def __init__(self, kernel_metadata_file=None, wave_scaling_strategy=unified_wave_scaling,
                 mlp_predictors=None):
        """`kernel_metadata_file`: sqlite register table (default: data/kernels.sqlite
        if present, else no table).  `mlp_predictors`: {'conv2d'|'lstm'|'linear'|'bmm':
        RuntimePredictor}; missing ones are loaded from data/<kind>/model.pth when
        that file exists and are otherwise left without weights."""
        default_lut = path_to_data("kernels.sqlite")
        if kernel_metadata_file is not None:
            self._kernel_metadata = MetadataManager(kernel_metadata_file)
        elif os.path.exists(default_lut):
            self._kernel_metadata = MetadataManager(default_lut)
        else:
            self._kernel_metadata = NullMetadataManager()
        self._wave_scaling_strategy = wave_scaling_strategy
        self._record_cache = collections.OrderedDict()

        mlp_predictors = dict(mlp_predictors or {})
        for kind in _MLP_KINDS:
            if kind not in mlp_predictors:
                path = path_to_data("%s/model.pth" % kind)
                mlp_predictors[kind] = RuntimePredictor(
                    kind, 8, 1024, path if os.path.exists(path) else None)
        self.linear_pred = mlp_predictors["linear"]
        self.lstm_pred = mlp_predictors["lstm"]
        self.conv2d_pred = mlp_predictors["conv2d"]
        self.bmm_pred = mlp_predictors["bmm"]

    def _mlp(self, kind):
        return getattr(self, kind + "_pred")

    # ------------------------------------------------------------------ one op
    def predict_operation(self, operation, dest_device):
        return self.predict_operations([operation], dest_device)[0]

    # ------------------------------------------------------------- many ops
    def predict_operations(self, operations, dest_device):
        """[PredictedOperation] for `operations`, with one wave-scaling launch
        for all their kernels and one MLP launch per operation kind."""
        results = [None] * len(operations)
        scaled, special = [], {}
        for i, op in enumerate(operations):
            if op.name not in SPECIAL_OPERATIONS:
                scaled.append(i)
            elif op.name in _ARGUMENTS:
                special.setdefault(op.name, []).append(i)
            else:
                logger.warning("Unhandled special operation: %s", op.name)
                results[i] = PredictedOperation(op, op.forward, op.backward, dest_device)

        # The MLP launches go first and are read back last, so that the GPU runs
        # them while the host assembles the wave-scaled passes.
        pending = [(idxs, [operations[i] for i in idxs]) for idxs in special.values()]
        pending = [(idxs, ops, self._special_enqueue(ops[0].name, ops, dest_device))
                   for idxs, ops in pending]

        if scaled:
            passes = []  # (op index, is_backward, run_time)
            for i in scaled:
                op = operations[i]
                passes.append((i, False, op.forward))
                if op.backward is not None:
                    passes.append((i, True, op.backward))
            predicted = self._wave_scale_passes([p[2] for p in passes], dest_device)
            fwd, bwd = {}, {}
            for (i, is_bwd, _), pred in zip(passes, predicted):
                (bwd if is_bwd else fwd)[i] = pred
            for i in scaled:
                results[i] = PredictedOperation(operations[i], fwd[i], bwd.get(i), dest_device)

        for idxs, ops, y in pending:
            for i, ms in zip(idxs, self._special_finish(ops, y)):
                results[i] = PredictedOperation(
                    operations[i], RunTimePurePrediction(ms, dest_device), None, dest_device)
        return results

    def _wave_scale(self, run_time, dest_device):
        return self._wave_scale_passes([run_time], dest_device)[0]

    def _wave_scale_passes(self, run_times, dest_device):
        """predictor.py:111-130 for several passes at once."""
        mode = _BUILTIN.get(self._wave_scaling_strategy)
        out = []
        if mode is None:
            # A caller-supplied strategy: one call per kernel, as in the reference.
            for rt in run_times:
                preds = [self._wave_scaling_strategy(k, rt.device, dest_device,
                                                     self._kernel_metadata) for k in rt.kernels]
                out.append(self._assemble(rt, preds, dest_device))
            return out

        # Group passes by origin device; one launch per origin.
        by_origin = {}
        for idx, rt in enumerate(run_times):
            by_origin.setdefault(rt.device.name, (rt.device, []))[1].append(idx)
        out = [None] * len(run_times)
        for origin, idxs in by_origin.values():
            passes = [run_times[idx] for idx in idxs]
            rec, measured_ns, overheads_ns = self._records_of(passes, dest_device, mode)
            t = []
            if measured_ns:
                res = wave_scale(rec, occupancy_device(origin, mode),
                                 [occupancy_device(dest_device, mode)], waves=False)
                t = res.time_ns[0].cpu().tolist()
                st = res.status[0].cpu().numpy()
                if st.any():
                    raise_for_status(int(st[np.flatnonzero(st)[0]]))
                # an unchanged time keeps the measured value's own type (an int)
                t = [m if v == m else v for m, v in zip(measured_ns, t)]
            pos = 0
            for idx, rt, overhead_ns in zip(idxs, passes, overheads_ns):
                ks = rt.kernels
                out[idx] = RunTimePrediction.from_times(overhead_ns, ks, t[pos:pos + len(ks)],
                                                        dest_device)
                pos += len(ks)
        return out

    def _records_of(self, passes, dest_device, mode):
        """(kernel records of `passes` as columns on the GPU, the kernels'
        measured times, each pass's overhead).  The last few sets are kept, so
        that predicting one trace for one destination after another converts
        and uploads its kernels once.  A set is recognised by the identity of
        its passes AND a fingerprint of what they hold (`_fingerprint`): a pass
        whose kernels were replaced, added to, or given other times or block
        counts since is converted afresh, as the reference reads every kernel
        on every call (predictor.py:111-130).  The register column depends on
        the destination's architecture only."""
        lut = not isinstance(self._kernel_metadata, NullMetadataManager)
        key = (tuple(id(p) for p in passes), mode, dest_device.compute_capability if lut else None,
               torch.cuda.current_device())
        mark = _fingerprint(passes)
        hit = self._record_cache.get(key)
        if hit is not None and hit[4] == mark:
            self._record_cache.move_to_end(key)
            return hit[:3]
        kernels = [k for p in passes for k in p.kernels]
        rec = (records_from_kernels(kernels, dest_device, self._kernel_metadata, mode)
               if kernels else None)
        measured_ns = [k.run_time_ns for k in kernels]
        overheads_ns = [self._overhead_ns(p) for p in passes]
        # the passes stay alive with their ids
        self._record_cache[key] = (rec, measured_ns, overheads_ns, list(passes), mark)
        self._record_cache.move_to_end(key)
        while len(self._record_cache) > self._RECORD_CACHE_SETS:
            self._record_cache.popitem(last=False)
        return rec, measured_ns, overheads_ns

    def clear_record_cache(self):
        """Forget the cached kernel-record columns (only needed for kernel
        objects of another implementation whose metrics were changed in place:
        for those the fingerprint covers launch fields and times only)."""
        self._record_cache.clear()

    @staticmethod
    def _overhead_ns(run_time):
        """What a measured pass took beyond its kernels, never negative
        (predictor.py:126-130)."""
        overhead_ns = ms_to_ns(run_time.run_time_ms) - sum(k.run_time_ns for k in run_time.kernels)
        return 0 if overhead_ns < 0 else overhead_ns

    @classmethod
    def _assemble(cls, run_time, predicted_kernels, dest_device):
        return RunTimePrediction(overhead_ns=cls._overhead_ns(run_time),
                                 predicted_kernels=predicted_kernels, device=dest_device)

    def _special_scale_many(self, kind, operations, dest_device):
        """predictor.py:132-148 and the four scalers (:150-283), batched: one MLP
        launch evaluates every operation on its origin and on the destination."""
        return self._special_finish(operations,
                                    self._special_enqueue(kind, operations, dest_device))

    def _special_enqueue(self, kind, operations, dest_device):
        """The MLP launch of _special_scale_many.  Operations with equal features
        and origin share their two rows (destination, origin); returns (the
        launch's output, still on the GPU, and each operation's row pair)."""
        pred = self._mlp(kind)
        rows, pair_of, pairs = [], {}, []
        dest_feats = get_device_features(dest_device.name, pred.device_params)
        for op in operations:
            a = _ARGUMENTS[kind](op)
            feats = [a[x] for x in pred.model.features]
            key = (tuple(feats), op.device.name)
            if key not in pair_of:
                pair_of[key] = len(rows) // 2
                rows.append(feats + dest_feats)
                rows.append(feats + get_device_features(op.device.name, pred.device_params))
            pairs.append(pair_of[key])
        return pred.predict_batch(np.asarray(rows, np.float64)), pairs

    @staticmethod
    def _special_finish(operations, enqueued):
        """Measured time x predicted destination time / predicted origin time,
        not below zero (predictor.py:132-148)."""
        y, pairs = enqueued
        y = y.cpu().numpy().astype(np.float64)
        out = []
        for op, i in zip(operations, pairs):
            ms = op.run_time_ms * float(y[2 * i]) / float(y[2 * i + 1])
            if ms < 0:
                logger.warning("Operation %s predicted run time %.2f ms", op.name, ms)
                ms = 0.
            out.append(ms)
        return out

    # scalar faces kept for callers of the reference's private helpers
    def _special_scale(self, operation, dest_device, scaler):
        ms = scaler(operation, dest_device)
        if ms < 0:
            logger.warning("Operation %s predicted run time %.2f ms", operation.name, ms)
            ms = 0.
        return PredictedOperation(operation, RunTimePurePrediction(ms, dest_device), None,
                                  dest_device)

    def _scale_with(self, kind, operation, dest_device):
        pred = self._mlp(kind)
        a = _ARGUMENTS[kind](operation)
        feats = [a[x] for x in pred.model.features]
        pred_dest = pred.predict(feats, dest_device.name)
        pred_orig = pred.predict(feats, operation.device.name)
        return operation.run_time_ms * pred_dest / pred_orig

    def _conv2d_scale(self, operation, dest_device):
        return self._scale_with("conv2d", operation, dest_device)

    def _linear_scale(self, operation, dest_device):
        return self._scale_with("linear", operation, dest_device)

    def _bmm_scale(self, operation, dest_device):
        return self._scale_with("bmm", operation, dest_device)

    def _lstm_scale(self, operation, dest_device):
        return self._scale_with("lstm", operation, dest_device)

    # ------------------------------------------------------- device sweeps
    def predict_trace_times(self, trace, dest_devices, device_features=None):
        """Predicted iteration time [ms] of `trace` on every device of
        `dest_devices` (the sum of analysis/trace.py:27-36 over predicted
        operations).  Kernel records are scaled for all destinations at once."""
        from habitat_amd.analysis.sweep import predict_trace_times
        return predict_trace_times(self, trace, dest_devices, device_features)

    def predict_trace_sweep(self, trace, dest_devices, device_features=None):
        """Like predict_trace_times, with the per-pass and per-operation pieces
        (a habitat_amd.analysis.sweep.TraceSweep)."""
        from habitat_amd.analysis.sweep import predict_trace_sweep
        return predict_trace_sweep(self, trace, dest_devices, device_features)

    def plan_trace(self, trace):
        """The destination-independent part of a sweep, resident on the GPU (a
        habitat_amd.analysis.sweep.TracePlan): build it once per trace, then
        `plan.run(dest_devices)` per set of destinations, or
        `plan.prepare(dest_devices).launch()` to repeat or graph-capture the
        GPU work."""
        from habitat_amd.analysis.sweep import TracePlan
        return TracePlan(self, trace)
