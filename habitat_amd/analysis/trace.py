"""An iteration trace: the operations measured on one device, and its
prediction for another (analyzer/habitat/analysis/trace.py:5-51).

Unlike the reference, importing this module needs no data files: the default
predictor is built on first use.
"""
from habitat_amd.analysis.operation import MeasuredOperation
from habitat_amd.analysis.predictor import Predictor


class _LazyDefaultPredictor:
    """`Trace.DefaultPredictor` (analysis/trace.py:11), built when first read."""

    def __get__(self, instance, owner):
        return owner.default_predictor()


class Trace:
    _default_predictor = None
    DefaultPredictor = _LazyDefaultPredictor()

    def __init__(self, device, operations):
        self._device = device
        self._operations = operations
        self._run_time_ms = None

    @classmethod
    def default_predictor(cls):
        if cls._default_predictor is None:
            cls._default_predictor = Predictor()
        return cls._default_predictor

    @property
    def operations(self):
        return self._operations

    @property
    def device(self):
        return self._device

    @property
    def run_time_ms(self):
        if self._run_time_ms is None:
            self._run_time_ms = sum(op.run_time_ms for op in self._operations)
        return self._run_time_ms

    def to_device(self, dest_device, predictor=None):
        """The predicted trace on `dest_device` (all kernels of the trace are
        scaled in one GPU launch, all MLP operations of a kind in one more)."""
        if dest_device.name == self.device.name:
            return self
        predictor = predictor if predictor is not None else Trace.default_predictor()
        # Each operation keeps the contract of its own to_device (trace.py:46-49
        # maps it over the operations): one already measured on the destination
        # is returned as it is and a predicted one refuses; the measured ones
        # that do need predicting go to the GPU together.
        operations = list(self._operations)
        batch = [i for i, op in enumerate(operations)
                 if isinstance(op, MeasuredOperation) and op.device.name != dest_device.name]
        for i, op in enumerate(operations):
            if not isinstance(op, MeasuredOperation) or op.device.name == dest_device.name:
                operations[i] = op.to_device(dest_device, predictor)
        predicted = predictor.predict_operations([operations[i] for i in batch], dest_device)
        for i, op in zip(batch, predicted):
            operations[i] = op
        return Trace(dest_device, operations)

    def to_devices(self, dest_devices, predictor=None, device_features=None):
        """Predicted run time [ms] of the whole trace on each device of a sweep,
        computed on the GPU; returns a list of floats.  `device_features` maps
        device names to their four MLP features where the built-in table has
        none."""
        predictor = predictor if predictor is not None else Trace.default_predictor()
        return predictor.predict_trace_times(self, dest_devices, device_features)
