"""Operations of a trace: measured on a device, or predicted for another.

Same three classes and read-only attributes as the reference
(analyzer/habitat/analysis/operation.py:3-138): `name`, `arguments`, `forward`,
`backward`, `device`, the sums `run_time_ms` and `ktime_ns` over the passes an
operation has, and `to_device`.
"""
import operator


def _read_only(slot):
    return property(operator.attrgetter(slot))


def _abstract(self):
    raise NotImplementedError


class Operation:
    __slots__ = ()

    name = property(_abstract)
    forward = property(_abstract)
    backward = property(_abstract)
    device = property(_abstract)
    arguments = property(lambda self: None)

    def _over_passes(self, attribute):
        total = getattr(self.forward, attribute)
        if self.backward is not None:
            total = total + getattr(self.backward, attribute)
        return total

    run_time_ms = property(lambda self: self._over_passes("run_time_ms"))
    ktime_ns = property(lambda self: self._over_passes("ktime_ns"))

    def __repr__(self):
        return self.name

    def to_device(self, dest_device, predictor):
        raise NotImplementedError


class MeasuredOperation(Operation):
    __slots__ = ("_name", "_arguments", "_forward", "_backward", "_device")

    def __init__(self, name, arguments, forward, backward, device):
        self._name, self._arguments = name, arguments
        self._forward, self._backward, self._device = forward, backward, device

    name = _read_only("_name")
    arguments = _read_only("_arguments")
    forward = _read_only("_forward")
    backward = _read_only("_backward")
    device = _read_only("_device")

    def to_device(self, dest_device, predictor):
        """Itself on its own device, else the predictor's answer."""
        if dest_device.name == self._device.name:
            return self
        return predictor.predict_operation(self, dest_device)


class PredictedOperation(Operation):
    __slots__ = ("_measured_operation", "_forward", "_backward", "_device")

    def __init__(self, measured_operation, forward, backward, device):
        self._measured_operation = measured_operation
        self._forward, self._backward, self._device = forward, backward, device

    name = property(lambda self: self._measured_operation.name)
    arguments = property(lambda self: self._measured_operation.arguments)
    forward = _read_only("_forward")
    backward = _read_only("_backward")
    device = _read_only("_device")

    def to_device(self, dest_device, predictor):
        # operation.py:137: predictions are not inputs to further predictions
        raise RuntimeError("Cannot make a prediction using a predicted operation.")
