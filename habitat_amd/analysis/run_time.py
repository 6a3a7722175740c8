"""Run times of one pass (forward or backward) of an operation: measured,
predicted from kernels, or predicted outright.  Same four classes and read-only
attributes as the reference (analyzer/habitat/analysis/run_time.py:5-88):
`run_time_ms`, `kernels`, `device` and the kernel-time sum `ktime_ns`."""
import operator


def ns_to_ms(ns):
    return ns / 1e6


def ms_to_ns(ms):
    return ms * 1e6


def _stored(slot):
    return property(operator.attrgetter(slot))


def _missing(self):
    raise NotImplementedError


class RunTime:
    __slots__ = ()

    run_time_ms = property(_missing)
    device = property(_missing)
    kernels = property(lambda self: [])
    ktime_ns = property(lambda self: sum(kernel.run_time_ns for kernel in self.kernels))


class RunTimeMeasurement(RunTime):
    __slots__ = ("_run_time_ms", "_kernels", "_device")

    def __init__(self, run_time_ms, kernels, device):
        self._run_time_ms, self._kernels, self._device = run_time_ms, kernels, device

    run_time_ms = _stored("_run_time_ms")
    kernels = _stored("_kernels")
    device = _stored("_device")


class RunTimePrediction(RunTime):
    """Overhead plus the predicted kernels' times (run_time.py:42-66); the sum
    is formed on first use and kept.  `from_times` makes one from the measured
    kernels and their predicted times, and wraps each pair in a PredictedKernel
    only when `kernels` is read."""
    __slots__ = ("_total_ms", "_overhead_ns", "_predicted_kernels", "_device", "_measured",
                 "_times")

    def __init__(self, overhead_ns, predicted_kernels, device):
        self._total_ms = None
        self._overhead_ns = overhead_ns
        self._predicted_kernels, self._device = predicted_kernels, device
        self._measured = self._times = None

    @classmethod
    def from_times(cls, overhead_ns, measured_kernels, times_ns, device):
        self = cls(overhead_ns, None, device)
        self._measured, self._times = measured_kernels, times_ns
        return self

    device = _stored("_device")

    @property
    def kernels(self):
        if self._predicted_kernels is None:
            from habitat_amd.analysis.kernels import PredictedKernel
            self._predicted_kernels = [PredictedKernel(k, t)
                                       for k, t in zip(self._measured, self._times)]
        return self._predicted_kernels

    @property
    def ktime_ns(self):
        if self._predicted_kernels is None:
            return sum(self._times)
        return sum(kernel.run_time_ns for kernel in self._predicted_kernels)

    @property
    def run_time_ms(self):
        if self._total_ms is None:
            self._total_ms = ns_to_ms(self._overhead_ns + self.ktime_ns)
        return self._total_ms


class RunTimePurePrediction(RunTime):
    """A predicted time with no kernel breakdown (MLP-predicted operations)."""
    __slots__ = ("_run_time_ms", "_device")

    def __init__(self, run_time_ms, device):
        self._run_time_ms, self._device = run_time_ms, device

    run_time_ms = _stored("_run_time_ms")
    device = _stored("_device")
