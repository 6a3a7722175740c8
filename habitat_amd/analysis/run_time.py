"""Run times of one pass (forward or backward) of an operation: measured,
predicted from kernels, or predicted outright
(analyzer/habitat/analysis/run_time.py:5-88)."""


def ns_to_ms(ns):
    return ns / 1e6


def ms_to_ns(ms):
    return ms * 1e6


class RunTime:
    @property
    def run_time_ms(self):
        raise NotImplementedError

    @property
    def ktime_ns(self):
        return sum(k.run_time_ns for k in self.kernels)

    @property
    def kernels(self):
        return []

    @property
    def device(self):
        raise NotImplementedError


class RunTimeMeasurement(RunTime):
    def __init__(self, run_time_ms, kernels, device):
        self._run_time_ms = run_time_ms
        self._kernels = kernels
        self._device = device

    @property
    def run_time_ms(self):
        return self._run_time_ms

    @property
    def kernels(self):
        return self._kernels

    @property
    def device(self):
        return self._device


class RunTimePrediction(RunTime):
    """overhead + sum of predicted kernel times (run_time.py:42-66)."""

    def __init__(self, overhead_ns, predicted_kernels, device):
        self._run_time_ms = None
        self._overhead_ns = overhead_ns
        self._predicted_kernels = predicted_kernels
        self._device = device

    @property
    def run_time_ms(self):
        if self._run_time_ms is None:
            total_ns = self._overhead_ns + sum(k.run_time_ns for k in self.kernels)
            self._run_time_ms = ns_to_ms(total_ns)
        return self._run_time_ms

    @property
    def kernels(self):
        return self._predicted_kernels

    @property
    def device(self):
        return self._device


class RunTimePurePrediction(RunTime):
    """A predicted time with no kernel breakdown (MLP-predicted operations)."""

    def __init__(self, run_time_ms, device):
        self._run_time_ms = run_time_ms
        self._device = device

    @property
    def run_time_ms(self):
        return self._run_time_ms

    @property
    def device(self):
        return self._device
