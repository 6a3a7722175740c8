"""TEST INFRASTRUCTURE — CPU oracle, not product code.

Operation- and trace-level arithmetic of the reference, restated over plain
numbers so that it can be fed from the other oracle modules:
  Predictor._wave_scale        analyzer/habitat/analysis/predictor.py:111-130
  RunTimePrediction.run_time_ms analyzer/habitat/analysis/run_time.py:50-58
  Predictor._special_scale     analyzer/habitat/analysis/predictor.py:132-148
  the four scalers' final line analyzer/habitat/analysis/predictor.py:182,218,238,283
  Operation.run_time_ms        analyzer/habitat/analysis/operation.py:10-14
  Trace.run_time_ms            analyzer/habitat/analysis/trace.py:27-36

pins (tests/test_oracle.py::test_predictor_arithmetic): a three-operation,
five-kernel trace worked by hand, the overhead clamp, the negative-prediction
clamp.
"""


def wave_scaled_pass_ms(run_time_ms, measured_kernel_ns, predicted_kernel_ns):
    """One forward or backward pass: the part of the measured time not spent in
    kernels is kept as overhead (never negative), kernels are replaced."""
    overhead_ns = run_time_ms * 1e6 - sum(measured_kernel_ns)
    overhead_ns = 0 if overhead_ns < 0 else overhead_ns
    return (overhead_ns + sum(predicted_kernel_ns)) / 1e6


def special_op_ms(run_time_ms, pred_dest, pred_orig):
    """An MLP-predicted operation: measured time (forward + backward) scaled by
    the ratio of the two predictions; negative results become 0."""
    ms = run_time_ms * pred_dest / pred_orig
    return 0. if ms < 0 else ms


def trace_ms(op_times_ms):
    return sum(op_times_ms)
