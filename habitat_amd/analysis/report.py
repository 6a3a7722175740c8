"""CSV outputs of a prediction run, in the two layouts the reference's
evaluation harness writes (experiments/run_experiment.py:41-60):

  <config>-<origin>-e2e.csv                 device,run_time_ms
  <config>-<origin>-<dest>-breakdown.csv    operation,run_time_ms
"""
import csv
import os


def e2e_file_name(config_name, origin_device):
    return "{}-{}-e2e.csv".format(config_name, origin_device.name)


def breakdown_file_name(config_name, origin_device, dest_device):
    return "{}-{}-{}-breakdown.csv".format(config_name, origin_device.name, dest_device.name)


def record_e2e(config_name, origin_device, data, directory="."):
    """data: iterable of (device, run_time_ms); the origin's measured time first,
    then one row per predicted destination.  Returns the path written."""
    path = os.path.join(directory, e2e_file_name(config_name, origin_device))
    with open(path, "w", newline="") as f:
        writer = csv.writer(f)
        writer.writerow(["device", "run_time_ms"])
        for device, run_time_ms in data:
            writer.writerow([device.name, run_time_ms])
    return path


def record_breakdown(config_name, origin_device, dest_device, trace, directory="."):
    """One row per operation of `trace` (measured or predicted)."""
    path = os.path.join(directory, breakdown_file_name(config_name, origin_device, dest_device))
    with open(path, "w", newline="") as f:
        writer = csv.writer(f)
        writer.writerow(["operation", "run_time_ms"])
        for op in trace.operations:
            writer.writerow([op.name, op.run_time_ms])
    return path


def record_sweep(config_name, trace, dest_devices, totals_ms, directory="."):
    """The e2e file for a device sweep: the origin's measured time, then the
    predicted total of every destination (from Trace.to_devices)."""
    rows = [(trace.device, trace.run_time_ms)] + list(zip(dest_devices, totals_ms))
    return record_e2e(config_name, trace.device, rows, directory)
