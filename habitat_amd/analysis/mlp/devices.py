"""Device features fed to the MLPs next to the operation features.

The reference keeps them in a CSV that it re-reads on every prediction
(analyzer/habitat/analysis/mlp/devices.py:5-20, devices.csv:1-7); here the table
is a module constant.  Columns used by the predictors: memory size [GB],
memory bandwidth [GB/s], SM count, peak single-precision TFLOP/s.
"""

# device: {mem, mem_type, mem_bw, num_sm, double, single, half}; None = not listed
_TABLE = {
    "P100":      dict(mem=16, mem_type="HBM2",  mem_bw=732, num_sm=56, double=4.7,     single=9.3,     half=18.7),
    "P4000":     dict(mem=8,  mem_type="GDDR5", mem_bw=243, num_sm=14, double=0.1656,  single=5.3,     half=None),
    "RTX2070":   dict(mem=8,  mem_type="GDDR6", mem_bw=448, num_sm=36, double=0.20304, single=6.49728, half=12.99456),
    "RTX2080Ti": dict(mem=11, mem_type="GDDR6", mem_bw=616, num_sm=68, double=0.3672,  single=11.7504, half=23.5008),
    "T4":        dict(mem=16, mem_type="GDDR6", mem_bw=320, num_sm=40, double=None,    single=8.1,     half=None),
    "V100":      dict(mem=16, mem_type="HBM2",  mem_bw=900, num_sm=80, double=None,    single=14.028,  half=None),
    # this build's synthetic destination
    "MI355X":    dict(mem=288, mem_type="HBM3E", mem_bw=8000, num_sm=256, double=78.6, single=157.3,  half=2500.0),
}
_TABLE["MI355X_cdna"] = _TABLE["MI355X"]   # the same GPU under its compute-unit description

DEVICE_PARAMS = ["mem", "mem_bw", "num_sm", "single"]

# name -> [mem, mem_bw, num_sm, single]
DEVICE_FEATURES = {name: [row[p] for p in DEVICE_PARAMS] for name, row in _TABLE.items()}


def register_device(name, mem, mem_bw, num_sm, single, **extra):
    """Add (or replace) a device row, e.g. for a synthetic device sweep."""
    row = dict(mem=mem, mem_type=extra.get("mem_type"), mem_bw=mem_bw, num_sm=num_sm,
               double=extra.get("double"), single=single, half=extra.get("half"))
    _TABLE[name] = row
    DEVICE_FEATURES[name] = [row[p] for p in DEVICE_PARAMS]


def unregister_device(name):
    """Remove a row added with register_device."""
    _TABLE.pop(name, None)
    DEVICE_FEATURES.pop(name, None)


def get_device_features(device_name, device_params):
    """[row[p] for p in device_params] of one device.  An unknown device raises
    IndexError, as the reference's pandas lookup does (devices.py:9)."""
    if device_name not in _TABLE:
        raise IndexError("single positional indexer is out-of-bounds")
    row = _TABLE[device_name]
    return [row[p] for p in device_params]


def get_all_devices(device_params=None):
    """{device: [features]} (devices.py:12-20)."""
    params = device_params if isinstance(device_params, list) else [
        "mem", "mem_type", "mem_bw", "num_sm", "double", "single", "half"]
    return {name: [row[p] for p in params] for name, row in _TABLE.items()}
