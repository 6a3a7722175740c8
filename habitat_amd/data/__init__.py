"""Data files shipped with the package (device table; optionally the register
table and MLP checkpoints)."""
from pathlib import Path

_HERE = Path(__file__).resolve().parent


def path_to_data(data_file):
    """Absolute path, as a str, of `data_file` in this directory (the role of
    the reference's habitat.data.path_to_data, analyzer/habitat/data/__init__.py:6)."""
    return str(_HERE / data_file)
