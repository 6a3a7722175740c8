import os

_DATA_PATH = os.path.abspath(os.path.dirname(__file__))


def path_to_data(data_file):
    """Absolute path of a file shipped in this directory (the reference's
    habitat.data.path_to_data, analyzer/habitat/data/__init__.py:6)."""
    return os.path.join(_DATA_PATH, data_file)
