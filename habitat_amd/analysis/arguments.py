"""What an operation was called with, reduced to shapes and scalars
(analyzer/habitat/analysis/arguments.py:4-38)."""
import torch


def _describe(value):
    """A tensor becomes its size; tuples and lists are walked (and come back as
    plain tuples and lists); anything else is kept."""
    if isinstance(value, torch.Tensor):
        return value.size()
    for container in (tuple, list):
        if isinstance(value, container):
            return container(_describe(item) for item in value)
    return value


class Arguments:
    def __init__(self, args, kwargs):
        self.args, self.kwargs = args, kwargs
        self.special = {}

    @classmethod
    def from_raw_arguments(cls, args, kwargs):
        return cls(_describe(tuple(args)), {name: _describe(v) for name, v in kwargs.items()})
