"""Shapes and scalars an operation was called with
(analyzer/habitat/analysis/arguments.py:4-38)."""
import torch


class Arguments:
    def __init__(self, args, kwargs):
        self.args = args
        self.kwargs = kwargs
        self.special = {}

    @classmethod
    def from_raw_arguments(cls, args, kwargs):
        return cls(tuple(_shape_of(a) for a in args),
                   {name: _shape_of(value) for name, value in kwargs.items()})


def _shape_of(argument):
    """Tensors are replaced by their sizes; containers are walked; scalars stay."""
    if isinstance(argument, tuple):
        return tuple(_shape_of(a) for a in argument)
    if isinstance(argument, list):
        return [_shape_of(a) for a in argument]
    if isinstance(argument, torch.Tensor):
        return argument.size()
    return argument
