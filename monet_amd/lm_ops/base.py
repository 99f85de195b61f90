"""Operator base class, backward-storage descriptors and the mode registry.

Same contract as the reference's monet/lm_ops/base.py:2-53: an operator class
declares, through `backward_storage`, what its backward needs kept from the
forward pass (some inputs, the output, or a compact intermediate it produces
itself), and registers itself for one or more aten op names under one or more
solver "modes".  `list_ops(mode, name)` returns the implementations in
REGISTRATION ORDER; a schedule refers to an implementation by that index.
"""
from typing import Callable, Dict, List, Optional, Sequence, Union


class StorageInfo:
    """Base of the three descriptors below."""


class InputStorage(StorageInfo):
    """Backward needs the forward inputs at positions `ids`."""

    def __init__(self, *ids: int):
        self.ids = ids

    def __repr__(self):
        return f"InputStorage{self.ids}"


class OutputStorage(StorageInfo):
    """Backward needs the forward output."""

    def __repr__(self):
        return "OutputStorage()"


class IntermediateStorage(StorageInfo):
    """Backward needs an intermediate the forward returns next to its output.

    `size(shape)` gives the intermediate's size in BYTES for an output shape.
    """

    def __init__(self, size_fn: Callable[[Sequence[int]], int]):
        self.size = size_fn

    def __repr__(self):
        return "IntermediateStorage(...)"


class OP:
    """An operator implementation: `forward(*aten_args)` and
    `backward(grad, stored, nodel=False)`.

    `stored` is a list the backward consumes: unless `nodel` is true it deletes
    each entry as soon as it has taken its own reference, so the caller's list
    no longer keeps the tensor alive.
    """
    names: List[str] = []
    backward_storage: Optional[Union[StorageInfo, List[StorageInfo]]] = None
    # True: `backward` writes into the storage of the gradient it is given (the reference's
    # ReLU backward does, lrrelu.cpp:14-15).  The executor hands such an operator a private
    # copy when another pending gradient still shares that storage.
    overwrites_grad = False

    def intermediate(self, *args, **kwargs):
        return None

    def forward(self, *args, **kwargs):
        raise NotImplementedError

    def backward(self, *args, **kwargs):
        raise NotImplementedError


all_modes = ["none", "normal", "multiway", "newnode", "multiway_newnode", "conv_multiway_newnode",
             "conv_normal", "gist"]
registry: Dict[str, Dict[str, list]] = {}


def implements(names: Sequence[str], modes: Sequence[str]):
    """Class decorator: register the class for every (mode, aten name) pair."""
    unknown = [m for m in modes if m not in all_modes]
    assert not unknown, f"unknown modes {unknown}"

    def register(cls):
        for mode in modes:
            by_name = registry.setdefault(mode, {})
            for name in names:
                by_name.setdefault(name, []).append(cls)
        cls.names = names
        return cls

    return register


def list_ops(mode: str, name: str) -> list:
    return registry[mode][name]
