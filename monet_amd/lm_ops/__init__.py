"""Low-memory operator library for MI355X: the operator classes a MONeT
schedule selects between, backed by hand-written gfx950 kernels."""
from .base import (OP, InputStorage, IntermediateStorage, OutputStorage, all_modes, implements,
                   list_ops, registry)
from . import conv, relu, elementary, pool, linear, bn, cat, funcs, softmax  # noqa: F401  (registration)
from .elementary import NativeOP
