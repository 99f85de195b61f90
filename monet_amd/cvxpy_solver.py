"""Name-compatible home of `Solution` and `Model` (the reference keeps them in
monet/cvxpy_solver.py); the implementation is monet_amd.solver."""
from .solver import Model, Solution  # noqa: F401
