"""GACT activation compression on MI355X.

The import surface of the reference package (``gact.ops``, ``gact.controller``, ``gact.config``,
``gact.set_optimization_level``, ``gact.set_adapt_interval``) over hand-written HIP kernels; see
``gact.cpp_extension`` for the extension-style entry points and ``gact.batched`` for the one-launch
mixed-width path.
"""
from .conf import config, set_adapt_interval, set_optimization_level
from . import controller, ops

__all__ = ["config", "controller", "ops", "set_adapt_interval", "set_optimization_level"]
