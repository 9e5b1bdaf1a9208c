"""GACT activation compression on MI355X: the reference's import surface over hand-written HIP kernels."""
from . import ops
from . import controller
from .conf import config, set_optimization_level, set_adapt_interval
