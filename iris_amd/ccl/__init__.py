"""Stand-alone collectives over the symmetric heap (the rank-local part of iris.ccl's all-reduce and
reduce-scatter).  As in the reference (iris/ccl/__init__.py) the module exports the configuration
types; the operations are reached through the context: `ctx.ccl.all_reduce(output, input)`.
"""

from .config import Config
from .utils import ReduceOp

__all__ = ["Config", "ReduceOp"]
