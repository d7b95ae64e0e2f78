"""Rank-tagged logging for the package.

Mirrors iris/host/logging/logging.py:13-92 of the reference: a logger named "iris", level taken
from IRIS_LOG_LEVEL, records formatted as "HH:MM:SS LEVEL [Iris] [rank/world] message".
"""

import logging
import os

DEBUG = logging.DEBUG
INFO = logging.INFO
WARNING = logging.WARNING
ERROR = logging.ERROR


class IrisFormatter(logging.Formatter):
    """Formatter that prefixes every record with the rank it was emitted on."""

    def format(self, record):
        rank = getattr(record, "iris_rank", "?")
        world = getattr(record, "iris_num_ranks", "?")
        stamp = self.formatTime(record, "%H:%M:%S")
        where = f" [{record.module}]" if getattr(record, "iris_internal", False) else ""
        return f"{stamp} {record.levelname:<5s} [Iris] [{rank}/{world}]{where} {record.getMessage()}"


logger = logging.getLogger("iris")
logger.setLevel(logging.INFO)
_level = os.environ.get("IRIS_LOG_LEVEL", "").upper()
if _level in ("DEBUG", "INFO", "WARNING", "ERROR"):
    logger.setLevel(getattr(logging, _level))
if not logger.handlers:
    _handler = logging.StreamHandler()
    _handler.setFormatter(IrisFormatter())
    logger.addHandler(_handler)


def log_rank(level, msg, *args, rank=None, num_ranks=None):
    """Emit `msg % args` at `level`, tagged with the given rank (reference: `_log_rank`)."""
    if logger.isEnabledFor(level):
        extra = {"iris_internal": True}
        if rank is not None:
            extra["iris_rank"] = rank
        if num_ranks is not None:
            extra["iris_num_ranks"] = num_ranks
        logger.log(level, msg, *args, extra=extra, stacklevel=2)


def debug_on():
    """Whether DEBUG records are emitted: lets a hot path skip building a record's arguments."""
    return logger.isEnabledFor(logging.DEBUG)


def set_logger_level(level):
    """Set the level of the "iris" logger (iris.DEBUG, iris.INFO, iris.WARNING, iris.ERROR)."""
    logger.setLevel(level)
