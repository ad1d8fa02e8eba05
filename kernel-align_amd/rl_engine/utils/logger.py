"""Process-wide logger of the engine.

Mirrors the interface of the reference's rl_engine/utils/logger.py:44-67: a
stdout logger named "RL-Engine" whose instance also offers ``info_once``,
``warn_once`` and ``info_on_rank``.
"""
from __future__ import annotations

import logging
import sys
import threading

LOG_FORMAT = "%(levelname)s %(asctime)s [%(name)s]: %(message)s"
LOG_DATEFMT = "%m-%d %H:%M:%S"


class EngineLogger(logging.Logger):
    """logging.Logger plus once-only and rank-filtered helpers."""

    def __init__(self, name: str, level: int = logging.INFO):
        super().__init__(name, level)
        self._seen: set = set()
        self._seen_lock = threading.Lock()

    def _once(self, level: int, msg: str, args: tuple) -> None:
        key = (level, msg, args)
        with self._seen_lock:
            if key in self._seen:
                return
            self._seen.add(key)
        self.log(level, msg, *args, stacklevel=3)

    def info_once(self, msg: str, *args) -> None:
        """Log an INFO record the first time this (msg, args) pair is seen."""
        self._once(logging.INFO, msg, args)

    def warn_once(self, msg: str, *args) -> None:
        """Log a WARNING record the first time this (msg, args) pair is seen."""
        self._once(logging.WARNING, msg, args)

    def info_on_rank(self, msg: str, rank: int = 0, *args) -> None:
        """Log only when the process is the given rank (single-GPU processes are rank 0)."""
        from rl_engine.platforms.device import device_ctx

        if getattr(device_ctx, "rank", 0) == rank:
            self.info(msg, *args)


_loggers: dict = {}


def init_logger(name: str) -> EngineLogger:
    """Return the engine logger `name`, creating it with a stdout handler on first use."""
    lg = _loggers.get(name)
    if lg is None:
        lg = EngineLogger(name)
        handler = logging.StreamHandler(sys.stdout)
        handler.setFormatter(logging.Formatter(LOG_FORMAT, datefmt=LOG_DATEFMT))
        lg.addHandler(handler)
        lg.propagate = False
        _loggers[name] = lg
    return lg


logger = init_logger("RL-Engine")
