"""``kvcore_amd.*`` loggers.  Reference: kvcore/utils/log.py:6-59 (default WARNING, an
environment variable for the level, ``configure_logging(level, force)``)."""

from __future__ import annotations

import logging
import os

ENV_LEVEL = "KVCORE_AMD_LOG_LEVEL"
_ROOT = "kvcore_amd"


def get_logger(name: str) -> logging.Logger:
    return logging.getLogger(name if name.startswith(_ROOT) else f"{_ROOT}.{name}")


def configure_logging(level: str | int | None = None, *, force: bool = False) -> None:
    root = logging.getLogger(_ROOT)
    if root.handlers and not force:
        return
    for h in list(root.handlers):
        root.removeHandler(h)
    handler = logging.StreamHandler()
    handler.setFormatter(logging.Formatter("%(asctime)s %(levelname)s %(name)s: %(message)s"))
    root.addHandler(handler)
    root.propagate = False
    if level is None:
        level = os.environ.get(ENV_LEVEL, "WARNING")
    root.setLevel(level if isinstance(level, int) else str(level).upper())


def set_log_level(level: str | int) -> None:
    logging.getLogger(_ROOT).setLevel(level if isinstance(level, int) else str(level).upper())
