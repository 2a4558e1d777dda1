"""Environment-driven logging used by the executor's debug mode.

``DCP_DEBUG=DEBUG`` turns file logging on, ``DCP_LOGGING_DEBUG_DIR`` chooses
where the per-component files go (same switches as the reference's
``dcp/utils/logger.py:19-38,129-199``).
"""

import logging
import os
import sys

_LEVELS = {
    "DEBUG": logging.DEBUG,
    "INFO": logging.INFO,
    "WARNING": logging.WARNING,
    "ERROR": logging.ERROR,
}
_default_level = _LEVELS.get(os.environ.get("DCP_DEBUG", "INFO").upper(), logging.INFO)
_debug_log_dir = os.environ.get("DCP_LOGGING_DEBUG_DIR", "./dcp_debug_logs")


def read_env_bool(key: str, default: bool = False) -> bool:
    value = os.environ.get(key)
    if value is None:
        return default
    return value in ("1", "True", "true")


def read_env_int(key: str, default: int = 0) -> int:
    value = os.environ.get(key)
    return default if value is None else int(value)


def create_logger(name=None, prefix=None, level=_default_level, log_file=None):
    if name is None:
        raise ValueError("name for logger cannot be None")
    if level > logging.DEBUG:
        log_file = None
    tag = f"[{prefix}] " if prefix else ""
    fmt = logging.Formatter(f"[%(asctime)s] [%(levelname)s] {tag}%(message)s")
    log = logging.getLogger(name if prefix is None else f"{name}.{prefix}")
    log.handlers.clear()
    log.setLevel(level)
    log.propagate = False
    if log_file is not None:
        path = os.path.join(_debug_log_dir, log_file)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        handler = logging.FileHandler(path, mode="w")
    else:
        handler = logging.StreamHandler(stream=sys.stdout)
    handler.setFormatter(fmt)
    handler.setLevel(level)
    log.addHandler(handler)
    return log


logger = create_logger(name="DCP", level=_default_level)
