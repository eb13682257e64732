"""Logging and environment-variable names.

The logger name, its child-logger scheme and the environment variable names are
those of the reference (src/xpu_graph/utils.py:13-67,185-201) because its tests
assert on the emitted text ("Pattern.<Name> changed graph", ...).
"""
import logging
import os
import sys


class _LoggerProxy:
    """Forwards to a swappable logging.Logger so `local_logger` can redirect output to a child logger."""

    def __init__(self, name):
        base = logging.getLogger(name)
        if not base.handlers:
            handler = logging.StreamHandler(stream=sys.stdout)
            handler.setFormatter(
                logging.Formatter(
                    fmt="%(asctime)s.%(msecs)03d %(process)d-%(thread)d %(filename)s:%(lineno)d [XPU_GRAPH][%(levelname)s]: %(message)s",
                    datefmt="%Y-%m-%d %H:%M:%S",
                )
            )
            base.addHandler(handler)
            base.propagate = False
        object.__setattr__(self, "_logger", base)

    def __getattr__(self, item):
        return getattr(object.__getattribute__(self, "_logger"), item)

    def __setattr__(self, key, value):
        if key == "_logger":
            object.__setattr__(self, key, value)
        else:
            setattr(object.__getattribute__(self, "_logger"), key, value)


logger = _LoggerProxy("xpu_graph")


def setup_logger(is_debug):
    logger.setLevel(logging.DEBUG if is_debug else logging.INFO)


_DEBUG_CHILDREN = {"xpu_graph." + n for n in os.getenv("XPUGRAPH_LOGS", "").split(",") if n}


class local_logger:
    """Context manager: log through the child logger `xpu_graph.<name>`; XPUGRAPH_LOGS=a,b turns children to DEBUG."""

    def __init__(self, name, level=None):
        self._child = logger.getChild(name)
        if self._child.name in _DEBUG_CHILDREN:
            level = logging.DEBUG
        self._level = level or logger.level

    def __enter__(self):
        self._saved = logger._logger
        self._child.setLevel(self._level)
        logger._logger = self._child
        return self

    def __exit__(self, *exc):
        logger._logger = self._saved
        return False


class ENV:
    cache_dir = "XPUGRAPH_CACHE_DIR"
    dump_dir = "XPUGRAPH_DUMP_DIR"
    debug = "XPUGRAPH_DEBUG"
    opt_level = "XPUGRAPH_OPT_LEVEL"
    vendor_compiler_mode = "VENDOR_COMPILER_MODE"
    enable_interceptor = "XPUGRAPH_INTERCEPTOR"
    logs = "XPUGRAPH_LOGS"
    include_patterns = "XPUGRAPH_DEBUG_INCLUDE_PATTERNS"
    skip_patterns = "XPUGRAPH_DEBUG_SKIP_PATTERNS"
    fallback_legacy_dispatch = "XPUGRAPH_FALLBACK_LEGACY_DISPATCH"
    partition_fn = "XPUGRAPH_PARTITIONER"


def env_flag(name, default):
    raw = os.environ.get(name)
    if raw is None:
        return default
    low = raw.lower()
    if low in ("true", "1", "on"):
        return True
    if low in ("false", "0", "off"):
        return False
    raise ValueError(f"Invalid value for {name}: {raw}")
