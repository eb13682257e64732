"""Configuration of the compiler backend.

Mirrors the public configuration surface of the reference
(src/xpu_graph/config.py:11-131): the `Target` and `OptLevel` enums, the
`XpuGraphConfig` dataclass with the same field names and defaults, and the same
environment overrides.  The one addition is `Target.mi355x`.
"""
import dataclasses
import enum
import os
import tempfile
import warnings
from typing import Any, Callable, Dict, List, Optional, Union

from .utils import ENV, env_flag, logger


class Target(enum.Enum):
    mi355x = "mi355x"
    none = "none"


class OptLevel(enum.Enum):
    """level0: no optimisation; level1: bitwise-preserving rewrites only;
    level2: fusions that may change rounding; level3: as level2 plus fast activations."""

    level0 = 0
    level1 = 1
    level2 = 2
    level3 = 3

    def _cmp(self, other, op):
        if not isinstance(other, OptLevel):
            return NotImplemented
        return op(self.value, other.value)

    def __lt__(self, other):
        return self._cmp(other, lambda a, b: a < b)

    def __le__(self, other):
        return self._cmp(other, lambda a, b: a <= b)

    def __gt__(self, other):
        return self._cmp(other, lambda a, b: a > b)

    def __ge__(self, other):
        return self._cmp(other, lambda a, b: a >= b)


_VENDOR_MODES = ("default", "cudagraphs", "reduce-overhead", "max-autotune", "max-autotune-no-cudagraphs")


@dataclasses.dataclass
class XpuGraphConfig:
    is_training: bool  # required: training compiler (fw/bw stages) or inference compiler
    debug: bool = False
    target: Target = dataclasses.field(default_factory=lambda: Target.none)
    opt_level: OptLevel = dataclasses.field(default_factory=lambda: OptLevel.level1)
    dump_graph: bool = False
    enable_cache: bool = True
    freeze: bool = False  # inference only: parameters become graph attributes
    constant_folding: bool = True
    folding_freezed_params: bool = True
    vendor_compiler_config: Optional[Dict[str, Any]] = None
    enable_interceptor: Optional[str] = None
    include_patterns: List[str] = dataclasses.field(default_factory=list)
    skip_patterns: List[str] = dataclasses.field(default_factory=list)
    fallback_legacy_dispatch: bool = True
    partition_fn: Optional[Union[Callable, str]] = None

    def _reset_config_with_env(self):
        """Environment variables win over constructor arguments (reference config.py:82-131)."""
        if os.getenv(ENV.debug) is not None:
            self.debug = env_flag(ENV.debug, False)
        lvl = os.getenv(ENV.opt_level)
        if lvl is not None:
            if lvl in ("0", "1", "2", "3"):
                self.opt_level = OptLevel(int(lvl))
            else:
                warnings.warn("Illegal XPUGRAPH_OPT_LEVEL value, XPUGRAPH_OPT_LEVEL will not take effect.")
        mode = os.getenv(ENV.vendor_compiler_mode)
        if mode is not None:
            if mode == "none":
                self.vendor_compiler_config = None
            elif mode in _VENDOR_MODES:
                self.vendor_compiler_config = {"mode": mode}
            else:
                warnings.warn("Illegal VENDOR_COMPILER_MODE value, VENDOR_COMPILER_MODE will not take effect.")
        if os.getenv(ENV.enable_interceptor) is not None:
            self.enable_interceptor = os.getenv(ENV.enable_interceptor)
        if os.getenv(ENV.include_patterns) is not None:
            self.include_patterns = os.getenv(ENV.include_patterns).split(",")
        if os.getenv(ENV.skip_patterns) is not None:
            self.skip_patterns = os.getenv(ENV.skip_patterns).split(",")
        if os.getenv(ENV.fallback_legacy_dispatch) is not None:
            self.fallback_legacy_dispatch = env_flag(ENV.fallback_legacy_dispatch, self.fallback_legacy_dispatch)
        if os.getenv(ENV.partition_fn) is not None:
            self.partition_fn = get_partition_fn(os.getenv(ENV.partition_fn))


_cache_dir = os.getenv(ENV.cache_dir)


def get_cache_dir():
    """XPUGRAPH_CACHE_DIR, or a fresh temporary directory that is then exported under that name so that child
    processes share it (reference config.py:134-145)."""
    global _cache_dir
    if _cache_dir is None:
        _cache_dir = tempfile.mkdtemp(prefix="xpugraph_")
        os.environ[ENV.cache_dir] = _cache_dir
        logger.debug(f"Use {_cache_dir} as default local cache")
    return _cache_dir


_dump_dir = os.getenv(ENV.dump_dir)


def get_dump_dir():
    global _dump_dir
    if _dump_dir is None:
        _dump_dir = tempfile.mkdtemp(prefix="xpugraph_")
        os.environ[ENV.dump_dir] = _dump_dir
        logger.debug(f"Use {_dump_dir} as default dump path")
    return _dump_dir


def get_partition_fn(spec):
    """'default' | 'mincut' | dotted path of a callable | a callable (reference config.py:158-185)."""
    if not isinstance(spec, str):
        return spec
    from torch._functorch.partitioners import default_partition, min_cut_rematerialization_partition

    key = spec.lower()
    if key == "default":
        return default_partition
    if key == "mincut":
        return min_cut_rematerialization_partition
    try:
        import importlib

        mod_name, fn_name = spec.rsplit(".", 1)
        fn = getattr(importlib.import_module(mod_name), fn_name)
        if not callable(fn):
            raise TypeError(spec)
        return fn
    except Exception:
        warnings.warn(f"Failed to import partition function {spec}, use default partition function")
        return None
