"""xpu_graph for AMD Instinct MI355X: a torch.compile backend whose `mi355x`
target lowers matched Aten subgraphs to hand-written gfx950 HIP kernels.

    import torch
    from xpu_graph_amd import XpuGraph, XpuGraphConfig, Target, OptLevel

    backend = XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level2))
    fast = torch.compile(model, backend=backend)

Public names follow the reference package (src/xpu_graph/__init__.py).
"""
import os

from .cache import XpuGraphCache, XpuGraphLocalCache, default_cache, no_cache
from .compiler import XpuGraph, XpuGraphCompiler, XpuGraphRuntimeArtifact
from .config import OptLevel, Target, XpuGraphConfig
from .device_graph_runner import GraphRunner, HIPGraphRunner
from .guard_filters import skip_all_guards_unsafe
from .passes.patterns.plugin_pattern import (
    deregister_plugin_patterns,
    enable_plugin_patterns,
    register_plugin_pattern,
    register_this_as_pattern_constraint,
    register_this_as_plugin_pattern,
)

__version__ = "0.1.0"

__all__ = [
    "XpuGraph",
    "XpuGraphCompiler",
    "XpuGraphConfig",
    "XpuGraphRuntimeArtifact",
    "XpuGraphCache",
    "XpuGraphLocalCache",
    "default_cache",
    "no_cache",
    "Target",
    "OptLevel",
    "mi355x_compiler",
    "GraphRunner",
    "HIPGraphRunner",
    "register_plugin_pattern",
    "register_this_as_plugin_pattern",
    "register_this_as_pattern_constraint",
    "deregister_plugin_patterns",
    "enable_plugin_patterns",
    "skip_all_guards_unsafe",
]


def mi355x_compiler(is_training=False, opt_level=OptLevel.level2, debug=False, cache=None, **config_kwargs):
    """Ready-made backend for the MI355X target (counterpart of the reference's mlu_compiler / npu_compiler
    convenience constructors, src/xpu_graph/__init__.py:32-154).  `cache`: None (no compile-artifact cache), a
    directory, or an XpuGraphCache."""
    if isinstance(cache, (str, os.PathLike)):
        cache = XpuGraphLocalCache(cache)
    cfg = XpuGraphConfig(
        is_training=is_training, target=Target.mi355x, opt_level=opt_level, debug=debug, enable_cache=cache is not None, **config_kwargs
    )
    return XpuGraph(cfg, cache)
