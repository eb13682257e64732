"""Post-pass compile hook: after the pass pipeline, a configuration with `vendor_compiler_config` hands the
rewritten graph to `<target>_compile(gm, fake_inputs, is_inference=, is_backward=, **config)` of the module
`backends/<target>.py` (reference src/xpu_graph/backends/__init__.py:10-29).  A target with no such module
runs the graph as it is."""
import importlib
from typing import Any, Callable, Dict

import torch

from ..config import Target
from ..utils import logger

__all__ = ["vendor_compiler"]


def vendor_compiler(gm: torch.fx.GraphModule, fake_inputs: list, target: Target, *, is_inference: bool = False,
                    is_backward: bool = False, **config_dict: Dict[str, Any]) -> Callable:
    try:
        backend = importlib.import_module(f".{target.value}", __package__)
    except ImportError:
        logger.warning(f"{target.value}_compiler not found, return gm")
        return gm
    compile_fn = getattr(backend, f"{target.value}_compile")
    logger.info(f"{target.value}_compile start...")
    compiled = compile_fn(gm, fake_inputs, is_inference=is_inference, is_backward=is_backward, **config_dict)
    logger.info(f"{target.value}_compile complete")
    return compiled
