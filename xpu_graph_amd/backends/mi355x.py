"""`mi355x_compile`: what `vendor_compiler_config` selects on this target.

{"compiler": "device_graph"} records the rewritten graph into HIP graphs (inference only, like the reference's
mlu_compile / npu_compile, src/xpu_graph/backends/mlu.py:21-24).  There is no tracing compiler behind this
target -- the rewritten graph already calls the hand-written kernels -- so every other setting ("mode": ...)
leaves the graph as it is and says so once."""
from typing import Dict

import torch

from ..utils import logger
from . import device_graph

__all__ = ["mi355x_compile"]


def mi355x_compile(module: torch.nn.Module, example_inputs, *, is_inference: bool = False, is_backward: bool = False,
                   **config_dict: Dict) -> torch.nn.Module:
    if config_dict.get("compiler") == "device_graph":
        if not is_inference:
            # forward-stage regions would hand activations saved for backward out of a pool that the next replay
            # overwrites (a second forward before the backward corrupts gradients): training graphs are not recorded
            raise ValueError("device-graph capture / replay is for inference graphs: drop vendor_compiler_config when is_training=True")
        return device_graph.device_graph_compiler(module, example_inputs, target="cuda", **config_dict)
    logger.warning(f"vendor_compiler_config {config_dict} selects no compiler on mi355x: the rewritten graph runs as it is")
    return module
