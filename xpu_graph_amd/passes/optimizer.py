"""Base class of every graph pass.

A pass implements `process(gm) -> bool` (True when it rewrote the graph).  The
call wrapper lints and recompiles the module after a change and emits the debug
line the reference's tests assert on (src/xpu_graph/passes/optimizer.py:33-49):

    "<BaseClassName>.<ClassName> changed graph, before: N nodes, after: M nodes."
"""
import abc
import os
import time

import torch.fx as fx

from ..config import OptLevel
from ..fx_utils import FxStage
from ..utils import logger

_dump_counter = 0


class Optimizer(abc.ABC):
    _debug = False
    _dump_graph = False
    _opt_level = OptLevel.level1
    _support_stages = [FxStage.inference]

    @abc.abstractmethod
    def process(self, gm: fx.GraphModule) -> bool:
        ...

    def get_pass_with_stage(self, stage):
        return self if stage in self._support_stages else None

    def _set_level(self, opt_level):
        self._opt_level = opt_level

    def __str__(self):
        return type(self).__name__

    def __call__(self, gm: fx.GraphModule) -> bool:
        before = len(gm.graph.nodes)
        t0 = time.time()
        changed = bool(self.process(gm))
        logger.debug(f"{self}.__call__ cost {time.time() - t0:.4f}s")
        if not changed:
            return False
        gm.graph.lint()
        gm.recompile()
        # the family a pass belongs to ("Pattern", "Optimizer"), however many helper classes sit in between
        base = next((c.__name__ for c in type(self).__mro__[1:] if c.__name__ in ("Pattern", "Optimizer")), type(self).__bases__[0].__name__)
        logger.debug(f"{base}.{self} changed graph, before: {before} nodes, after: {len(gm.graph.nodes)} nodes.")
        if self._dump_graph:
            self._dump(gm)
        return True

    def _dump(self, gm):
        global _dump_counter
        folder = f"xpu_graph_debugs_pid{os.getpid()}"
        os.makedirs(folder, exist_ok=True)
        path = os.path.join(folder, f"optimization_{_dump_counter}_after_pass_{self}.txt")
        with open(path, "w") as f:
            f.write(str(gm.graph))
        _dump_counter += 1
