"""Fixed-point driver of the pass pipeline (reference
src/xpu_graph/passes/pass_manager.py:8-85): re-propagate fake values, run every
enabled pass, repeat while any pass changed the graph.  As in the reference the
`changed or pass(gm)` chain short-circuits, so after the first change in a sweep
the remaining passes wait for the next iteration."""
import torch
from torch._guards import detect_fake_mode
from torch._subclasses.fake_tensor import FakeTensor

from ..fx_utils import FxStage
from .fake_prop import propagate_missing
from .optimizer import Optimizer


class PassManager:
    def __init__(self, config):
        from .general import ConstantFolding, Cse, Dce, RemoveAssertions, ViewToReshape
        from .patterns.pattern_manager import PatternManager

        self._config = config
        Optimizer._debug = config.debug
        Optimizer._dump_graph = config.dump_graph
        self._pattern_manager = PatternManager(config)
        self._passes = []
        for cls in (RemoveAssertions, ViewToReshape, Dce, Cse):
            if cls._opt_level <= config.opt_level:
                self._passes.append(cls())
        self._passes.append(self._pattern_manager)
        if config.constant_folding and ConstantFolding._opt_level <= config.opt_level:
            self._passes.append(ConstantFolding(config.folding_freezed_params))
        for p in self._passes:
            p._set_level(config.opt_level)
        self._enabled = []

    def get_pattern_manager(self):
        return self._pattern_manager

    def __call__(self, gm, example_inputs, stage: FxStage):
        self._enabled = [q for q in (p.get_pass_with_stage(stage) for p in self._passes) if q]
        assert all(isinstance(t, FakeTensor) for t in example_inputs if isinstance(t, torch.Tensor))
        fake_mode = detect_fake_mode(example_inputs)
        if fake_mode is None:
            from torch._subclasses.fake_tensor import FakeTensorMode

            fake_mode = FakeTensorMode(allow_non_fake_inputs=True)
        changed = True
        while changed:
            propagate_missing(gm, fake_mode)
            changed = False
            for p in self._enabled:
                changed = changed or p(gm)
        return gm
