"""Pattern base class: a graph pass with an optimisation level, an execution
group and the stages it supports; switched on/off by class name through
`XpuGraphConfig.include_patterns / skip_patterns` (reference
src/xpu_graph/passes/patterns/pattern.py:15-49)."""
import enum

import torch.fx as fx

from ...config import OptLevel, XpuGraphConfig
from ...fx_utils import FxStage
from ...utils import logger
from ..optimizer import Optimizer


class PatternGroup(enum.Enum):
    GROUP0 = 0
    GROUP1 = 1
    GROUP2 = 2

    def __lt__(self, other):
        if isinstance(other, PatternGroup):
            return self.value < other.value
        return NotImplemented


class Pattern(Optimizer):
    _opt_level = OptLevel.level1
    _pattern_group = PatternGroup.GROUP0
    _support_stages = [FxStage.inference]

    def __init__(self):
        super().__init__()
        self._current_stage = FxStage.inference

    def process(self, gm: fx.GraphModule) -> bool:
        raise NotImplementedError

    def set_current_stage(self, stage: FxStage):
        self._current_stage = stage

    @classmethod
    def filter(cls, config: XpuGraphConfig) -> bool:
        if cls.__name__ in config.skip_patterns:
            logger.debug(f"Skip {cls._opt_level} pattern {cls.__name__}")
            return False
        if cls.__name__ in config.include_patterns:
            logger.debug(f"Add {cls._opt_level} pattern {cls.__name__}")
            return True
        return cls._opt_level <= config.opt_level


def collect_patterns(package_name, package_path, config, factory=lambda cls: cls()):
    """Instantiate every Pattern subclass defined in the modules of a package that
    passes `filter(config)`; `factory` may return None to skip a class."""
    import importlib
    import pkgutil

    groups = {g: [] for g in PatternGroup}
    for _, mod_name, _ in pkgutil.iter_modules(package_path):
        module = importlib.import_module(f"{package_name}.{mod_name}")
        for attr in dir(module):
            cls = getattr(module, attr)
            if (
                isinstance(cls, type)
                and issubclass(cls, Pattern)
                and cls is not Pattern
                and cls.__module__ == module.__name__
                and not attr.startswith("_")
                and cls.filter(config)
            ):
                inst = factory(cls)
                if inst is not None:
                    groups[cls._pattern_group].append(inst)
    return groups
