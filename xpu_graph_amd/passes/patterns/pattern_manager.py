"""Owns every pattern and runs them: groups in order, five sweeps per group
(reference src/xpu_graph/passes/patterns/pattern_manager.py:14-139)."""
from typing import List

import torch.fx as fx

from ...config import OptLevel, XpuGraphConfig
from ...fx_utils import FxStage
from ...utils import logger
from ..optimizer import Optimizer
from .pattern import Pattern, PatternGroup

SWEEPS_PER_GROUP = 5


class PatternManager(Optimizer):
    def __init__(self, config: XpuGraphConfig):
        super().__init__()
        self._patterns = {g: [] for g in PatternGroup}
        self._enable_patterns = {g: [] for g in PatternGroup}
        from .common import get_all_patterns as common_patterns
        from .structure import get_all_patterns as structure_patterns
        from .targets import get_all_patterns as target_patterns

        for source in (common_patterns, structure_patterns, target_patterns):
            for group, pats in source(config).items():
                self._patterns[group].extend(pats)

    def reset_patterns_with_stage(self, stage: FxStage):
        self._enable_patterns = {g: [] for g in PatternGroup}
        for group, pats in self._patterns.items():
            for pat in pats:
                if stage in pat._support_stages:
                    pat.set_current_stage(stage)
                    self._enable_patterns[group].append(pat)
        for group, pats in self._enable_patterns.items():
            logger.debug(f"xpu_graph enable builtin {group} patterns: {[str(p) for p in pats]}")

    def get_pass_with_stage(self, stage):
        self.reset_patterns_with_stage(stage)
        return self

    def process(self, gm: fx.GraphModule) -> bool:
        changed = False
        for group in sorted(self._patterns):
            for _ in range(SWEEPS_PER_GROUP):
                for pat in self._enable_patterns[group]:
                    changed = changed or pat(gm)
        return changed

    def register_pattern(self, *args, **kwargs):
        """register_pattern(pattern) or register_pattern(matcher_fn, replacement_fn[, supported_stages=, opt_level=])."""
        if len(args) == 1:
            pat = args[0]
        elif len(args) == 2:
            matcher, replacement = args

            class _Pattern(Pattern):
                def __call__(self, gm):
                    from torch.fx import subgraph_rewriter

                    return len(subgraph_rewriter.replace_pattern(gm, matcher, replacement))

            if "supported_stages" in kwargs:
                _Pattern._support_stages = kwargs["supported_stages"]
            if "opt_level" in kwargs:
                _Pattern._opt_level = kwargs["opt_level"]
            pat = _Pattern()
        else:
            raise TypeError("register_pattern takes a Pattern, or a matcher and a replacement")
        if pat._opt_level <= self._opt_level:
            self._patterns[pat._pattern_group].append(pat)
            pat._set_level(self._opt_level)
        else:
            logger.warning(
                f"xpu_graph skip pattern {pat} with opt_level {pat._opt_level} and current opt_level is {self._opt_level}"
            )

    def insert_patterns(self, patterns: List[Pattern]):
        """Put `patterns` in front of the built-in ones of their groups (plugin patterns run first)."""
        front = {g: [] for g in PatternGroup}
        for pat in patterns:
            front[pat._pattern_group].append(pat)
        for group in self._patterns:
            self._patterns[group] = front[group] + self._patterns[group]

    def _set_level(self, level: OptLevel):
        self._opt_level = level
        for pats in self._patterns.values():
            for pat in pats:
                pat._set_level(level)
