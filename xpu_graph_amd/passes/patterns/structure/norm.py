"""DefaultRMSNorm / DefaultLayerNorm call_module nodes -> the target's norm module
(reference structure/custom_rmsnorm.py:10-31, structure/custom_layernorm.py:10-31).
Only affine norms are swapped: RMSNorm needs a weight, LayerNorm weight and bias."""
import torch

from ....config import OptLevel
from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.default_replacements import DefaultLayerNorm, DefaultRMSNorm


def _swap(gm, default_cls, name, target_mod, needs):
    if not hasattr(gm, name):
        gm.add_submodule(name, target_mod())
    changed = False
    for node in gm.graph.nodes:
        if node.op != "call_module" or not isinstance(getattr(gm, node.target, None), default_cls):
            continue
        if any(node.args[i] is None for i in needs):
            continue
        with gm.graph.inserting_before(node):
            new = gm.graph.call_module(name, tuple(node.args))
        node.replace_all_uses_with(new, propagate_meta=True)
        changed = True
    return changed


class CustomRMSNorm(Pattern):
    _opt_level = OptLevel.level2
    # the reference keeps the custom norms out of training graphs (structure/custom_rmsnorm.py:12); here the
    # target's norm ops carry backward formulas, so the swap may also happen before autograd is traced
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def process(self, gm):
        return _swap(gm, DefaultRMSNorm, "custom_rms_norm", self.target_mod, needs=(1,))


class CustomLayerNorm(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def process(self, gm):
        return _swap(gm, DefaultLayerNorm, "custom_layer_norm", self.target_mod, needs=(1, 2))
