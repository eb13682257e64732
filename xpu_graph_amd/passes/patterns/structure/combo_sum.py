"""Several sum(dim 1 | 2) over 3-D tensors that come out of one slice-gather
module -> one combo_sum module call returning a list
(reference structure/fuse_combosum.py:21-109)."""
import operator

import torch
from torch import fx

from ....config import OptLevel
from ..pattern import Pattern, PatternGroup
from ..utils.node_utils import aten, has_val, hoist_users_after, is_call, is_getitem, rank, skip_layout_ops

COMBO_NAME = "combo_sum"


def _from_slice_gather(node):
    return isinstance(node, fx.Node) and node.op == "call_module" and str(node.target).startswith("fuse_slice_cat")


def group_sums(gm):
    groups = {}
    for s in gm.graph.nodes:
        if not is_call(s, aten.sum.dim_IntList) or not has_val(s) or rank(s) != 2 or len(s.args) > 2:
            continue
        if s.args[1] not in ([1], [2]):
            continue
        src = skip_layout_ops(s.args[0])
        if not is_getitem(src) or not _from_slice_gather(src.args[0]):
            continue
        groups.setdefault((src.args[0], s.args[1][0]), []).append(s)
    return groups


class ComboSum3dInp(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP1

    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def process(self, gm):
        if not hasattr(gm, COMBO_NAME):
            gm.add_submodule(COMBO_NAME, self.target_mod())
        g = gm.graph
        changed = False
        for (_, dim), sums in group_sums(gm).items():
            last = sums[-1]
            with g.inserting_after(last):
                combo = g.call_module(COMBO_NAME, args=([s.args[0] for s in sums], [dim]))
            for i, old in enumerate(sums):
                with g.inserting_after(combo):
                    item = g.call_function(operator.getitem, (combo, i))
                old.replace_all_uses_with(item)
                hoist_users_after(item)
                g.erase_node(old)
            changed = True
        return changed
