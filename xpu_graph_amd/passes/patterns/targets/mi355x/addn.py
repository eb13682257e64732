"""stack(list) + sum(dim 0)  ->  one add-N launch.

FusedAddN (a common pattern) turns long add chains into stack + sum, which
materialises the stacked tensor.  On this target the pair is replaced by a
kernel that reads the operands through a pointer table and accumulates left
to right in fp32 -- for fp32 tensors bit-identical to the original chain.
"""
import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern, PatternGroup
from ...utils.node_utils import aten, is_call, same_shape, sole_user_is

_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


class AddNModule(nn.Module):
    def forward(self, tensors):
        return torch.ops.xpu_ops.addn(list(tensors))


def match_stack_sum(node):
    if not is_call(node, aten.sum.dim_IntList) or len(node.args) > 2 and node.args[2]:
        return None
    if node.args[1] != [0] or node.kwargs.get("dtype") is not None:
        return None
    stack = node.args[0]
    if not is_call(stack, aten.stack.default) or not sole_user_is(stack, node):
        return None
    if len(stack.args) > 1 and stack.args[1] != 0:
        return None
    parts = list(stack.args[0])
    if len(parts) < 2 or not all(isinstance(p, fx.Node) for p in parts):
        return None
    first = parts[0].meta["val"]
    if first.dtype not in _DTYPES:
        return None
    for p in parts[1:]:
        v = p.meta["val"]
        if v.dtype != first.dtype or not same_shape(v.shape, first.shape):
            return None
    return stack, parts


class FusedStackSumToAddN(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP1
    _support_stages = [FxStage.inference]

    def process(self, gm):
        if not hasattr(gm, "mi355x_addn"):
            gm.add_submodule("mi355x_addn", AddNModule())
        g = gm.graph
        changed = False
        for node in reversed(list(g.nodes)):
            m = match_stack_sum(node)
            if m is None:
                continue
            stack, parts = m
            with g.inserting_before(node):
                new = g.call_module("mi355x_addn", args=(parts,))
            node.replace_all_uses_with(new)
            g.erase_node(node)
            g.erase_node(stack)
            changed = True
        return changed
