"""Left-leaning add chains -> stack + sum(dim 0)
(reference src/xpu_graph/passes/patterns/common/fuse_addn.py:14-76).

Only the left operand is followed, so the accumulation order of the chain
((t0 + t1) + t2) + ... is the order of the stacked list.  Links must be
tensor + tensor of identical shape and dtype, inner links single-use, and the
chain must have at least FUSED_ADDN_LIMIT operands.
"""
import torch
from torch import fx

from ....config import OptLevel
from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.node_utils import aten, is_call, same_shape

FUSED_ADDN_LIMIT = 4


def _is_link(node):
    if not is_call(node, aten.add.Tensor):
        return False
    a, b = node.args[0], node.args[1]
    if not (isinstance(a, fx.Node) and isinstance(b, fx.Node)):
        return False
    va, vb = a.meta.get("val"), b.meta.get("val")
    if not (isinstance(va, torch.Tensor) and isinstance(vb, torch.Tensor)):
        return False
    if len(node.args) > 2 or node.kwargs.get("alpha", 1) != 1:
        return False
    return same_shape(va.shape, vb.shape) and va.dtype == vb.dtype


def collect_chain(top, links):
    """Operands of the chain ending in `top`, left to right, and the add nodes it spans."""
    operands, spanned = [top.args[1]], [top]
    cur = top
    while True:
        left = cur.args[0]
        if left in links and len(left.users) == 1:
            operands.append(left.args[1])
            spanned.append(left)
            cur = left
        else:
            operands.append(left)
            break
    operands.reverse()
    return operands, spanned


class FusedAddN(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.forward, FxStage.pregrad, FxStage.backward]

    def process(self, gm):
        g = gm.graph
        links = [n for n in reversed(g.nodes) if _is_link(n)]
        link_set = set(links)
        changed = False
        for top in links:
            if top not in link_set:
                continue  # already consumed by a longer chain
            operands, spanned = collect_chain(top, link_set)
            if len(operands) < FUSED_ADDN_LIMIT:
                continue
            with g.inserting_before(top):
                stack = g.create_node("call_function", aten.stack.default, (operands,), name=top.name + "_fusedaddn_stack")
                total = g.create_node("call_function", aten.sum.dim_IntList, (stack, [0]), name=top.name + "_fusedaddn_sum")
            top.replace_all_uses_with(total)
            for n in spanned:
                link_set.discard(n)
                if len(n.users) == 0:
                    g.erase_node(n)
            changed = True
        return changed
