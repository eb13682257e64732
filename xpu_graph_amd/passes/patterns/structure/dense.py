"""[activation](mm | addmm)(x, W or W^T) -> target dense module
(reference structure/custom_denselayer.py:18-99).

The module is called as (inputs, weight, weight_trans, bias | None, act_str).
The target's constraint function sees the FakeTensor values of the same
arguments and may veto the rewrite, which leaves the Aten subgraph in place."""
from torch import fx

from ....config import OptLevel
from ..pattern import Pattern
from ..utils.node_utils import activation_name, arg, aten, is_call, mm_operands, sole_user_is, strip_transpose

DENSE_NAME = "custom_dense_layer_replacement"


def match_dense(node):
    act = activation_name(node)
    if act is None:
        act, lin = "none", node
    else:
        lin = node.args[0]
        if not isinstance(lin, fx.Node) or not sole_user_is(lin, node):
            return None
    ops = mm_operands(lin) if isinstance(lin, fx.Node) else None
    if ops is not None:
        x, w, bias = ops[0], ops[1], None
    elif is_call(lin, aten.addmm.default):
        if lin.kwargs.get("beta", 1) != 1 or lin.kwargs.get("alpha", 1) != 1:
            return None
        bias, x, w = arg(lin, 0), arg(lin, 1), arg(lin, 2)
    else:
        return None
    trans, w = strip_transpose(w)
    return [x, w, trans, bias, act], lin


class CustomDenseLayer(Pattern):
    _opt_level = OptLevel.level2

    def __init__(self, target_mod, constraint_fn=None):
        super().__init__()
        self.target_mod = target_mod
        self.constraint_fn = constraint_fn or (lambda *a: True)

    def process(self, gm):
        if not hasattr(gm, DENSE_NAME):
            gm.add_submodule(DENSE_NAME, self.target_mod(self._opt_level == OptLevel.level3))
        g = gm.graph
        changed = False
        for node in reversed(g.nodes):
            m = match_dense(node)
            if m is None:
                continue
            params, lin = m
            if not self.constraint_fn(*fx.map_arg(params, lambda n: n.meta["val"])):
                continue
            with g.inserting_before(node):
                new = g.call_module(DENSE_NAME, tuple(params))
            node.replace_all_uses_with(new)
            g.erase_node(node)
            if lin is not node:
                g.erase_node(lin)
            changed = True
        return changed
