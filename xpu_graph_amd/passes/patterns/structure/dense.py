"""[activation](mm | addmm)(x, W or W^T) -> target dense module
(reference structure/custom_denselayer.py:18-99).

The module is called as (inputs, weight, weight_trans, bias | None, act_str).
The target's constraint function sees the FakeTensor values of the same
arguments and may veto the rewrite, which leaves the Aten subgraph in place."""
from torch import fx

from ....config import OptLevel
from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.node_utils import VIEW_OPS, activation_name, arg, aten, is_call, mm_operands, sole_user_is, strip_transpose

DENSE_NAME = "custom_dense_layer_replacement"


def match_dense(node):
    """([x, w, trans, bias, act], product node, reshape node | None): an activation applied to the product directly,
    or to one reshape of it (a linear layer on [B, S, H] input is view -> addmm -> view -> activation; an elementwise
    activation commutes with the view, which is then re-applied to the fused result)."""
    act = activation_name(node)
    view = None
    if act is None:
        act, lin = "none", node
    else:
        lin = node.args[0]
        if not isinstance(lin, fx.Node) or not sole_user_is(lin, node):
            return None
        if is_call(lin, *VIEW_OPS) and isinstance(lin.args[0], fx.Node) and sole_user_is(lin.args[0], lin):
            view, lin = lin, lin.args[0]
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
    return [x, w, trans, bias, act], lin, view


class CustomDenseLayer(Pattern):
    _opt_level = OptLevel.level2
    # pregrad as well: the target's dense op carries a backward formula (the reference keeps it to inference)
    _support_stages = [FxStage.inference, FxStage.pregrad]

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
            params, lin, view = m
            if not self.constraint_fn(*fx.map_arg(params, lambda n: n.meta["val"])):
                continue
            with g.inserting_before(node):
                new = g.call_module(DENSE_NAME, tuple(params))
                if view is not None:
                    new = g.call_function(view.target, (new,) + tuple(view.args[1:]), dict(view.kwargs))
            node.replace_all_uses_with(new)
            g.erase_node(node)
            if view is not None:
                g.erase_node(view)
            if lin is not node:
                g.erase_node(lin)
            changed = True
        return changed


BATCH_DENSE_NAME = "custom_batch_dense_layer_replacement"


def _strip_batched_transpose(node):
    """(was_transposed, inner) for a transpose of the last two dims of a 3-D weight."""
    if is_call(node, aten.transpose.int) and tuple(sorted(d % 3 for d in (node.args[1], node.args[2]))) == (1, 2):
        return True, node.args[0]
    if is_call(node, aten.permute.default) and list(node.args[1]) in ([0, 2, 1], [0, -1, -2]):
        return True, node.args[0]
    return False, node


def match_batch_dense(node):
    """[activation](bmm(x, W) | baddbmm(bias, x, W) | bmm(x, W) + bias) -> ([x, W, trans, bias, act], nodes to erase)
    (reference structure/custom_denselayer.py:40-68, 102-128)."""
    act = activation_name(node)
    dead = []
    if act is None:
        act, lin = "none", node
    else:
        lin = node.args[0]
        if not isinstance(lin, fx.Node) or not sole_user_is(lin, node):
            return None
        dead.append(lin)
    bias = None
    if is_call(lin, aten.add.Tensor) and lin.kwargs.get("alpha", 1) == 1 and len(lin.args) == 2:
        for prod, other in ((lin.args[0], lin.args[1]), (lin.args[1], lin.args[0])):
            if is_call(prod, aten.bmm.default) and sole_user_is(prod, lin) and isinstance(other, fx.Node):
                bias, dead, lin = other, dead + [prod], prod
                break
        else:
            return None
    if is_call(lin, aten.bmm.default):
        x, w = lin.args[0], lin.args[1]
    elif is_call(lin, aten.baddbmm.default) and bias is None:
        if lin.kwargs.get("beta", 1) != 1 or lin.kwargs.get("alpha", 1) != 1:
            return None
        bias, x, w = arg(lin, 0), arg(lin, 1), arg(lin, 2)
    else:
        return None
    trans, w = _strip_batched_transpose(w)
    return [x, w, trans, bias, act], dead


class CustomBatchDenseLayer(Pattern):
    _opt_level = OptLevel.level2

    def __init__(self, target_mod, constraint_fn=None):
        super().__init__()
        self.target_mod = target_mod
        self.constraint_fn = constraint_fn or (lambda *a: True)

    def process(self, gm):
        if not hasattr(gm, BATCH_DENSE_NAME):
            gm.add_submodule(BATCH_DENSE_NAME, self.target_mod())
        g = gm.graph
        changed = False
        for node in reversed(g.nodes):
            m = match_batch_dense(node)
            if m is None:
                continue
            params, dead = m
            if not self.constraint_fn(*fx.map_arg(params, lambda n: n.meta["val"])):
                continue
            with g.inserting_before(node):
                new = g.call_module(BATCH_DENSE_NAME, tuple(params))
            node.replace_all_uses_with(new)
            g.erase_node(node)
            for d in dead:
                if not d.users:
                    g.erase_node(d)
            changed = True
        return changed
