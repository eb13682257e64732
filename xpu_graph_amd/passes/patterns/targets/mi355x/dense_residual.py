"""dense(x, W) + r  ->  dense with r as its residual.

    add(reshape?(dense(x, W, trans, None, "none")), r)   ->   reshape?(dense(x, W, trans, reshape(r, [M, N]), "none"))

The dense module follows the reference's convention that a 2-D `bias` is a
residual added in the epilogue (DenseLayerModule.forward,
targets/mlu/structure_replacements/dense_layer_modules.py:28-41), so the
residual add after an output projection costs no extra pass over the
activations.  `r` must have the output's shape and dtype, be defined before the
dense call, and the dense result must have no other user.
"""
import torch
from torch import fx

from .....config import OptLevel
from ...pattern import Pattern, PatternGroup
from ...structure.dense import DENSE_NAME
from ...utils.node_utils import VIEW_OPS, aten, is_call


def _val(n):
    v = n.meta.get("val") if isinstance(n, fx.Node) else None
    return v if isinstance(v, torch.Tensor) else None


def _dense_behind(node):
    """(dense node, view node or None) when `node` is a plain dense call or a reshape of one, each with one user."""
    view = None
    if is_call(node, *VIEW_OPS) and len(node.users) == 1:
        view, node = node, node.args[0]
    if isinstance(node, fx.Node) and node.op == "call_module" and node.target == DENSE_NAME and len(node.users) == 1:
        return node, view
    return None, None


class FusedDenseResidual(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP2

    def process(self, gm):
        changed = False
        order = {n: i for i, n in enumerate(gm.graph.nodes)}
        for add in [n for n in gm.graph.nodes if is_call(n, aten.add.Tensor)]:
            if len(add.args) != 2 or add.kwargs.get("alpha", 1) != 1:
                continue
            out = _val(add)
            for lhs, res in ((add.args[0], add.args[1]), (add.args[1], add.args[0])):
                dense, view = _dense_behind(lhs)
                rv, dv = _val(res), _val(dense) if dense is not None else None
                if dense is None or out is None or rv is None or dv is None:
                    continue
                if len(dense.args) < 5 or dense.args[3] is not None or dense.args[4] != "none":
                    continue
                if rv.dtype != dv.dtype or tuple(rv.shape) != tuple(out.shape) or tuple(_val(lhs).shape) != tuple(out.shape):
                    continue
                if not all(isinstance(d, int) for d in (*rv.shape, *dv.shape)) or order[res] > order[dense]:
                    continue
                with gm.graph.inserting_before(dense):
                    res2d = res if rv.dim() == 2 else gm.graph.call_function(aten.reshape.default, (res, list(dv.shape)))
                dense.args = (*dense.args[:3], res2d, dense.args[4])
                add.replace_all_uses_with(lhs)
                gm.graph.erase_node(add)
                for n in (dense, view):  # their values are the same tensors as before plus r: drop nothing, shapes are unchanged
                    if n is not None:
                        n.meta.pop("xg_in_sig", None)
                changed = True
                break
        return changed
