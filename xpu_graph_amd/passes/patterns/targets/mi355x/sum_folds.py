"""Sums and copies that a kernel next to them can do on the way (no counterpart in the reference: its targets
leave these to the vendor compiler; here they are the Aten launches left between the HIP kernels of a training step).

    add(dense(x, w, .., residual=None, "none"), t)        ->  dense(x, w, .., residual=t, "none")
    add(rms_norm_bwd(.., gh=None)[0], t)                  ->  rms_norm_bwd(.., gh=t)[0]      (layer_norm_bwd alike)
    clone(v) where v is already laid out the way asked    ->  v

The first two appear where autograd sums the gradients of a value with several uses (the three projections of one
normalised input, the two branches of a residual stream); the kernels add their operand in fp32 before the one
rounding, so the result is at least as close to exact arithmetic as the separate sum.  The third is what
`x.transpose(1, 2).contiguous()` leaves behind when the producer already wrote x in the transposed layout.
"""
import operator

import torch
from torch import fx

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern
from ...utils.node_utils import VIEW_OPS, aten, is_call, same_shape, sole_user_is

_xpu = torch.ops.xpu_ops
_POST_AOT = [FxStage.inference, FxStage.forward, FxStage.backward]


def _tensor(node):
    v = node.meta.get("val") if isinstance(node, fx.Node) else None
    return v if isinstance(v, torch.Tensor) else None


def _plain_add(node):
    """(a, b) of add.Tensor with alpha 1 and no broadcasting or promotion, else None."""
    if not is_call(node, aten.add.Tensor) or len(node.args) != 2 or node.kwargs.get("alpha", 1) != 1:
        return None
    a, b = node.args
    va, vb, vo = _tensor(a), _tensor(b), _tensor(node)
    if va is None or vb is None or vo is None:
        return None
    if not (va.dtype == vb.dtype == vo.dtype) or not (same_shape(va.shape, vo.shape) and same_shape(vb.shape, vo.shape)):
        return None
    return a, b


def _dense_behind(node, user):
    """`node` is a dense call without residual or activation, or one reshape of it, used only by `user`:
    the dense node, else None."""
    if is_call(node, *VIEW_OPS) and sole_user_is(node, user) and len(node.users) == 1:
        inner = node.args[0]
        if is_call(inner, _xpu.dense.default) and sole_user_is(inner, node) and len(inner.users) == 1:
            node = inner
        else:
            return None
    elif not (sole_user_is(node, user) and len(node.users) == 1):
        return None
    if not is_call(node, _xpu.dense.default) or len(node.args) != 6:
        return None
    if node.args[4] is not None or node.args[5] != "none":
        return None
    return node


class FoldAddIntoDense(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = _POST_AOT

    def process(self, gm):
        g = gm.graph
        changed = False
        for add in list(g.nodes):
            ab = _plain_add(add)
            if ab is None:
                continue
            for mine, other in (ab, ab[::-1]):
                dense = _dense_behind(mine, add)
                if dense is None or other is dense:
                    continue
                vo, vd = _tensor(other), _tensor(dense)
                if vo.dtype != vd.dtype or not vo.is_contiguous():
                    continue
                with g.inserting_before(add):
                    res = other if same_shape(vo.shape, vd.shape) else g.call_function(aten.reshape.default, (other, list(vd.shape)))
                    new = g.call_function(_xpu.dense.default, dense.args[:4] + (res, "none"))
                    out = new if mine is dense else g.call_function(aten.reshape.default, (new, list(_tensor(add).shape)))
                add.replace_all_uses_with(out)
                g.erase_node(add)
                if mine is not dense:
                    g.erase_node(mine)
                g.erase_node(dense)
                changed = True
                break
        return changed


class FoldAddIntoNormBackward(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.backward]

    def process(self, gm):
        g = gm.graph
        changed = False
        for add in list(g.nodes):
            ab = _plain_add(add)
            if ab is None:
                continue
            for mine, other in (ab, ab[::-1]):
                if not (is_call(mine, operator.getitem) and mine.args[1] == 0):
                    continue
                bwd = mine.args[0]
                if not is_call(bwd, _xpu.rms_norm_bwd.default, _xpu.layer_norm_bwd.default) or len(bwd.args) < 7 or bwd.args[4] is not None:
                    continue
                if not (sole_user_is(mine, add) and len(mine.users) == 1):
                    continue
                vo = _tensor(other)
                if not vo.is_contiguous() or other is bwd:
                    continue
                # the kernel call moves down to the sum: its other results are selected again there, and what
                # uses them must come after that point
                others = [u for u in bwd.users if u is not mine]
                order = {n: i for i, n in enumerate(g.nodes)}
                if not all(is_call(u, operator.getitem) and all(order[w] > order[add] for w in u.users) for u in others):
                    continue
                with g.inserting_before(add):
                    new = g.call_function(bwd.target, bwd.args[:4] + (other,) + bwd.args[5:])
                    item = g.call_function(operator.getitem, (new, 0))
                    moved = [(u, g.call_function(operator.getitem, (new, u.args[1]))) for u in others]
                add.replace_all_uses_with(item)
                for u, v in moved:
                    u.replace_all_uses_with(v)
                    g.erase_node(u)
                g.erase_node(add)
                g.erase_node(mine)
                g.erase_node(bwd)
                changed = True
                break
        return changed


def _is_view_of_first_arg(node):
    """The node's result may share storage with its first argument: an operator whose schema says so, or the
    selection of one result of a multi-output call."""
    if node.op != "call_function":
        return False
    if node.target is operator.getitem:
        return True
    schema = getattr(node.target, "_schema", None)
    return schema is not None and any(r.alias_info is not None for r in schema.returns)


def _root(node):
    while isinstance(node, fx.Node) and _is_view_of_first_arg(node) and node.args and isinstance(node.args[0], fx.Node):
        node = node.args[0]
    return node


def _views_of(node, stop=None):
    """`node` and everything that may share its storage downstream (not looking past `stop`)."""
    seen, todo = [], [node]
    while todo:
        n = todo.pop()
        if n is stop or n in seen:
            continue
        seen.append(n)
        todo.extend(u for u in n.users if _is_view_of_first_arg(u) and u.args and u.args[0] is n)
    return seen


def _visible_outputs(gm):
    """(visible, all): the output values a caller can see and write to, and every output value.  The two differ
    only in a forward graph, where AOT appends the values saved for the backward after the `xg_user_outputs` it
    returns to the caller."""
    out = next(n for n in gm.graph.nodes if n.op == "output")
    results = out.args[0] if isinstance(out.args[0], (tuple, list)) else (out.args[0],)
    k = gm.meta.get("xg_user_outputs")
    visible, every = [], []
    fx.node.map_arg(tuple(results) if k is None else tuple(results[:k]), lambda n: visible.append(n))
    fx.node.map_arg(tuple(results), lambda n: every.append(n))
    return visible, every


class FoldCloneOfContiguous(Pattern):
    """clone(v) / clone(v, memory_format=contiguous) of a value that is already contiguous and whose storage this
    graph made itself: graphs at these stages are functional (nothing writes into v or the clone), so the copy
    only costs a pass over memory.  Kept when the copy and its source (or views of them) both leave the graph and
    the caller sees at least one of them: two results that were separate tensors must not come back sharing
    storage, and a result the caller may write into between forward and backward must not be the tensor that the
    backward saved.  Two values that are both only saved for the backward may share."""

    _opt_level = OptLevel.level2
    _support_stages = _POST_AOT

    def process(self, gm):
        g = gm.graph
        changed = False
        visible = None
        for node in list(g.nodes):
            if not is_call(node, aten.clone.default) or len(node.args) != 1:
                continue
            fmt = node.kwargs.get("memory_format", torch.preserve_format)
            if fmt not in (torch.contiguous_format, torch.preserve_format) or set(node.kwargs) - {"memory_format"}:
                continue
            src = node.args[0]
            vs, vn = _tensor(src), _tensor(node)
            if vs is None or vn is None or not vs.is_contiguous() or vs.stride() != vn.stride() or vs.numel() == 0:
                continue
            root = _root(src)
            if not (isinstance(root, fx.Node) and root.op in ("call_function", "call_module")) or _is_view_of_first_arg(root):
                continue  # an input, a constant, or a view of something this walk cannot follow
            if visible is None:
                visible, every = _visible_outputs(gm)
            copy_side, source_side = list(_views_of(node)), list(_views_of(root, stop=node))
            copy_seen, source_seen = any(n in visible for n in copy_side), any(n in visible for n in source_side)
            copy_out, source_out = any(n in every for n in copy_side), any(n in every for n in source_side)
            if (copy_seen and source_out) or (source_seen and copy_out):
                continue
            node.replace_all_uses_with(src)
            g.erase_node(node)
            changed = True
        return changed
