"""Predicates and accessors over FX nodes in Aten IR, shared by the matchers.

Covers the behaviour of the reference's helper module
(src/xpu_graph/passes/patterns/utils/check_ops.py:11-412): schema-normalised
argument access, op predicates, look-through of casts / views / clones and
use-count checks.
"""
import operator

import torch
from torch import fx
from torch.fx.experimental.symbolic_shapes import statically_known_true, sym_eq
from torch.fx.operator_schemas import normalize_function, normalize_module

aten = torch.ops.aten

VIEW_OPS = (aten.view.default, aten._unsafe_view.default, aten.reshape.default)
ACTIVATIONS = {
    aten.silu.default: "silu",
    aten.gelu.default: "gelu",
    aten.relu.default: "relu",
    aten.sigmoid.default: "sigmoid",
}


def is_call(node, *targets):
    """True when `node` is a call_function node whose target is one of `targets`."""
    return isinstance(node, fx.Node) and node.op == "call_function" and node.target in targets


def _normalised(node, only_kwargs):
    if node.op == "call_function":
        return normalize_function(node.target, node.args, node.kwargs, normalize_to_only_use_kwargs=only_kwargs)
    if node.op == "call_module":
        return normalize_module(node.graph.owning_module, node.target, node.args, node.kwargs, normalize_to_only_use_kwargs=only_kwargs)
    return None


def arg(node, idx):
    """Positional argument `idx` after filling defaults from the op schema (None if absent)."""
    norm = _normalised(node, False)
    if norm is None:
        return None
    args = norm[0]
    return args[idx] if -len(args) <= idx < len(args) else None


def kwarg(node, key):
    norm = _normalised(node, True)
    if norm is None:
        return None
    return norm[1].get(key)


def val(node):
    return node.meta["val"]


def shape(node):
    return node.meta["val"].shape


def dtype(node):
    return node.meta["val"].dtype


def has_val(node):
    return isinstance(node, fx.Node) and "val" in node.meta


def is_tensor_node(node):
    return has_val(node) and isinstance(node.meta["val"], torch.Tensor)


def rank(node):
    return len(node.meta["val"].shape)


def _dim_value(d):
    """A graph node that stands for a size (sym_size of a dynamic dim) compares by the symbol it carries."""
    if isinstance(d, fx.Node):
        return d.meta.get("val")
    return d


def same_shape(a, b):
    """Provably equal shapes; entries may be ints, SymInts or size-valued graph nodes.  Unknown -> False."""
    a = [_dim_value(d) for d in (a if isinstance(a, (list, tuple, torch.Size)) else [a])]
    b = [_dim_value(d) for d in (b if isinstance(b, (list, tuple, torch.Size)) else [b])]
    if len(a) != len(b) or any(d is None or isinstance(d, torch.Tensor) for d in a + b):
        return False
    return statically_known_true(sym_eq(a, b))


def sole_user_is(used, user):
    """Every use of `used` is `user` (so `used` disappears once `user` is rewritten)."""
    return all(u is user for u in used.users)


def is_cast(node):
    """A pure dtype conversion: _to_copy with only a dtype, or to.dtype."""
    if is_call(node, aten._to_copy.default):
        return len(node.kwargs) == 1 and "dtype" in node.kwargs
    return is_call(node, aten.to.dtype)


def is_view(node):
    return is_call(node, *VIEW_OPS)


def skip_layout_ops(node):
    """Walk up through _to_copy / view / clone nodes to the value they rearrange."""
    while is_call(node, aten._to_copy.default, aten.clone.default, *VIEW_OPS):
        node = node.args[0]
    return node


def activation_name(node):
    """Name of the activation a node applies, for the ops a dense epilogue can evaluate; a gelu that asks for the
    tanh approximation is not the erf gelu of the kernels."""
    if isinstance(node, fx.Node) and node.op == "call_function":
        name = ACTIVATIONS.get(node.target)
        if name == "gelu" and node.kwargs.get("approximate", "none") != "none":
            return None
        return name
    return None


def mm_operands(node):
    """(lhs, rhs) of mm, or of a matmul with a 2-D result; None otherwise."""
    if is_call(node, aten.mm.default) or (is_call(node, aten.matmul.default) and has_val(node) and rank(node) == 2):
        return node.args[0], node.args[1]
    return None


def strip_transpose(node):
    """(was_transposed, inner): looks through t() / transpose of the last two dims of a 2-D weight."""
    if is_call(node, aten.t.default):
        return True, node.args[0]
    if is_call(node, aten.transpose.int) and (node.args[1], node.args[2]) in ((0, 1), (1, 0), (-2, -1), (-1, -2)):
        return True, node.args[0]
    return False, node


def cat_axis(node):
    """Axis of a cat node, or None when `node` is not a cat."""
    if is_call(node, aten.cat.default, aten.concat.default):
        return node.args[1] if len(node.args) > 1 else node.kwargs.get("dim", 0)
    return None


def is_getitem(node):
    return is_call(node, operator.getitem)


def norm_module_kind(node):
    """'layer_norm' / 'rms_norm' for the call_module nodes the norm patterns emit, else None."""
    if not isinstance(node, fx.Node) or node.op != "call_module":
        return None
    if node.target in ("fused_layer_norm", "custom_layer_norm"):
        return "layer_norm"
    if node.target in ("fused_rms_norm", "custom_rms_norm"):
        return "rms_norm"
    return None


def longest_run(items, pred):
    """(start, end) inclusive of the longest run of consecutive items satisfying pred, (-1, -1) if none
    (reference utils/match_sub_list.py:4-36)."""
    best = (-1, -1)
    best_len = 0
    start = None
    for i, it in enumerate(items):
        if pred(it):
            if start is None:
                start = i
            if i - start + 1 > best_len:
                best_len = i - start + 1
                best = (start, i)
        else:
            start = None
    return best


def fresh_submodule_name(gm, base):
    """base_0, base_1, ... : first name not yet taken on gm (reference utils/submodule_manager.py:7-29)."""
    i = 0
    while hasattr(gm, f"{base}_{i}"):
        i += 1
    return f"{base}_{i}"


def hoist_users_after(anchor):
    """Move users of `anchor` that precede it in graph order right behind it, then their users, and so on.
    Moving a node later never breaks its own inputs; the recursion repairs its outputs."""
    work = [anchor]
    while work:
        cur = work.pop()
        for user in list(cur.users):
            if user < cur:
                cur.append(user)
                work.append(user)


class SymShapes:
    """Maps symbolic sizes back to graph nodes that carry them, so a rewritten
    node can be given concrete-or-node shape arguments (reference utils/shape_utils.py:8-32)."""

    def __init__(self, graph):
        self._by_expr = {}
        for n in graph.nodes:
            v = n.meta.get("val")
            if isinstance(v, torch.SymInt):
                self._by_expr.setdefault(v.node.expr, n)

    def bind(self, dim):
        if not isinstance(dim, torch.SymInt):
            return dim
        expr = dim.node.expr
        if expr.is_Integer:
            return int(expr)
        return self._by_expr.get(expr)

    def bind_shape(self, shp):
        out = [self.bind(d) for d in shp]
        return None if any(d is None for d in out) else out
