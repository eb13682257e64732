"""Level-1 algebraic and shape clean-ups: operations that provably return one of their operands (or a constant)
are replaced by that operand, so that the matchers downstream see the graph without them.

Behaviour of the reference's fold_add.py / fold_sub.py / fold_mul.py / fold_div.py (x + 0, x - 0, 0 rsub x, x * 1,
x / 1), fold_detach.py, fold_squeeze.py, fold_stack.py, fold_where.py, fold_reduce.py, fold_slice_like.py and
change_tensor_like.py (src/xpu_graph/passes/patterns/common/).  A folded arithmetic node is replaced by a COPY of
the surviving operand, broadcast and converted to the node's own shape and dtype (reference
utils/get_binary_fold_result.py:10-57): the result of `x + 0` never aliases x; `FoldClone` drops the copy again
where that is safe.
"""
import torch
import torch.fx as fx

from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.node_utils import SymShapes, aten, arg, is_call, kwarg, same_shape

_ALL = [FxStage.inference, FxStage.pregrad, FxStage.forward, FxStage.backward]
_INT64_MAX = 9223372036854775807


def _is_const(x, value, makers):
    if type(x) in (int, float):
        return x == value
    return is_call(x, *makers)


def _is_zero(x):
    return _is_const(x, 0, (aten.zeros.default, aten.zeros_like.default))


def _is_one(x):
    return _is_const(x, 1, (aten.ones.default, aten.ones_like.default))


def _has_symbolic_dim(shape):
    return any(isinstance(d, torch.SymInt) for d in shape)


def _stand_in(graph, kept, like):
    """A node with the shape and dtype of FakeTensor `like` holding the value of `kept` (a scalar or a node), or
    None when that needs a symbolic size written out."""
    if type(kept) in (int, float):
        if _has_symbolic_dim(like.shape) or not like.is_contiguous():
            return None  # full(shape) is contiguous: a permuted result layout would be lost
        return graph.call_function(aten.full.default, (list(like.shape), kept), {"dtype": like.dtype, "device": like.device})
    have = kept.meta["val"]
    node = kept
    if not same_shape(have.shape, like.shape):
        if _has_symbolic_dim(like.shape):
            return None
        node = graph.call_function(aten.expand.default, (node, list(like.shape)))
    if have.dtype != like.dtype:
        return graph.call_function(aten._to_copy.default, (node,), {"dtype": like.dtype})
    return graph.call_function(aten.clone.default, (node,))


def _replace_with_operand(gm, node, kept):
    with gm.graph.inserting_before(node):
        res = _stand_in(gm.graph, kept, node.meta["val"])
    if res is None:
        return False
    node.replace_all_uses_with(res)
    gm.graph.erase_node(node)
    return True


def _fold_neutral(gm, targets, survivor):
    """Binary ops with a neutral operand: `survivor(node)` names the operand that IS the result, or None."""
    changed = False
    for n in reversed(list(gm.graph.nodes)):
        if not is_call(n, *targets) or "val" not in n.meta:
            continue
        kept = survivor(n)
        if kept is not None and _replace_with_operand(gm, n, kept):
            changed = True
    return changed


_NOTHING = object()


class FoldAdd0(Pattern):
    _support_stages = _ALL
    targets = (aten.add.Tensor, aten.add.Scalar)

    def survivor(self, n):
        a, b = n.args[0], n.args[1]
        return b if _is_zero(a) else (a if _is_zero(b) else None)

    def process(self, gm):
        return _fold_neutral(gm, self.targets, self.survivor)


class FoldSub0(Pattern):
    _support_stages = _ALL
    targets = (aten.sub.Tensor, aten.sub.Scalar, aten.rsub.Tensor, aten.rsub.Scalar)

    def survivor(self, n):
        a, b = n.args[0], n.args[1]
        if n.target in (aten.rsub.Tensor, aten.rsub.Scalar):  # rsub(a, b) = b - a
            return b if _is_zero(a) else None
        return a if _is_zero(b) else None

    def process(self, gm):
        return _fold_neutral(gm, self.targets, self.survivor)


class FoldMul1(Pattern):
    _support_stages = _ALL
    targets = (aten.mul.Tensor, aten.mul.Scalar)

    def survivor(self, n):
        a, b = n.args[0], n.args[1]
        return b if _is_one(a) else (a if _is_one(b) else None)

    def process(self, gm):
        return _fold_neutral(gm, self.targets, self.survivor)


class FoldDiv1(Pattern):
    _support_stages = _ALL
    targets = (aten.div.Tensor, aten.div.Scalar)

    def survivor(self, n):
        return n.args[0] if _is_one(n.args[1]) and not n.kwargs.get("rounding_mode") else None

    def process(self, gm):
        return _fold_neutral(gm, self.targets, self.survivor)


class FoldDetach(Pattern):
    """detach is an identity once no gradient is traced."""

    _support_stages = [FxStage.inference]

    def process(self, gm):
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, aten.detach.default)]:
            n.replace_all_uses_with(n.args[0])
            gm.graph.erase_node(n)
            changed = True
        return changed


_SQUEEZES = (aten.squeeze.default, aten.squeeze.dim, aten.squeeze.dims)


def _names_dim(squeeze_dims, d):
    return squeeze_dims == d if isinstance(squeeze_dims, int) else (len(squeeze_dims) == 1 and d in squeeze_dims)


class FoldSqueeze0(Pattern):
    """squeeze(squeeze(x)): an all-dims squeeze makes the inner one redundant, and is itself redundant after an
    all-dims inner squeeze."""

    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in reversed(list(gm.graph.nodes)):
            if not is_call(n, *_SQUEEZES):
                continue
            inner = n.args[0]
            if not is_call(inner, *_SQUEEZES) or len(inner.users) > 1:
                continue
            if len(n.args) == 1:
                n.replace_input_with(inner, inner.args[0])
                changed = True
            elif len(inner.args) == 1:
                n.replace_all_uses_with(inner)
                gm.graph.erase_node(n)
                changed = True
        return changed


class FoldSqueeze1(Pattern):
    """squeeze(unsqueeze(x, d)): the all-dims squeeze absorbs the unsqueeze; squeeze(., d) of the same d undoes it."""

    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in reversed(list(gm.graph.nodes)):
            if not is_call(n, *_SQUEEZES):
                continue
            inner = n.args[0]
            if not is_call(inner, aten.unsqueeze.default) or len(inner.users) > 1:
                continue
            if len(n.args) == 1:
                n.replace_input_with(inner, inner.args[0])
                changed = True
            elif _names_dim(n.args[1], inner.args[1]):
                n.replace_all_uses_with(inner.args[0])
                gm.graph.erase_node(n)
                changed = True
        return changed


class FoldStack(Pattern):
    """stack of ONE tensor is an unsqueeze of a copy; stack of all the pieces of an unbind along the same dim, in
    order, is a copy of the tensor that was taken apart."""

    _support_stages = _ALL

    @staticmethod
    def _whole_unbind(pieces):
        src = None
        for i, p in enumerate(pieces):
            if not (isinstance(p, fx.Node) and p.op == "call_function" and p.target.__name__ == "getitem"):
                return None
            if not is_call(p.args[0], aten.unbind.int) or p.args[1] != i or (src is not None and p.args[0] is not src):
                return None
            src = p.args[0]
        if src is None or len(pieces) != len(src.meta["val"]):
            return None
        return src

    def process(self, gm):
        changed = False
        for n in reversed([n for n in gm.graph.nodes if is_call(n, aten.stack.default)]):
            pieces = arg(n, 0)
            dim = kwarg(n, "dim") or 0
            if len(pieces) == 1:
                with gm.graph.inserting_before(n):
                    copy = gm.graph.call_function(aten.clone.default, (pieces[0],))
                    res = gm.graph.call_function(aten.unsqueeze.default, (copy, dim))
            else:
                unbind = self._whole_unbind(pieces)
                if unbind is None:
                    continue
                rank = len(n.meta["val"].shape)
                u_dim = kwarg(unbind, "dim") or 0
                if u_dim % rank != dim % rank:
                    continue
                with gm.graph.inserting_before(n):
                    res = gm.graph.call_function(aten.clone.default, (unbind.args[0],))
            n.replace_all_uses_with(res)
            gm.graph.erase_node(n)
            changed = True
        return changed


def _fill_value(node):
    """The scalar a constant-filled tensor node holds, or _NOTHING."""
    if is_call(node, aten.ones.default, aten.ones_like.default):
        return 1
    if is_call(node, aten.zeros.default, aten.zeros_like.default):
        return 0
    if is_call(node, aten.full.default, aten.full_like.default):
        return node.args[1]
    return _NOTHING


class FoldWhere(Pattern):
    """where(c, x, x) is x (also when both branches are all ones or all zeros); a full-size constant branch next to a
    tensor branch of the result's shape shrinks to one broadcast element."""

    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in reversed(list(gm.graph.nodes)):
            if not is_call(n, aten.where.self) or "val" not in n.meta:
                continue
            a, b = n.args[1], n.args[2]
            if a is b or (type(a) in (int, float) and type(b) in (int, float) and a == b) or (_is_one(a) and _is_one(b)) or (_is_zero(a) and _is_zero(b)):
                if _replace_with_operand(gm, n, a):
                    changed = True
                continue
            for pos, const, other in ((1, a, b), (2, b, a)):
                if not (isinstance(const, fx.Node) and isinstance(other, fx.Node) and isinstance(other.meta.get("val"), torch.Tensor)):
                    continue
                value = _fill_value(const)
                if value is _NOTHING or not same_shape(n.meta["val"].shape, other.meta["val"].shape):
                    continue
                have = const.meta["val"]
                if same_shape(have.shape, [1]):
                    continue  # already one element
                with gm.graph.inserting_before(n):
                    one = gm.graph.call_function(aten.full.default, ([1], value), {"device": have.device, "dtype": have.dtype})
                n.update_arg(pos, one)
                changed = True
                break
        return changed


class FoldReduce(Pattern):
    """A sum over dims that all have size 1 moves no data: a copy, squeezed unless keepdim."""

    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in reversed([n for n in gm.graph.nodes if is_call(n, aten.sum.dim_IntList)]):
            src = arg(n, 0)
            shp = src.meta["val"].shape
            dims = kwarg(n, "dim")
            if dims is None or dims == []:
                dims = list(range(len(shp)))
            if not isinstance(dims, (list, tuple)):
                dims = [dims]
            if not all(same_shape(shp[d], 1) for d in dims):
                continue
            if kwarg(n, "dtype") not in (None, src.meta["val"].dtype):
                continue  # an accumulate-in-wider-type request also converts
            with gm.graph.inserting_before(n):
                res = gm.graph.call_function(aten.clone.default, (src,))
                if not kwarg(n, "keepdim"):
                    res = gm.graph.call_function(aten.squeeze.dims, (res, list(dims)))
            n.replace_all_uses_with(res)
            gm.graph.erase_node(n)
            changed = True
        return changed


def _as_value(x):
    """An int, a SymInt (from a size-valued node) or None."""
    if isinstance(x, fx.Node):
        return x.meta.get("val")
    return x


class FoldSliceLike(Pattern):
    """slice(x, d, 0, len or more) is x; slice_scatter that overwrites ALL of its base is the source."""

    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        changed = False
        for n in list(gm.graph.nodes):
            if is_call(n, aten.slice.Tensor):
                src, dim, start, end, step = (arg(n, i) for i in range(5))
                if "val" not in src.meta or isinstance(start, fx.Node) or start not in (0, None) or step not in (1, None):
                    continue
                shp = src.meta["val"].shape
                if not -len(shp) <= dim < len(shp):
                    continue
                end = _as_value(end)
                whole = end is None or (isinstance(end, int) and end >= _INT64_MAX) or same_shape(end, shp[dim])
                if whole:
                    n.replace_all_uses_with(src)
                    gm.graph.erase_node(n)
                    changed = True
            elif is_call(n, aten.slice_scatter.default):
                base, src, dim, start, end, step = (arg(n, i) for i in range(6))
                if not all(isinstance(t, fx.Node) and "val" in t.meta for t in (base, src)):
                    continue
                if not isinstance(dim, int) or start not in (0, None) or step not in (1, None):
                    continue
                if not same_shape(base.meta["val"].shape, src.meta["val"].shape):
                    continue
                end = _as_value(end)
                length = src.meta["val"].shape[dim]
                if end is None or (isinstance(end, int) and end >= _INT64_MAX) or same_shape(end, length):
                    n.replace_all_uses_with(src)
                    gm.graph.erase_node(n)
                    changed = True
        return changed


class ChangeTensorLike(Pattern):
    """ones_like / zeros_like / full_like(t) become ones / zeros / full(shape of t): the constant no longer hangs on
    the tensor it copied its shape from, and constant folding can take it."""

    _support_stages = [FxStage.inference, FxStage.pregrad]
    _MAKERS = {aten.ones_like.default: aten.ones.default, aten.zeros_like.default: aten.zeros.default, aten.full_like.default: aten.full.default}

    def process(self, gm):
        changed = False
        shapes = SymShapes(gm.graph)
        for n in [n for n in gm.graph.nodes if is_call(n, *self._MAKERS)]:
            like = n.args[0]
            if "val" not in like.meta:
                continue
            fmt = n.kwargs.get("memory_format")
            if fmt not in (None, torch.preserve_format, torch.contiguous_format):
                continue
            if fmt is not torch.contiguous_format and not like.meta["val"].is_contiguous():
                continue  # the *_like result would copy the template's strides
            size = shapes.bind_shape(like.meta["val"].shape)
            if size is None:
                continue  # a symbolic size no graph node carries
            have = like.meta["val"]
            args = [size] + ([n.args[1]] if n.target is aten.full_like.default else [])
            kwargs = {k: (n.kwargs.get(k) if n.kwargs.get(k) is not None else getattr(have, k)) for k in ("dtype", "device", "layout")}
            if n.kwargs.get("pin_memory") is not None:
                kwargs["pin_memory"] = n.kwargs["pin_memory"]
            with gm.graph.inserting_before(n):
                res = gm.graph.call_function(self._MAKERS[n.target], tuple(args), kwargs)
            n.replace_all_uses_with(res)
            gm.graph.erase_node(n)
            changed = True
        return changed


def _close(a, b):
    return type(a) in (int, float) and abs(a - b) <= 1e-6 * max(1.0, abs(b))


def _factors(node, root=True):
    """Leaves of the product tree under `node` (a mul.Tensor): inner muls are opened when nothing else reads them."""
    if is_call(node, aten.mul.Tensor, aten.mul.Scalar) and (root or len(node.users) == 1):
        return _factors(node.args[0], False) + _factors(node.args[1], False)
    return [node]


def _split(factors, n_nodes):
    """(scalar product, node factors) when there are exactly n_nodes node factors, else None."""
    scalar, nodes = 1.0, []
    for f in factors:
        if isinstance(f, fx.Node):
            nodes.append(f)
        elif type(f) in (int, float):
            scalar *= f
        else:
            return None
    return (scalar, nodes) if len(nodes) == n_nodes else None


def _one_plus(node, inner_target):
    """node == 1 + inner_target(arg): returns the inner call, else None."""
    if not is_call(node, aten.add.Tensor, aten.add.Scalar) or kwarg(node, "alpha") not in (None, 1):
        return None
    a, b = node.args[0], node.args[1]
    inner = a if _close(b, 1.0) else (b if _close(a, 1.0) else None)
    return inner if is_call(inner, inner_target) else None


class Gelu(Pattern):
    """Hand-written GELU becomes aten.gelu, which the dense-layer pattern can then take as its activation:
    0.5 * x * (1 + erf(x / sqrt 2)) -> gelu(x);  0.5 * x * (1 + tanh(sqrt(2 / pi) * (x + 0.044715 x^3))) ->
    gelu(x, approximate="tanh").  Factors may come in any order and association (reference common/gelu.py:9-56,
    which maps the tanh form to the exact gelu; the approximation is kept here)."""

    _support_stages = [FxStage.inference, FxStage.pregrad]

    @staticmethod
    def _erf_form(x, plus):
        erf = _one_plus(plus, aten.erf.default)
        if erf is None:
            return False
        inner = erf.args[0]
        if is_call(inner, aten.div.Tensor, aten.div.Scalar):
            return inner.args[0] is x and _close(inner.args[1], 2**0.5) and not inner.kwargs.get("rounding_mode")
        if is_call(inner, aten.mul.Tensor, aten.mul.Scalar):
            got = _split(_factors(inner), 1)
            return got is not None and got[1][0] is x and _close(got[0], 0.5**0.5)
        return False

    @staticmethod
    def _cube_of(node, x):
        if is_call(node, aten.pow.Tensor_Scalar):
            return node.args[0] is x and _close(node.args[1], 3.0)
        got = _split(_factors(node), 3) if is_call(node, aten.mul.Tensor) else None
        return got is not None and _close(got[0], 1.0) and all(f is x for f in got[1])

    @classmethod
    def _tanh_form(cls, x, plus):
        tanh = _one_plus(plus, aten.tanh.default)
        if tanh is None or not is_call(tanh.args[0], aten.mul.Tensor, aten.mul.Scalar):
            return False
        got = _split(_factors(tanh.args[0]), 1)
        if got is None or not _close(got[0], (2.0 / 3.141592653589793) ** 0.5):
            return False
        poly = got[1][0]  # x + 0.044715 x^3
        if not is_call(poly, aten.add.Tensor) or kwarg(poly, "alpha") not in (None, 1):
            return False
        for lin, cub in ((poly.args[0], poly.args[1]), (poly.args[1], poly.args[0])):
            if lin is not x or not is_call(cub, aten.mul.Tensor, aten.mul.Scalar):
                continue
            parts = _factors(cub)
            scalar = 1.0
            rest = []
            for f in parts:
                if type(f) in (int, float):
                    scalar *= f
                else:
                    rest.append(f)
            if not _close(scalar, 0.044715):
                continue
            if len(rest) == 1 and cls._cube_of(rest[0], x):
                return True
            if len(rest) == 3 and all(f is x for f in rest):
                return True
        return False

    def process(self, gm):
        changed = False
        for n in reversed(list(gm.graph.nodes)):
            if not is_call(n, aten.mul.Tensor, aten.mul.Scalar) or "val" not in n.meta or not n.users:
                continue
            got = _split(_factors(n), 2)
            if got is None or not _close(got[0], 0.5):
                continue
            for x, plus in (got[1], got[1][::-1]):
                if "val" not in x.meta or x.meta["val"].shape != n.meta["val"].shape or x.meta["val"].dtype != n.meta["val"].dtype:
                    continue
                kind = "none" if self._erf_form(x, plus) else ("tanh" if self._tanh_form(x, plus) else None)
                if kind is None:
                    continue
                with gm.graph.inserting_before(n):
                    res = gm.graph.call_function(aten.gelu.default, (x,), {} if kind == "none" else {"approximate": "tanh"})
                n.replace_all_uses_with(res)
                changed = True
                break
        return changed

