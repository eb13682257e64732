"""Recognisers for RMSNorm and LayerNorm written out in Aten ops.

    FusedRMSNorm / FusedLayerNorm   subgraph -> call_module(DefaultRMSNorm / DefaultLayerNorm)
    RemoveRMSNormCast / RemoveLayerNormCast   drop fp32 up/down casts around those modules

The accepted spellings are those of the reference matchers
(src/xpu_graph/passes/patterns/common/fuse_rmsnorm.py:29-193,
fuse_layernorm.py:32-255): x * rsqrt(..) / x / sqrt(..) / pow(.., +-0.5); the
square as pow 2, x*x or aten.square; eps on either side of the add; mean over
[-1] with keepdim; every intermediate used only inside the pattern.  For
LayerNorm the variance may be aten.var.dim or aten.var.correction with
correction 0 (what `unbiased=False` traces to on current torch).
"""
from torch import fx

from ....config import OptLevel
from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.default_replacements import DefaultLayerNorm, DefaultRMSNorm
from ..utils.node_utils import arg, aten, is_call, is_cast, kwarg, same_shape, shape, sole_user_is

_NUM = (int, float)
RMS_NAME = "fused_rms_norm"
LN_NAME = "fused_layer_norm"


def _mul_or_div(node):
    """(lhs, rhs, is_div) for mul.Tensor / div.Tensor nodes, else None."""
    if is_call(node, aten.mul.Tensor, aten.div.Tensor):
        return arg(node, 0), arg(node, 1), node.target == aten.div.Tensor
    return None


def _is_pow(node, exponent):
    return is_call(node, aten.pow.Tensor_Scalar) and arg(node, 1) == exponent


def _inverse_root_operand(node, is_div):
    """If `node` computes sqrt(t) (divisor) or rsqrt(t) (multiplier), return t."""
    if is_div:
        ok = is_call(node, aten.sqrt.default) or _is_pow(node, 0.5)
    else:
        ok = is_call(node, aten.rsqrt.default) or _is_pow(node, -0.5)
    return arg(node, 0) if ok else None


def _split_eps_add(node):
    """add.Tensor(t, eps) or add.Tensor(eps, t) with a python-number eps -> (t, eps)."""
    if not is_call(node, aten.add.Tensor, aten.add.Scalar) or kwarg(node, "alpha") not in (None, 1):
        return None
    a, b = arg(node, 0), arg(node, 1)
    if isinstance(b, _NUM) and isinstance(a, fx.Node):
        return a, b
    if isinstance(a, _NUM) and isinstance(b, fx.Node):
        return b, a
    return None


def _last_dim_only(dims, src):
    """dims names exactly the last axis of `src` ([-1], or [rank-1] as library decompositions write it)."""
    if not isinstance(dims, (list, tuple)) or len(dims) != 1:
        return False
    return dims[0] == -1 or (isinstance(src, fx.Node) and "val" in src.meta and dims[0] == len(src.meta["val"].shape) - 1)


def match_unweighted_rmsnorm(node):
    """x * rsqrt(mean(x^2, -1, keepdim) + eps) in any accepted spelling -> (x, eps)."""
    parts = _mul_or_div(node)
    if parts is None:
        return None
    x, root, is_div = parts
    if not isinstance(root, fx.Node):
        return None
    inner = _inverse_root_operand(root, is_div)
    if inner is None and not is_div and isinstance(x, fx.Node):
        # rsqrt(..) * x : operands the other way round
        inner = _inverse_root_operand(x, False)
        if inner is not None:
            x, root = root, x
    if inner is None or not isinstance(x, fx.Node) or not isinstance(inner, fx.Node):
        return None
    if not sole_user_is(root, node) or not sole_user_is(inner, root):
        return None
    split = _split_eps_add(inner)
    if split is None:
        return None
    mean, eps = split
    if not sole_user_is(mean, inner):
        return None
    if not is_call(mean, aten.mean.dim) or not _last_dim_only(arg(mean, 1), arg(mean, 0)) or kwarg(mean, "keepdim") is not True:
        return None
    if kwarg(mean, "dtype") not in (None, mean.meta["val"].dtype if "val" in mean.meta else None, arg(mean, 0).meta["val"].dtype):
        return None  # a mean that also converts its input
    sq = arg(mean, 0)
    if not isinstance(sq, fx.Node) or not sole_user_is(sq, mean):
        return None
    if is_call(sq, aten.pow.Tensor_Scalar):
        ok = arg(sq, 0) is x and arg(sq, 1) == 2
    elif is_call(sq, aten.mul.Tensor):
        ok = arg(sq, 0) is x and arg(sq, 1) is x
    elif is_call(sq, aten.square.default):
        ok = arg(sq, 0) is x
    else:
        ok = False
    return (x, eps) if ok else None


def _module_call(node, cls):
    if not isinstance(node, fx.Node) or node.op != "call_module":
        return False
    return isinstance(getattr(node.graph.owning_module, node.target, None), cls)


def _emit(gm, node, name, args, stage):
    """Insert call_module(name, args) before `node`, cast back if the matched node's dtype differs, reroute users."""
    x = args[0]
    with gm.graph.inserting_before(node):
        new = gm.graph.call_module(name, args)
        if x.meta["val"].dtype != node.meta["val"].dtype:
            cast = aten.to.dtype if stage is FxStage.pregrad else aten._to_copy.default
            new = gm.graph.call_function(cast, (new,), {"dtype": node.meta["val"].dtype})
    node.replace_all_uses_with(new, propagate_meta=True)


class FusedRMSNorm(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        if not hasattr(gm, RMS_NAME):
            gm.add_module(RMS_NAME, DefaultRMSNorm())
        changed = False
        for node in gm.graph.nodes:
            m = match_unweighted_rmsnorm(node)
            if m is not None:
                _emit(gm, node, RMS_NAME, (m[0], None, m[1]), self._current_stage)
                changed = True
                continue
            if not is_call(node, aten.mul.Tensor):
                continue
            # unweighted module * weight[last_dim]
            a, b = node.args[0], node.args[1]
            bare = lambda n: _module_call(n, DefaultRMSNorm) and n.args[1] is None  # noqa: E731
            if bare(a):
                norm, weight = a, b
            elif bare(b):
                norm, weight = b, a
            else:
                continue
            if not isinstance(weight, fx.Node) or not same_shape(shape(norm)[-1:], shape(weight)):
                continue
            x, _, eps = norm.args
            _emit(gm, node, RMS_NAME, (x, weight, eps), self._current_stage)
            changed = True
        return changed


def _strip_casts(gm, node, name, n_tensor_args, stage):
    """Shared body of the Remove*Cast patterns: the module computes in fp32 anyway,
    so casts on its tensor inputs and a single trailing cast are redundant."""
    args = list(node.args)
    touched = False
    for i in range(n_tensor_args):
        if is_cast(args[i]):
            args[i] = arg(args[i], 0)
            touched = True
    if not touched:
        return False
    result = node
    if len(node.users) == 1 and is_cast(next(iter(node.users))):
        result = next(iter(node.users))
    with gm.graph.inserting_before(node):
        new = gm.graph.call_module(name, tuple(args))
        if args[0].meta["val"].dtype != result.meta["val"].dtype:
            cast = aten.to.dtype if stage is FxStage.pregrad else aten._to_copy.default
            new = gm.graph.call_function(cast, (new,), {"dtype": result.meta["val"].dtype})
    result.replace_all_uses_with(new, propagate_meta=True)
    return True


class RemoveRMSNormCast(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        if not hasattr(gm, RMS_NAME):
            gm.add_module(RMS_NAME, DefaultRMSNorm())
        changed = False
        for node in reversed(gm.graph.nodes):
            if _module_call(node, DefaultRMSNorm):
                changed |= _strip_casts(gm, node, RMS_NAME, 2, self._current_stage)
        return changed


def match_plain_layernorm(node):
    """(x - mean(x)) * rsqrt(var(x) + eps)  or  / sqrt(..) -> (x, eps)."""
    parts = _mul_or_div(node)
    if parts is None:
        return None
    centred, root, is_div = parts
    if not is_call(centred, aten.sub.Tensor) or not isinstance(root, fx.Node):
        return None
    x, mean = arg(centred, 0), arg(centred, 1)
    if not is_call(mean, aten.mean.dim) or arg(mean, 0) is not x or not _last_dim_only(arg(mean, 1), x) or arg(mean, 2) is not True:
        return None
    if not sole_user_is(mean, centred):
        return None
    inner = _inverse_root_operand(root, is_div)
    if inner is None or not isinstance(inner, fx.Node) or not sole_user_is(inner, root):
        return None
    split = _split_eps_add(inner)
    if split is None:
        return None  # a variance without eps has no python-number eps to hand to the module
    var, eps = split
    if not sole_user_is(var, inner):
        return None
    if not is_call(var, aten.var.dim, aten.var.correction):
        return None
    if arg(var, 0) is not x or not _last_dim_only(arg(var, 1), x) or kwarg(var, "keepdim") is not True:
        return None
    if kwarg(var, "unbiased") is not False and kwarg(var, "correction") != 0:
        return None
    return x, eps


class FusedLayerNorm(Pattern):
    """Does not fuse residual adds; that is a target pattern."""

    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        if not hasattr(gm, LN_NAME):
            gm.add_module(LN_NAME, DefaultLayerNorm())
        changed = False
        for node in gm.graph.nodes:
            m = match_plain_layernorm(node)
            if m is not None:
                with gm.graph.inserting_before(node):
                    new = gm.graph.call_module(LN_NAME, (m[0], None, None, m[1]))
                node.replace_all_uses_with(new, propagate_meta=True)
                changed = True
                continue
            if is_call(node, aten.mul.Tensor):
                a, b = node.args[0], node.args[1]
                bare = lambda n: _module_call(n, DefaultLayerNorm) and n.args[1] is None and n.args[2] is None  # noqa: E731
                if bare(a):
                    norm, weight = a, b
                elif bare(b):
                    norm, weight = b, a
                else:
                    continue
                x, _, _, eps = norm.args
                if not isinstance(weight, fx.Node) or not same_shape(shape(x)[-1:], shape(weight)):
                    continue
                _emit(gm, node, LN_NAME, (x, weight, None, eps), self._current_stage)
                changed = True
            elif is_call(node, aten.add.Tensor):
                a, b = node.args[0], node.args[1]
                unbiased = lambda n: _module_call(n, DefaultLayerNorm) and n.args[2] is None  # noqa: E731
                through_cast = lambda n: is_cast(n) and unbiased(arg(n, 0))  # noqa: E731
                if unbiased(a):
                    norm, bias = a, b
                elif unbiased(b):
                    norm, bias = b, a
                elif through_cast(a):
                    norm, bias = arg(a, 0), b
                elif through_cast(b):
                    norm, bias = arg(b, 0), a
                else:
                    continue
                x, weight, _, eps = norm.args
                if not isinstance(bias, fx.Node) or not same_shape(shape(x)[-1:], shape(bias)):
                    continue
                _emit(gm, node, LN_NAME, (x, weight, bias, eps), self._current_stage)
                changed = True
        return changed


class RemoveLayerNormCast(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        if not hasattr(gm, LN_NAME):
            gm.add_module(LN_NAME, DefaultLayerNorm())
        changed = False
        for node in reversed(gm.graph.nodes):
            if _module_call(node, DefaultLayerNorm):
                changed |= _strip_casts(gm, node, LN_NAME, 3, self._current_stage)
        return changed
