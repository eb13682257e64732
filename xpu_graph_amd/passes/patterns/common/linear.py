"""mm + bias -> addmm (reference src/xpu_graph/passes/patterns/common/fuse_addmm.py:12-90).

Fires when one operand of an add.Tensor is an mm (or 2-D matmul) used only by
that add and the sum has the mm's shape.  A python-number / symbolic bias
becomes a scalar_tensor; a bias of another dtype is cast to the input's dtype,
and the result is cast back if the add had promoted it.
"""
import torch
from torch import fx

from ....config import OptLevel
from ....fx_utils import FxStage
from ..pattern import Pattern
from ..utils.node_utils import aten, is_call, mm_operands, same_shape


def bmm_operands(node):
    """(lhs, rhs) of a bmm, or of a matmul of two 3-D tensors; None otherwise."""
    if is_call(node, aten.bmm.default):
        return node.args[0], node.args[1]
    if is_call(node, aten.matmul.default) and all(isinstance(a, fx.Node) and "val" in a.meta and a.meta["val"].dim() == 3 for a in node.args[:2]):
        return node.args[0], node.args[1]
    return None


def match_mm_plus_bias(node, operands=mm_operands):
    if not is_call(node, aten.add.Tensor) or len(node.args) != 2 or node.kwargs.get("alpha", 1) != 1:
        return None  # add(mm, bias, alpha=a) scales the bias: not an addmm with beta = 1
    for mm, bias in ((node.args[0], node.args[1]), (node.args[1], node.args[0])):
        ops = operands(mm) if isinstance(mm, fx.Node) else None
        if ops is None:
            continue
        if len(mm.users) != 1 or not same_shape(node.meta["val"].shape, mm.meta["val"].shape):
            return None
        return bias, ops[0], ops[1]
    return None


class FusedAddMM(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.forward, FxStage.pregrad]
    _operands = staticmethod(mm_operands)
    _fused = aten.addmm.default
    _name = "addmm_replacement"

    def process(self, gm):
        g = gm.graph
        cast = aten.to.dtype if self._current_stage == FxStage.pregrad else aten._to_copy.default
        changed = False
        for node in reversed(g.nodes):
            m = match_mm_plus_bias(node, self._operands)
            if m is None:
                continue
            bias, x, w = m
            x_val = x.meta["val"]
            with g.inserting_before(node):
                if isinstance(bias, (int, float)) or (isinstance(bias, fx.Node) and not isinstance(bias.meta["val"], torch.Tensor)):
                    bias = g.create_node(
                        "call_function", aten.scalar_tensor.default, (bias,), {"dtype": x_val.dtype, "device": x_val.device}, name="bias_constant"
                    )
                elif bias.meta["val"].dtype != x_val.dtype:
                    bias = g.create_node("call_function", cast, (bias,), {"dtype": x_val.dtype}, name="bias_cast")
                new = g.create_node("call_function", self._fused, (bias, x, w), name=self._name)
                if x_val.dtype != node.meta["val"].dtype:
                    new = g.create_node("call_function", cast, (new,), {"dtype": node.meta["val"].dtype}, name="input_cast")
            node.replace_all_uses_with(new)
            g.erase_node(node)
            changed = True
        return changed


class FusedBAddBMM(FusedAddMM):
    """bmm + bias -> baddbmm, the batched twin of FusedAddMM (reference common/fuse_baddbmm.py:11-89)."""

    _operands = staticmethod(bmm_operands)
    _fused = aten.baddbmm.default
    _name = "baddbmm_replacement"


class DecomposeLinear(Pattern):
    """Pre-dispatch graphs keep `aten.linear(x, W, b)` whole; the dense patterns speak mm / addmm:

        linear(x, W, b)  ->  reshape(addmm(b, reshape(x, [-1, K]), t(W)), [..., N])      (mm without b)

    Only in the pregrad stage (after autograd is traced, linear is already decomposed this way)."""

    _opt_level = OptLevel.level2
    _support_stages = [FxStage.pregrad]

    def process(self, gm):
        g = gm.graph
        changed = False
        for node in list(g.nodes):
            if not is_call(node, aten.linear.default):
                continue
            x, w = node.args[0], node.args[1]
            bias = node.args[2] if len(node.args) > 2 else node.kwargs.get("bias")
            xv, wv = x.meta.get("val"), w.meta.get("val")
            if not isinstance(xv, torch.Tensor) or not isinstance(wv, torch.Tensor) or wv.dim() != 2 or xv.dim() < 1:
                continue
            if bias is not None and bias.meta["val"].dim() != 1:
                continue
            k, n = wv.shape[1], wv.shape[0]
            with g.inserting_before(node):
                x2 = x if xv.dim() == 2 else g.call_function(aten.reshape.default, (x, [-1, k]))
                wt = g.call_function(aten.t.default, (w,))
                y = g.call_function(aten.mm.default, (x2, wt)) if bias is None else g.call_function(aten.addmm.default, (bias, x2, wt))
                if xv.dim() != 2:
                    y = g.call_function(aten.reshape.default, (y, list(xv.shape[:-1]) + [n]))
            node.replace_all_uses_with(y)
            g.erase_node(node)
            changed = True
        return changed
