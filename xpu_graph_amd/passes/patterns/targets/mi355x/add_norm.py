"""Residual add feeding a norm module -> one fused launch.

    y = norm(add(x, residual), ...)            ->  add_*_norm_only(x, residual, ...)
    y = norm(h := add(x, residual), ...); h used elsewhere
                                               ->  (y, h) = add_*_norm(x, residual, ...)

Working counterpart of the reference's switched-off MLU patterns
(passes/patterns/targets/mlu/fuse_add_norm.py:86-215) and of the NPU
FusedAddRmsnorm (passes/patterns/targets/npu/fuse_add_rmsnorm.py:28-115), with
the module signature of FusedNormReplacement.forward (fuse_add_norm.py:21-83).
The kernel rounds the sum to the storage dtype before taking statistics, so the
second output is bit-identical to the eager add and eps is the matched one.
"""
import operator

import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern
from ...utils.node_utils import aten, hoist_users_after, is_call, norm_module_kind, same_shape

FUSED_NAME = "mi355x_fused_add_norm"


class FusedNormReplacement(nn.Module):
    def forward(self, input, residual, weight, bias, residual_bias, eps, store_output_before_norm, norm_type):
        dtype = torch.promote_types(input.dtype, residual.dtype)
        input, residual = input.to(dtype), residual.to(dtype)
        if residual_bias is not None:
            residual = residual + residual_bias
        ops = torch.ops.xpu_ops
        if norm_type == "layer_norm":
            if store_output_before_norm:
                return ops.add_layer_norm(input, residual, weight, bias, eps)
            return ops.add_layer_norm_only(input, residual, weight, bias, eps)
        if store_output_before_norm:
            return ops.add_rms_norm(input, residual, weight, eps)
        return ops.add_rms_norm_only(input, residual, weight, eps)


def match_add_norm(node, kind):
    if norm_module_kind(node) != kind:
        return None
    add = node.args[0]
    if not is_call(add, aten.add.Tensor) or len(add.args) > 2 or add.kwargs.get("alpha", 1) != 1:
        return None
    x, res = add.args[0], add.args[1]
    if not (isinstance(x, fx.Node) and isinstance(res, fx.Node)):
        return None
    vx, vr = x.meta.get("val"), res.meta.get("val")
    if not (isinstance(vx, torch.Tensor) and isinstance(vr, torch.Tensor)):
        return None
    if not same_shape(vx.shape, vr.shape):
        return None
    # the kernel adds in one dtype; a promoting add keeps its own node
    if vx.dtype != vr.dtype or vx.dtype != add.meta["val"].dtype:
        return None
    if kind == "layer_norm":
        _, weight, bias, eps = node.args
    else:
        _, weight, eps = node.args
        bias = None
    if weight is None:
        return None
    store = len(add.users) > 1
    return add, (x, res, weight, bias, None, eps, store, kind)


def _rewrite(gm, kind):
    if not hasattr(gm, FUSED_NAME):
        gm.add_submodule(FUSED_NAME, FusedNormReplacement())
    g = gm.graph
    changed = False
    for node in reversed(g.nodes):
        m = match_add_norm(node, kind)
        if m is None:
            continue
        add, params = m
        with g.inserting_before(node):
            fused = g.call_module(FUSED_NAME, args=params)
            if params[6]:
                y = g.call_function(operator.getitem, (fused, 0))
                h = g.call_function(operator.getitem, (fused, 1))
            else:
                y, h = fused, None
        node.replace_all_uses_with(y)
        g.erase_node(node)
        if h is not None:
            add.replace_all_uses_with(h)
            hoist_users_after(h)  # other users of the sum may sit between the add and the norm
        g.erase_node(add)
        changed = True
    return changed


class FusedAddLayerNorm(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]  # the fused ops carry backward formulas

    def process(self, gm):
        return _rewrite(gm, "layer_norm")


class FusedAddRMSNorm(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]  # the fused ops carry backward formulas

    def process(self, gm):
        return _rewrite(gm, "rms_norm")
