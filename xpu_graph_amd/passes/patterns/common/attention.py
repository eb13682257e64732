"""bmm -> [scale] -> [mask] -> softmax -> bmm  =>  aten.scaled_dot_product_attention
(reference src/xpu_graph/passes/patterns/common/fuse_scaled_dot_product_attention.py:21-242).

Walks back from the second bmm through casts / views / clones; accepts an
optional additive (or subtractive) mask, an optional mul / div scale (number,
symbol or one-element tensor) and baddbmm(mask, q, k) as the first product.  The
3-D bmm operands are made contiguous and reshaped to [B, H, S, D]; B and H come
from broadcasting the mask against [Sq, Skv].  No grouped-query attention.
Causality is not detected here: a causal mask travels as `attn_mask`; the
mi355x target pattern recognises it afterwards.
"""
import operator

import torch
import torch.fx as fx

from ....config import OptLevel
from ....fx_utils import FxStage
from ....utils import logger
from ...general import is_constant
from ..pattern import Pattern
from ..utils.default_replacements import SDPAWrappedScale
from ..utils.node_utils import SymShapes, arg, aten, is_call, kwarg, same_shape, skip_layout_ops


def attention_dims(q_shape, k_shape, v_shape, mask_shape):
    """[B, H, Sq, Skv, Dqk, Dv] from the 3-D operand shapes (k already as [BH, Skv, D]) and the mask shape, or None."""
    if not (len(q_shape) == 3 and len(k_shape) == 3 and len(v_shape) == 3):
        return None
    if not (
        same_shape(q_shape[0], k_shape[0])
        and same_shape(q_shape[0], v_shape[0])
        and same_shape(q_shape[-1], k_shape[-1])
        and same_shape(k_shape[1], v_shape[1])
    ):
        return None
    bh, sq, skv = q_shape[0], q_shape[1], k_shape[1]
    try:
        full = torch.broadcast_shapes(mask_shape, [sq, skv])
    except Exception:
        return None
    if len(full) > 4:
        return None
    if len(full) == 4:
        batch, heads = full[0], full[1]
    elif len(full) == 3:
        batch, heads = 1, full[0]
    else:
        batch, heads = 1, 1
    if heads == 1:
        if bh % batch != 0:
            return None
        return [batch, bh // batch, sq, skv, q_shape[-1], v_shape[-1]]
    if bh % heads != 0:
        return None
    return [bh // heads, heads, sq, skv, q_shape[-1], v_shape[-1]]


def _const_value(node):
    gm = node.graph.owning_module
    obj = gm
    for part in node.target.split("."):
        obj = getattr(obj, part)
    return obj.item() if isinstance(obj, torch.Tensor) and obj.numel() == 1 else obj


def match_attention(node):
    if not is_call(node, aten.bmm.default):
        return None
    probs, v = arg(node, 0), arg(node, 1)
    softmax = skip_layout_ops(probs)
    if not is_call(softmax, aten._softmax.default, aten._safe_softmax.default):
        return None
    sm_rank = len(softmax.meta["val"].shape)
    sm_dim = arg(softmax, 1)
    if not isinstance(sm_dim, int) or sm_dim % sm_rank != sm_rank - 1:
        return None  # attention normalises over the keys, the last dim of the scores
    if is_call(softmax, aten._softmax.default) and arg(softmax, 2):
        return None  # half_to_float: probabilities leave in fp32, which the fused op does not return
    cur = skip_layout_ops(softmax.args[0])

    mask, mask_added, has_mask = None, False, False
    if is_call(cur, aten.add.Tensor, aten.sub.Tensor) and kwarg(cur, "alpha") in (None, 1):
        mask, mask_added, has_mask = arg(cur, 1), cur.target == aten.add.Tensor, True
        cur = skip_layout_ops(cur.args[0])

    scale, scale_divides, has_scale = 1.0, False, False
    if is_call(cur, aten.mul.Tensor, aten.div.Tensor):
        scale, scale_divides, has_scale = arg(cur, 1), cur.target == aten.div.Tensor, True
        if isinstance(scale, fx.Node) and isinstance(scale.meta["val"], torch.Tensor):
            if scale.meta["val"].numel() != 1:
                return None
            if is_constant(scale):
                scale = _const_value(scale)
        cur = skip_layout_ops(arg(cur, 0))

    if is_call(cur, aten.bmm.default):
        q, k = arg(cur, 0), arg(cur, 1)
    elif is_call(cur, aten.baddbmm.default) and not has_mask and not has_scale and kwarg(cur, "beta") in (None, 1) and kwarg(cur, "alpha") in (None, 1):
        mask, q, k = arg(cur, 0), arg(cur, 1), arg(cur, 2)
        has_mask, mask_added = True, True
    else:
        if is_call(cur, aten.baddbmm.default):
            logger.debug("Flash attention pass: Too many add operations")
        return None

    if has_mask and isinstance(mask, fx.Node) and isinstance(mask.meta.get("val"), torch.Tensor):
        # what aten.scaled_dot_product_attention accepts as an additive mask: fp32 or the dtype of q
        if mask.meta["val"].dtype not in (torch.float32, q.meta["val"].dtype):
            return None
    k_shape = k.meta["val"].shape
    k_shape = tuple(k_shape[:-2]) + (k_shape[-1], k_shape[-2])
    mask_shape = mask.meta["val"].shape if has_mask and isinstance(mask, fx.Node) else []
    dims = attention_dims(q.meta["val"].shape, k_shape, v.meta["val"].shape, mask_shape)
    if dims is None:
        return None
    return q, k, v, scale, scale_divides, mask, mask_added, dims


def match_attention_predispatch(node):
    """The same chain as it looks BEFORE dispatch (the `pregrad` stage of a training graph), on 4-D [B, H, S, D]
    operands: matmul(q, transpose(k)) -> [mul / div by a number] -> [add mask] -> softmax.int(-1[, float32]) ->
    [cast back] -> matmul(., v).  Returns (q, k, v, scale, mask) or None.  Equal head counts only; the mask, if any,
    has the dtype of q (what aten.scaled_dot_product_attention accepts)."""
    if not is_call(node, aten.matmul.default):
        return None
    probs, v = arg(node, 0), arg(node, 1)
    cast_back = is_call(probs, aten._to_copy.default) and set(probs.kwargs) == {"dtype"}
    softmax = probs.args[0] if cast_back else probs
    if not is_call(softmax, aten.softmax.int):
        return None
    scores, sm_dim, sm_dtype = arg(softmax, 0), arg(softmax, 1), arg(softmax, 2)
    if not (isinstance(scores, fx.Node) and isinstance(scores.meta.get("val"), torch.Tensor)):
        return None
    sm_rank = len(scores.meta["val"].shape)
    if sm_rank != 4 or not isinstance(sm_dim, int) or sm_dim % sm_rank != sm_rank - 1:
        return None
    vv = v.meta.get("val") if isinstance(v, fx.Node) else None
    if not isinstance(vv, torch.Tensor) or probs.meta["val"].dtype != vv.dtype:
        return None  # the probabilities must enter the second product in the dtype of v
    if sm_dtype not in (None, torch.float32, vv.dtype):
        return None
    cur = scores
    mask = None
    if is_call(cur, aten.add.Tensor) and kwarg(cur, "alpha") in (None, 1):
        mask, cur = arg(cur, 1), arg(cur, 0)
        if not (isinstance(mask, fx.Node) and isinstance(mask.meta.get("val"), torch.Tensor) and mask.meta["val"].dtype == vv.dtype):
            return None
    scale = 1.0
    if is_call(cur, aten.mul.Tensor, aten.div.Tensor):
        factor = arg(cur, 1)
        if not isinstance(factor, (int, float)) or (cur.target == aten.div.Tensor and factor == 0):
            return None
        scale = float(factor) if cur.target == aten.mul.Tensor else 1.0 / float(factor)
        cur = arg(cur, 0)
    if not is_call(cur, aten.matmul.default):
        return None
    q, kt = arg(cur, 0), arg(cur, 1)
    if is_call(kt, aten.transpose.int) and {arg(kt, 1) % 4, arg(kt, 2) % 4} == {2, 3}:
        k = arg(kt, 0)
    else:
        return None
    vals = [t.meta.get("val") if isinstance(t, fx.Node) else None for t in (q, k)]
    if not all(isinstance(t, torch.Tensor) and t.dim() == 4 and t.dtype == vv.dtype for t in vals) or vv.dim() != 4:
        return None
    qv, kv = vals
    if not (same_shape(qv.shape[:2], kv.shape[:2]) and same_shape(kv.shape[:3], vv.shape[:3]) and same_shape(qv.shape[3], kv.shape[3])):
        return None
    if mask is not None:
        try:
            full = torch.broadcast_shapes(mask.meta["val"].shape, scores.meta["val"].shape)
        except Exception:
            return None
        if not same_shape(full, scores.meta["val"].shape):
            return None
    return q, k, v, scale, mask


class FusedSDPA(Pattern):
    _opt_level = OptLevel.level2
    # pregrad: beyond the reference (inference only, pattern.py:29), so that a hand-written attention in a training
    # graph reaches the target's attention kernels, which carry a backward
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def _process_predispatch(self, gm):
        g = gm.graph
        changed = False
        for node in reversed(g.nodes):
            m = match_attention_predispatch(node)
            if m is None:
                continue
            q, k, v, scale, mask = m
            with g.inserting_before(node):
                fused = g.call_function(aten.scaled_dot_product_attention.default, (q, k, v), {"attn_mask": mask, "scale": scale})
            fused.meta["val"] = node.meta.get("val")
            node.replace_all_uses_with(fused)
            changed = True
        return changed

    def process(self, gm):
        if self._current_stage == FxStage.pregrad:
            return self._process_predispatch(gm)
        g = gm.graph
        syms = SymShapes(g)
        inference = self._current_stage == FxStage.inference
        changed = False
        for node in reversed(g.nodes):
            m = match_attention(node)
            if m is None:
                continue
            q, k, v, scale, scale_divides, mask, mask_added, dims = m
            bound = syms.bind_shape(dims)
            out_shape = syms.bind_shape(node.meta["val"].shape)
            if bound is None or out_shape is None:
                continue
            B, H, Sq, Skv, Dqk, Dv = bound
            with g.inserting_before(node):
                wrapped = False
                if isinstance(scale, fx.Node) and isinstance(scale.meta["val"], torch.Tensor):
                    if self._opt_level > OptLevel.level2:
                        q = g.call_function(aten.div.Tensor if scale_divides else aten.mul.Tensor, (q, scale))
                        scale, scale_divides = 1.0, False
                    elif not inference:
                        logger.debug("Note: we currently do not provide SDPAWrappedScale.backward")
                        continue
                    else:
                        logger.warning("Unwrap scale for scaled_dot_product_attention, which may introduce extra sync")
                        wrapped = True
                if scale_divides:
                    if wrapped:
                        scale = g.call_function(aten.reciprocal.default, (scale,))
                    elif isinstance(scale, fx.Node):
                        scale = g.call_function(operator.truediv, (1.0, scale))
                    else:
                        scale = 1.0 / float(scale)
                k = g.call_function(aten.transpose.int, (k, -1, -2))
                contiguous = {"memory_format": torch.contiguous_format}
                q = g.call_function(aten.reshape.default, (g.call_function(aten.clone.default, (q,), contiguous), (B, H, Sq, Dqk)))
                k = g.call_function(aten.reshape.default, (g.call_function(aten.clone.default, (k,), contiguous), (B, H, Skv, Dqk)))
                v = g.call_function(aten.reshape.default, (g.call_function(aten.clone.default, (v,), contiguous), (B, H, Skv, Dv)))
                if mask is not None and not mask_added:
                    mask = g.call_function(aten.neg.default, (mask,)) if isinstance(mask, fx.Node) else -mask
                if wrapped:
                    if not hasattr(gm, "fused_sdpa"):
                        gm.add_submodule("fused_sdpa", SDPAWrappedScale())
                    fused = g.call_module("fused_sdpa", (q, k, v, mask, scale))
                else:
                    fused = g.call_function(aten.scaled_dot_product_attention.default, (q, k, v), {"attn_mask": mask, "scale": scale})
                out = g.call_function(aten.reshape.default, (fused, tuple(out_shape)))
            node.replace_all_uses_with(out)
            changed = True
        return changed
