"""Attention ops -> the flash-style gfx950 kernel.

Handles `aten.scaled_dot_product_attention` (what FusedSDPA emits) and the
backend-specific ops it decomposes to when the user calls
F.scaled_dot_product_attention directly.  An additive mask that is a
compile-time constant equal to the causal mask (-inf or the dtype's lowest
value strictly above the diagonal, 0 elsewhere) is dropped and the kernel masks
by index; the reference never detects causality
(fuse_scaled_dot_product_attention.py:184-234 forwards the mask as attn_mask).
Any other floating-point additive mask ([Sq, Skv] with broadcast batch / head
dims) goes to the kernel as an operand, and so does the one-element scale
tensor of the reference's `xpu_graph::sdpa_wrapped_scale` form
(utils/default_replacements.py:39-55), which the kernel reads on the device
instead of the host reading it with .item().  In training graphs these two
forms are taken when the mask and the scale tensor need no gradient (the
backward kernels produce dq, dk, dv only); otherwise the Aten subgraph stays.

The rewrite also looks through the contiguous clones and 3-D reshapes FusedSDPA
puts in front of q, k, v: the kernel takes strides, so the [B, H, S, D] views
are passed as they are.
"""
import math

import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage, outside_fake_mode
from ...pattern import Pattern, PatternGroup
from ...utils.node_utils import VIEW_OPS, aten, is_call, is_getitem, same_shape

SDPA_NAME = "mi355x_sdpa"
SDPA_MASKED_NAME = "mi355x_sdpa_masked"
_DTYPES = (torch.bfloat16, torch.float16)
_HEAD_DIMS = (64, 128)
_MAX_CONST_ELEMS = 1 << 26


class SDPAModule(nn.Module):
    def forward(self, q, k, v, is_causal, scale):
        if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
            # a graph that will be differentiated: the forward also writes the log-sum-exp of every row, which is
            # all the backward kernels need beside q, k, v and the output
            return torch.ops.xpu_ops.sdpa_lse(q, k, v, is_causal, scale)[0]
        return torch.ops.xpu_ops.sdpa(q, k, v, is_causal, scale)


class SDPAMaskedModule(nn.Module):
    def forward(self, q, k, v, mask, scale_t, is_causal, scale):
        if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
            return torch.ops.xpu_ops.sdpa_masked_lse(q, k, v, mask, scale_t, is_causal, scale)[0]
        return torch.ops.xpu_ops.sdpa_masked(q, k, v, mask, scale_t, is_causal, scale)


def _needs_no_grad(node):
    """In a graph that will be differentiated: the operand is known not to require a gradient, i.e. every graph input
    it is computed from is marked as not requiring one (the pregrad stage marks the placeholders; an unmarked input
    counts as requiring a gradient)."""
    if not isinstance(node, fx.Node):
        return False
    seen, todo = set(), [node]
    while todo:
        n = todo.pop()
        if n in seen:
            continue
        seen.add(n)
        if n.op == "placeholder":
            if n.meta.get("xg_requires_grad", True):
                return False
        elif n.op == "get_attr":
            obj = n.graph.owning_module
            for part in n.target.split("."):
                obj = getattr(obj, part, None)
            if not isinstance(obj, torch.Tensor) or obj.requires_grad:
                return False
        else:
            todo.extend(n.all_input_nodes)
    return True


def _mask_operand_ok(mask, q, k):
    """A floating-point additive mask the kernel can index (see ops.sdpa_mask_fits), static in its last two dims."""
    from ..... import ops as _xops

    mv, qv, kv = mask.meta.get("val"), q.meta["val"], k.meta["val"]
    if not isinstance(mv, torch.Tensor) or not mv.dtype.is_floating_point or mv.dtype not in (qv.dtype, torch.float32):
        return False
    if not all(isinstance(d, int) for d in list(mv.shape)[-2:]):
        return False
    lead = list(mv.shape)[:-2]
    if any(not isinstance(d, int) and not same_shape([d], [qv.shape[0]]) for d in lead):
        return False
    shape = tuple(d if isinstance(d, int) else qv.shape[0] for d in mv.shape)
    return _xops.sdpa_mask_fits(shape, tuple(qv.shape), kv.shape[2])


def _const_eval(node, memo):
    """Value of a node computed from no graph input (factories, constants and ops on them), on CPU; None otherwise."""
    if node in memo:
        return memo[node]
    out = None
    if node.op == "get_attr":
        obj = node.graph.owning_module
        for part in node.target.split("."):
            obj = getattr(obj, part)
        out = obj.detach().cpu() if isinstance(obj, torch.Tensor) else None
    elif node.op == "call_function" and isinstance(node.target, torch._ops.OpOverload):
        v = node.meta.get("val")
        ok = isinstance(v, torch.Tensor) and all(isinstance(d, int) for d in v.shape) and v.numel() <= _MAX_CONST_ELEMS
        if ok and torch.Tag.nondeterministic_seeded not in node.target.tags:
            vals = {}
            for inp in node.all_input_nodes:
                vals[inp] = _const_eval(inp, memo)
                if vals[inp] is None:
                    ok = False
                    break
            if ok:
                args = fx.map_arg(node.args, lambda n: vals[n])
                kwargs = dict(fx.map_arg(node.kwargs, lambda n: vals[n]))
                if "device" in kwargs:
                    kwargs["device"] = torch.device("cpu")
                kwargs.pop("pin_memory", None)
                try:
                    out = node.target(*args, **kwargs)
                except Exception:
                    out = None
    memo[node] = out
    return out


def is_causal_constant(mask, sq, skv):
    """True when `mask` is a compile-time constant that broadcasts to the [sq, skv] causal additive mask."""
    if not isinstance(mask, fx.Node) or not isinstance(sq, int) or not isinstance(skv, int):
        return False
    with outside_fake_mode():
        val = _const_eval(mask, {})
        if not isinstance(val, torch.Tensor) or not val.dtype.is_floating_point:
            return False
        if val.dim() < 2 or val.shape[-2:] != (sq, skv):
            return False
        lead = val.reshape(-1, sq, skv)
        if not all(torch.equal(lead[0], lead[i]) for i in range(1, lead.shape[0])):
            return False
        m = lead[0].float()
        upper = torch.ones(sq, skv, dtype=torch.bool).triu(1)  # key j hidden from query i when j > i, as is_causal=True means
        lowest = torch.finfo(val.dtype).min
        masked = m[upper]
        return bool((m[~upper] == 0).all()) and bool(((masked == float("-inf")) | (masked <= lowest)).all())


def _static(*dims):
    return all(isinstance(d, int) for d in dims)


def _same_attention_problem(src, dims):
    """src is 4-D [B', H', S, D] with B'*H' == B*H and the same S, D: every (batch, head) pair is an
    independent attention problem, so how the leading two axes are split does not matter.  S, D and the head
    counts must be static; the batch may be symbolic."""
    if not (isinstance(src, fx.Node) and "val" in src.meta and isinstance(src.meta["val"], torch.Tensor)):
        return False
    shp = list(src.meta["val"].shape)
    dims = list(dims)
    if len(shp) != 4 or len(dims) != 4 or not _static(*shp[2:], *dims[2:]):
        return False
    if shp[2:] != dims[2:]:
        return False
    return same_shape([shp[0] * shp[1]], [dims[0] * dims[1]])


def _through_clone(node):
    """The contiguous copy FusedSDPA inserts may already have been folded away."""
    return node.args[0] if is_call(node, aten.clone.default) else node


def _peel_qv(node, dims):
    """reshape(clone(reshape(x4d, [BH,S,D])), [B,H,S,D]) -> x4d.  Reshapes reinterpret row-major order and clones
    copy, so any chain of them that ends in a 4-D tensor with the same S, D and number of heads is looked through
    (the clone, or one of the reshapes, may already have been folded away)."""
    cur, found = node, node
    while is_call(cur, *VIEW_OPS) or is_call(cur, aten.clone.default):
        cur = cur.args[0]
        if _same_attention_problem(cur, dims):
            found = cur  # keep going: a copy further up is looked through as well
    return found


def _peel_k(node, dims):
    """reshape(clone(transpose(reshape(transpose(k4d, -1, -2), [BH,D,S]), -1, -2)), [B,H,S,D]) -> k4d."""
    if not is_call(node, *VIEW_OPS):
        return node
    t1 = _through_clone(node.args[0])
    if not is_call(t1, aten.transpose.int) or {t1.args[1], t1.args[2]} not in ({-1, -2}, {1, 2}):
        return node
    r = t1.args[0]
    if not is_call(r, *VIEW_OPS):
        return node
    t0 = _through_clone(r.args[0])  # batched matmul materialises k^T when k is a strided view
    if not is_call(t0, aten.transpose.int) or {t0.args[1], t0.args[2]} not in ({-1, -2}, {2, 3}):
        return node
    src = t0.args[0]
    return src if _same_attention_problem(src, dims) else node


def _peel_repeat(node):
    """reshape(clone(expand(unsqueeze(x, 2), [B, Hkv, n, S, D])), [B, Hkv * n, S, D]) -> x: key/value heads repeated for
    grouped-query attention (`repeat_kv` of the HF decoders, `repeat_interleave(n, dim=1)`).  Query head h of the
    repeated tensor is key/value head h // n of x, which is how the kernels index fewer key/value heads."""
    if not is_call(node, *VIEW_OPS):
        return node
    inner = _through_clone(node.args[0])
    if not is_call(inner, aten.expand.default):
        return node
    src = inner.args[0]
    if not is_call(src, aten.unsqueeze.default) or src.args[1] != 2:
        return node
    x = src.args[0]
    vals = [n.meta.get("val") if isinstance(n, fx.Node) else None for n in (x, inner, node)]
    if not all(isinstance(t, torch.Tensor) for t in vals):
        return node
    xs, es, ns = (list(t.shape) for t in vals)
    if len(xs) != 4 or len(es) != 5 or len(ns) != 4 or not _static(*xs[1:], *es[1:], *ns[1:]):
        return node
    ok = es[1] == xs[1] and es[3:] == xs[2:] and ns[1] == xs[1] * es[2] and ns[2:] == xs[2:]
    ok = ok and same_shape([es[0]], [xs[0]]) and same_shape([ns[0]], [xs[0]])
    return x if ok else node


def _supported(q, k, v):
    """bf16 / f16 4-D operands, head dim 64 or 128, static head counts and sequence lengths (the batch may be
    symbolic), kv heads dividing the query heads."""
    vq, vk, vv = (n.meta.get("val") for n in (q, k, v))
    if not all(isinstance(t, torch.Tensor) and t.dim() == 4 for t in (vq, vk, vv)):
        return False
    if vq.dtype not in _DTYPES or vk.dtype != vq.dtype or vv.dtype != vq.dtype:
        return False
    B, H, Sq, D = vq.shape
    if not _static(H, Sq, D, *vk.shape[1:], *vv.shape[1:]):
        return False
    if D not in _HEAD_DIMS or vk.shape[-1] != D or vv.shape[-1] != D:
        return False
    if not (same_shape([vk.shape[0]], [B]) and same_shape([vv.shape[0]], [B])):
        return False
    if list(vv.shape[1:]) != list(vk.shape[1:]) or vk.shape[1] == 0 or H % vk.shape[1] != 0:
        return False
    return True


class FusedCausalSDPA(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP1
    _support_stages = [FxStage.inference, FxStage.pregrad]  # sdpa carries a backward formula

    def _emit(self, gm, node, q, k, v, causal, scale, replace, mask=None, scale_t=None):
        k0, v0 = _peel_repeat(k), _peel_repeat(v)
        if k0 is not k and v0 is not v and _supported(q, k0, v0):
            k, v = k0, v0  # grouped heads go to the kernel unrepeated (the copies that repeated them die with their last user)
        if scale is None:
            scale = 1.0 / math.sqrt(q.meta["val"].shape[-1])
        if not isinstance(scale, (int, float)):
            return False
        with gm.graph.inserting_before(node):
            if mask is None and scale_t is None:
                new = gm.graph.call_module(SDPA_NAME, args=(q, k, v, bool(causal), float(scale)))
            else:
                if not hasattr(gm, SDPA_MASKED_NAME):
                    gm.add_submodule(SDPA_MASKED_NAME, SDPAMaskedModule())
                new = gm.graph.call_module(SDPA_MASKED_NAME, args=(q, k, v, mask, scale_t, bool(causal), float(scale)))
        replace(new)
        return True

    def _wrapped_scale_calls(self, gm):
        """call_module nodes of SDPAWrappedScale (what FusedSDPA emits for a tensor-valued scale)."""
        from ...utils.default_replacements import SDPAWrappedScale

        for node in list(gm.graph.nodes):
            if node.op == "call_module" and isinstance(gm.get_submodule(node.target), SDPAWrappedScale) and len(node.args) == 5:
                yield node

    def process(self, gm):
        if not hasattr(gm, SDPA_NAME):
            gm.add_submodule(SDPA_NAME, SDPAModule())
        g = gm.graph
        changed = False
        backend_ops = {}
        for name, (drop_idx, causal_idx, bias_idx) in {
            "_scaled_dot_product_flash_attention": (3, 4, None),
            "_scaled_dot_product_flash_attention_for_cpu": (3, 4, None),
            "_scaled_dot_product_efficient_attention": (5, 6, 3),
            "_scaled_dot_product_cudnn_attention": (5, 6, 3),
        }.items():
            op = getattr(aten, name, None)
            if op is not None:
                backend_ops[op.default] = (drop_idx, causal_idx, bias_idx)

        for node in reversed(list(g.nodes)):
            if is_call(node, aten.scaled_dot_product_attention.default):
                q, k, v = node.args[:3]
                mask = node.args[3] if len(node.args) > 3 else node.kwargs.get("attn_mask")
                dropout = node.args[4] if len(node.args) > 4 else node.kwargs.get("dropout_p", 0.0)
                causal = node.args[5] if len(node.args) > 5 else node.kwargs.get("is_causal", False)
                scale = node.kwargs.get("scale")
                if dropout != 0.0:
                    continue
                # enable_gqa=True (query head h reads key/value head h // (H / Hkv)) is what the kernels do with fewer
                # key/value heads; _supported checks that the head counts divide
                gqa = bool(node.kwargs.get("enable_gqa", False))
                if not gqa and isinstance(q, fx.Node) and isinstance(k, fx.Node):
                    vq, vk = q.meta.get("val"), k.meta.get("val")
                    if isinstance(vq, torch.Tensor) and isinstance(vk, torch.Tensor) and vq.dim() == 4 and vk.dim() == 4 and vq.shape[1] != vk.shape[1]:
                        continue  # eager broadcasts (or refuses) differing head counts without the flag: not this kernel's rule
                if not all(isinstance(n, fx.Node) and isinstance(n.meta.get("val"), torch.Tensor) and n.meta["val"].dim() == 4 for n in (q, k, v)):
                    continue
                sq, skv = q.meta["val"].shape[2], k.meta["val"].shape[2]
                mask_operand = None
                if mask is not None:
                    if not causal and is_causal_constant(mask, sq, skv):
                        causal = True
                    elif (isinstance(mask, fx.Node) and (self._current_stage == FxStage.inference or _needs_no_grad(mask))
                          and _supported(q, k, v) and _mask_operand_ok(mask, q, k)):
                        mask_operand = mask  # the kernel adds it; q, k, v go as they are (no peeling: the mask is indexed by [B, H])
                    else:
                        continue
                if mask_operand is not None:
                    changed |= self._emit(gm, node, q, k, v, causal, scale, node.replace_all_uses_with, mask=mask_operand)
                    continue
                q2 = _peel_qv(q, q.meta["val"].shape)
                k2 = _peel_k(k, k.meta["val"].shape)
                v2 = _peel_qv(v, v.meta["val"].shape)
                lead_q = list(q2.meta["val"].shape[:2])
                same_lead = all(same_shape(list(n.meta["val"].shape[:2]), lead_q) for n in (k2, v2))
                peeled = q2 is not q and k2 is not k and v2 is not v and same_lead
                out_shape = list(node.meta["val"].shape)
                # shape argument of the reshape back: ints, with -1 for the one dim that may be symbolic (the batch)
                symbolic = [i for i, d in enumerate(out_shape) if not isinstance(d, int)]
                back_shape = [(-1 if i in symbolic else d) for i, d in enumerate(out_shape)]
                needs_back = peeled and not same_shape(list(q2.meta["val"].shape), out_shape)
                if needs_back and len(symbolic) > 1:
                    peeled = needs_back = False
                if peeled and not _supported(q2, k2, v2):
                    peeled = needs_back = False
                if not peeled:
                    q2, k2, v2 = q, k, v
                    # (with a symbolic batch FusedSDPA folds it into the head axis: only the peeled views qualify)
                    if not _supported(q, k, v):
                        continue

                def replace(new, old=node, reshape_back=needs_back, shp=back_shape):
                    if reshape_back:
                        with gm.graph.inserting_after(new):
                            new = gm.graph.call_function(aten.reshape.default, (new, shp))
                    old.replace_all_uses_with(new)

                changed |= self._emit(gm, node, q2, k2, v2, causal, scale, replace)
            elif node.op == "call_function" and node.target in backend_ops:
                drop_idx, causal_idx, bias_idx = backend_ops[node.target]
                users = list(node.users)
                if not users or not all(is_getitem(u) and u.args[1] == 0 for u in users):
                    continue
                args = node.args
                q, k, v = args[:3]
                dropout = args[drop_idx] if len(args) > drop_idx else node.kwargs.get("dropout_p", 0.0)
                causal = args[causal_idx] if len(args) > causal_idx else node.kwargs.get("is_causal", False)
                bias = (args[bias_idx] if len(args) > bias_idx else None) if bias_idx is not None else node.kwargs.get("attn_mask")
                if dropout != 0.0 or not _supported(q, k, v):
                    continue
                mask_operand = None
                if bias is not None:
                    # the additive bias of the memory-efficient backend op is the attn_mask of the call it came from
                    sq, skv = q.meta["val"].shape[2], k.meta["val"].shape[2]
                    if not causal and is_causal_constant(bias, sq, skv):
                        causal = True
                    elif self._current_stage == FxStage.inference and isinstance(bias, fx.Node) and _mask_operand_ok(bias, q, k):
                        mask_operand = bias
                    else:
                        continue

                def replace(new, users=users):
                    for u in users:
                        u.replace_all_uses_with(new)

                changed |= self._emit(gm, node, q, k, v, causal, node.kwargs.get("scale"), replace, mask=mask_operand)
        for node in self._wrapped_scale_calls(gm):
            q, k, v, mask, scale_t = node.args
            if not all(isinstance(n, fx.Node) and isinstance(n.meta.get("val"), torch.Tensor) for n in (q, k, v, scale_t)):
                continue
            if self._current_stage != FxStage.inference and not (_needs_no_grad(scale_t) and (mask is None or _needs_no_grad(mask))):
                continue
            if not _supported(q, k, v) or scale_t.meta["val"].numel() != 1:
                continue
            causal = False
            if mask is not None:
                sq, skv = q.meta["val"].shape[2], k.meta["val"].shape[2]
                if isinstance(mask, fx.Node) and is_causal_constant(mask, sq, skv):
                    mask, causal = None, True
                elif not (isinstance(mask, fx.Node) and _mask_operand_ok(mask, q, k)):
                    continue
            changed |= self._emit(gm, node, q, k, v, causal, 1.0, node.replace_all_uses_with, mask=mask, scale_t=scale_t)
        return changed
