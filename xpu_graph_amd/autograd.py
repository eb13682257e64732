"""Backward formulas for the custom ops that the `pregrad` stage may put into a training graph.

The forward of each op is its HIP kernel; the backward is written in Aten ops (fp32 math on the saved inputs,
statistics recomputed rather than saved), so AOT traces it into the backward graph like any other code and it runs
on the device the tensors live on.  Registered once per process, on demand (`ops.enable_autograd()`, called by a
backend constructed with is_training=True on the mi355x target): a Python autograd formula costs every call of the op
a few microseconds of dispatch, which inference-only processes should not pay.

    rms_norm(x, w, eps)        y = x * r * w,            r = rsqrt(mean(x^2) + eps)   (gradients: the fused
                               xg_rms_norm_bwd kernel, also for the add + RMSNorm ops; the Aten formula below is
                               for shapes the kernel does not take)
    layer_norm(x, w, b, eps)   y = (x - m) * r * w + b,  r = rsqrt(var(x) + eps)
    silu_mul2(g, u)            y = silu(g) * u          (gradients: the fused xg_silu_mul2_bwd kernel)
    silu_mul(x)                y = silu(x[..., :d]) * x[..., d:]
    dense(x, W, trans, bias, residual, act)   y = act(x W(^T) + bias + residual)
    dense_glu(x, Wg, Wu)       y = silu(x Wg^T) * (x Wu^T)
    rope(x, cos, sin)          y = x * cos + rotate_half(x) * sin,  rotate_half(x) = cat(-x[D/2:], x[:D/2])
    sdpa(q, k, v, causal, scale)   y = softmax(scale q k^T [+ causal mask]) v
    sdpa_lse(q, k, v, causal, scale)   the same, also returning the log-sum-exp of every row for the backward kernels
    sdpa_masked(q, k, v, mask, scale_t, causal, scale) / sdpa_masked_lse   with an additive mask and / or the scale in a
                               one-element tensor: gradients for q, k, v (the mask and the scale tensor get none)
    add_rms_norm(x, r, w, eps) / add_layer_norm(x, r, w, b, eps)   h = x + r, y = norm(h); returns (y, h)
    add_rms_norm_only / add_layer_norm_only                         the same, returning y alone

The input gradient of the dense layer is itself a dense layer over the same weight read the other way, so it runs on
the HIP kernel; the weight gradient is a product with a transposed LEFT operand (gz^T x), which the same kernel
takes in place through xpu_ops::dense_at (shapes it does not take -- a dimension that is no multiple of 8 -- fall to
an Aten matmul).  For activations whose derivative cannot be told from the output (silu, gelu) the pre-activation is
recomputed with one more dense call.  The gated layer saves only its inputs: both projections are recomputed on the
dense kernel, the two input-gradient products run as one chain (the second takes the first as its residual).
"""
import torch

_REGISTERED = False


def _reduce_to(grad, shape):
    """Sum `grad` over its leading dims down to `shape` (the shape of a weight that was broadcast over rows)."""
    extra = grad.dim() - len(shape)
    return grad.sum(dim=list(range(extra))) if extra > 0 else grad


def _rms_setup(ctx, inputs, output):
    x, w, eps = inputs
    ctx.save_for_backward(x, w) if w is not None else ctx.save_for_backward(x)
    ctx.has_w, ctx.eps = w is not None, eps


def _rms_kernel_backward(x, res, w, gy, gh, eps, want_gw):
    """(g_sum, gw | None) on the fused backward kernel when it takes the shape, else None."""
    from . import ops

    if not (x.is_cuda and ops.rms_norm_bwd_fits(x, w)) or (res is not None and res.dtype != x.dtype):
        return None
    gx, gw = torch.ops.xpu_ops.rms_norm_bwd(x, res, w, gy, gh, eps, want_gw)
    return gx, (gw if want_gw and w is not None else None)


def _bias_is_one_row(b_meta, x):
    """The bias is a plain [cols] vector: its gradient is the column sum the kernel accumulates."""
    return b_meta is not None and len(b_meta[0]) == 1 and b_meta[0][0] == x.shape[-1]


def _ln_kernel_backward(x, res, w, gy, gh, eps, want_gw, b_meta, want_gb):
    """(g_sum, gw | None, gb | None) on the fused backward kernel when it takes the shape, else None."""
    from . import ops

    if not (x.is_cuda and ops.rms_norm_bwd_fits(x, w)) or (res is not None and res.dtype != x.dtype):
        return None
    want_gb = bool(want_gb)
    gx, gw, gb = torch.ops.xpu_ops.layer_norm_bwd(x, res, w, gy, gh, eps, want_gw, want_gb)
    return gx, (gw if want_gw and w is not None else None), (gb.to(b_meta[1]) if want_gb else None)


def _rms_backward(ctx, gy):
    saved = ctx.saved_tensors
    x = saved[0]
    w = saved[1] if ctx.has_w else None
    fused = _rms_kernel_backward(x, None, w, gy, None, ctx.eps, ctx.needs_input_grad[1])
    if fused is not None:
        return fused[0], fused[1], None
    xf, gf = x.float(), gy.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + ctx.eps)
    xhat = xf * r
    gxhat = gf * w.float() if w is not None else gf
    gx = r * (gxhat - xhat * (gxhat * xhat).mean(-1, keepdim=True))
    gw = _reduce_to(gf * xhat, w.shape).to(w.dtype) if w is not None and ctx.needs_input_grad[1] else None
    return gx.to(x.dtype), gw, None


def _ln_setup(ctx, inputs, output):
    x, w, b, eps = inputs
    ctx.save_for_backward(*(t for t in (x, w) if t is not None))
    ctx.has_w, ctx.has_b, ctx.eps = w is not None, b is not None, eps
    ctx.b_meta = (b.shape, b.dtype) if b is not None else None


def _ln_backward(ctx, gy):
    saved = ctx.saved_tensors
    x = saved[0]
    w = saved[1] if ctx.has_w else None
    want_gb = ctx.has_b and ctx.needs_input_grad[2]
    if not want_gb or _bias_is_one_row(ctx.b_meta, x):
        fused = _ln_kernel_backward(x, None, w, gy, None, ctx.eps, ctx.needs_input_grad[1], ctx.b_meta, want_gb)
        if fused is not None:
            return fused[0], fused[1], fused[2], None
    xf, gf = x.float(), gy.float()
    mean = xf.mean(-1, keepdim=True)
    xc = xf - mean
    r = torch.rsqrt(xc.pow(2).mean(-1, keepdim=True) + ctx.eps)
    xhat = xc * r
    gxhat = gf * w.float() if w is not None else gf
    gx = r * (gxhat - gxhat.mean(-1, keepdim=True) - xhat * (gxhat * xhat).mean(-1, keepdim=True))
    gw = _reduce_to(gf * xhat, w.shape).to(w.dtype) if w is not None and ctx.needs_input_grad[1] else None
    gb = _reduce_to(gf, ctx.b_meta[0]).to(ctx.b_meta[1]) if ctx.has_b and ctx.needs_input_grad[2] else None
    return gx.to(x.dtype), gw, gb, None


def _silu_grad(a):
    s = torch.sigmoid(a)
    return s * (1 + a * (1 - s))


def _silu_mul2_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _silu_mul2_backward(ctx, gy):
    g, u = ctx.saved_tensors
    return torch.ops.xpu_ops.silu_mul2_bwd(g, u, gy.to(g.dtype))


def _act_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0])
    ctx.act = inputs[1]


def _act_backward(ctx, gy):
    (z,) = ctx.saved_tensors
    return torch.ops.xpu_ops.act_bwd(z, gy.to(z.dtype), ctx.act), None


def _silu_mul_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0])


def _silu_mul_backward(ctx, gy):
    (x,) = ctx.saved_tensors
    d = x.shape[-1] // 2
    a, b = x[..., :d].float(), x[..., d:].float()
    yf = gy.float()
    return (torch.cat([yf * b * _silu_grad(a), yf * torch.nn.functional.silu(a)], dim=-1).to(x.dtype),)


def _weight_grad(a_t, b):
    """a_t^T @ b for 2-D operands [tokens, M], [tokens, N]: on the dense kernel when it takes the shape."""
    from . import ops

    if ops.dense_at_fits(tuple(a_t.shape), tuple(b.shape), a_t.dtype) and a_t.dtype == b.dtype:
        return torch.ops.xpu_ops.dense_at(a_t, b, None)
    return a_t.t() @ b


def _dense_setup(ctx, inputs, output):
    x, weight, weight_trans, bias, residual, act = inputs
    ctx.save_for_backward(x, weight, output, *(t for t in (bias, residual) if t is not None))
    ctx.trans, ctx.act = weight_trans, act
    ctx.has_bias, ctx.has_res = bias is not None, residual is not None


def _dense_backward(ctx, gy):
    saved = ctx.saved_tensors
    x, weight, y = saved[:3]
    rest = list(saved[3:])
    bias = rest.pop(0) if ctx.has_bias else None
    residual = rest.pop(0) if ctx.has_res else None
    act = ctx.act
    if act == "none":
        gz = gy  # the upstream gradient is the pre-activation's, as it is
    elif act == "relu":
        gz = gy.float() * (y > 0)
    elif act == "sigmoid":
        yf = y.float()
        gz = gy.float() * yf * (1 - yf)
    elif act in ("silu", "gelu"):
        # the pre-activation is not kept by the fused call: one more product, then one pass over it and gy
        z = torch.ops.xpu_ops.dense(x, weight, ctx.trans, bias, residual, "none")
        gz = torch.ops.xpu_ops.act_bwd(z, gy.to(z.dtype), act)
    else:
        raise NotImplementedError(f"dense backward: activation {act!r}")
    gz = gz.to(x.dtype)
    need = ctx.needs_input_grad
    gx = None
    if need[0]:
        # gz [M, N] times the weight read the other way: the product's inner size is N, its output width K.  The
        # kernel wants both as the forward wants K and N; an fp32 layer with K % 8 == 4 passes the forward's check
        # (4-element loads) and not this one, and then takes the Aten product.
        from . import ops

        if ops.dense_fits(gz.shape[1], x.shape[1], gz.dtype):
            gx = torch.ops.xpu_ops.dense(gz, weight, not ctx.trans, None, None, "none")
        else:
            gx = gz @ (weight if ctx.trans else weight.t())
    gw = None
    if need[1]:
        gw = _weight_grad(gz, x) if ctx.trans else _weight_grad(x, gz)
    gb = gz.float().sum(0).to(bias.dtype) if ctx.has_bias and need[3] else None
    gr = gz if ctx.has_res and need[4] else None
    return gx, gw, None, gb, gr, None


def _dense_glu_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _glu_grads(ctx, x, w_gate, w_up, gate, up, gy):
    dense = torch.ops.xpu_ops.dense
    d_gate, d_up = torch.ops.xpu_ops.silu_mul2_bwd(gate, up, gy.to(x.dtype))  # one pass instead of a dozen Aten kernels
    need = ctx.needs_input_grad
    gx = None
    if need[0]:
        gx = dense(d_up, w_up, False, None, dense(d_gate, w_gate, False, None, None, "none"), "none")
    gwg = _weight_grad(d_gate, x) if need[1] else None
    gwu = _weight_grad(d_up, x) if need[2] else None
    return gx, gwg, gwu


def _dense_glu_backward(ctx, gy):
    # the plain op saved only its inputs: both projections are run again
    x, w_gate, w_up = ctx.saved_tensors
    dense = torch.ops.xpu_ops.dense
    gate = dense(x, w_gate, True, None, None, "none")
    up = dense(x, w_up, True, None, None, "none")
    return _glu_grads(ctx, x, w_gate, w_up, gate, up, gy)


def _dense_glu_save_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs, output[1], output[2])
    ctx.set_materialize_grads(False)  # an unused output then hands over None, not zeros: a used one can be told apart


def _dense_glu_save_backward(ctx, gy, g_gate=None, g_up=None):
    # the two projection outputs exist for this formula; a gradient flowing into them is refused, not dropped
    if g_gate is not None or g_up is not None:
        raise NotImplementedError("xpu_ops::dense_glu_save: only its first output (the gated product) is differentiable")
    if gy is None:
        return None, None, None
    x, w_gate, w_up, gate, up = ctx.saved_tensors
    return _glu_grads(ctx, x, w_gate, w_up, gate, up, gy)


def _rotate_half(t):
    d = t.shape[-1] // 2
    return torch.cat([-t[..., d:], t[..., :d]], dim=-1)


def _rope_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _rope_backward(ctx, gy):
    # rotate_half is a signed permutation R with R^T = -R, so gx = gy * cos - R(gy * sin) = gy * cos + R(gy) * sin'
    # with sin' = -swap_halves(sin): the rotary kernel itself, on a rewritten [S, D] sine table.
    x, cos, sin = ctx.saved_tensors
    need = ctx.needs_input_grad
    gx = None
    if need[0]:
        d = sin.shape[-1] // 2
        sin_t = -torch.cat([sin[..., d:], sin[..., :d]], dim=-1)
        gx = torch.ops.xpu_ops.rope(gy, cos, sin_t)
    gcos = gsin = None
    if need[1] or need[2]:
        gf, xf = gy.float(), x.float()
        if need[1]:  # summed over everything the table was broadcast along (batch and heads; positions too for one row)
            gcos = (gf * xf).sum_to_size(*([1] * (4 - cos.dim()) + list(cos.shape))).reshape(cos.shape).to(cos.dtype)
        if need[2]:
            gsin = (gf * _rotate_half(xf)).sum_to_size(*([1] * (4 - sin.dim()) + list(sin.shape))).reshape(sin.shape).to(sin.dtype)
    return gx, gcos, gsin


def _sdpa_setup(ctx, inputs, output):
    q, k, v, ctx.causal, ctx.scale = inputs
    ctx.save_for_backward(q, k, v)


def _sdpa_backward(ctx, gy):
    # The plain op saves no row statistics: one more forward launch recomputes the output and its log-sum-exp (bit
    # for bit the forward's), then the backward kernels run.  Graphs built for training use sdpa_lse instead.
    q, k, v = ctx.saved_tensors
    out, lse = torch.ops.xpu_ops.sdpa_lse(q, k, v, ctx.causal, ctx.scale)
    gq, gk, gv = torch.ops.xpu_ops.sdpa_bwd(q, k, v, out, gy, lse, ctx.causal, ctx.scale)
    return gq, gk, gv, None, None


def _sdpa_lse_setup(ctx, inputs, output):
    q, k, v, ctx.causal, ctx.scale = inputs
    out, lse = output
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.set_materialize_grads(False)  # an unused log-sum-exp then hands over None, not zeros


def _sdpa_lse_backward(ctx, gy, g_lse=None):
    # the log-sum-exp output exists for this formula; a gradient flowing into it is refused, not dropped
    if g_lse is not None:
        raise NotImplementedError("xpu_ops::sdpa_lse: only its first output (the attention result) is differentiable")
    if gy is None:
        return None, None, None, None, None
    q, k, v, out, lse = ctx.saved_tensors
    gq, gk, gv = torch.ops.xpu_ops.sdpa_bwd(q, k, v, out, gy, lse, ctx.causal, ctx.scale)
    return gq, gk, gv, None, None


def _refuse_mask_or_scale_grad(ctx, name):
    if ctx.needs_input_grad[3] or ctx.needs_input_grad[4]:
        raise NotImplementedError(f"xpu_ops::{name}: no gradient for the mask or the scale tensor (only q, k, v are differentiable)")


def _sdpa_masked_setup(ctx, inputs, output):
    q, k, v, mask, scale_t, ctx.causal, ctx.scale = inputs
    ctx.has_mask, ctx.has_scale = mask is not None, scale_t is not None
    ctx.save_for_backward(q, k, v, *(t for t in (mask, scale_t) if t is not None))


def _masked_operands(ctx, rest):
    rest = list(rest)
    mask = rest.pop(0) if ctx.has_mask else None
    scale_t = rest.pop(0) if ctx.has_scale else None
    return mask, scale_t


def _sdpa_masked_backward(ctx, gy):
    # as for the plain op: one more forward launch for the row statistics, then the backward kernels
    _refuse_mask_or_scale_grad(ctx, "sdpa_masked")
    q, k, v, *rest = ctx.saved_tensors
    mask, scale_t = _masked_operands(ctx, rest)
    out, lse = torch.ops.xpu_ops.sdpa_masked_lse(q, k, v, mask, scale_t, ctx.causal, ctx.scale)
    gq, gk, gv = torch.ops.xpu_ops.sdpa_masked_bwd(q, k, v, out, gy, lse, mask, scale_t, ctx.causal, ctx.scale)
    return gq, gk, gv, None, None, None, None


def _sdpa_masked_lse_setup(ctx, inputs, output):
    q, k, v, mask, scale_t, ctx.causal, ctx.scale = inputs
    out, lse = output
    ctx.has_mask, ctx.has_scale = mask is not None, scale_t is not None
    ctx.save_for_backward(q, k, v, out, lse, *(t for t in (mask, scale_t) if t is not None))
    ctx.set_materialize_grads(False)


def _sdpa_masked_lse_backward(ctx, gy, g_lse=None):
    if g_lse is not None:
        raise NotImplementedError("xpu_ops::sdpa_masked_lse: only its first output (the attention result) is differentiable")
    if gy is None:
        return (None,) * 7
    _refuse_mask_or_scale_grad(ctx, "sdpa_masked_lse")
    q, k, v, out, lse, *rest = ctx.saved_tensors
    mask, scale_t = _masked_operands(ctx, rest)
    gq, gk, gv = torch.ops.xpu_ops.sdpa_masked_bwd(q, k, v, out, gy, lse, mask, scale_t, ctx.causal, ctx.scale)
    return gq, gk, gv, None, None, None, None


def _add_norm_formulas(layer, with_sum):
    """(setup, backward) of the residual-add + norm ops: the sum is recomputed, its gradient is the norm's input
    gradient plus whatever flows into the returned sum, and both addends receive it."""

    def setup(ctx, inputs, output):
        x, res, w = inputs[:3]
        b = inputs[3] if layer else None
        ctx.eps = inputs[-1]
        ctx.save_for_backward(*(t for t in (x, res, w) if t is not None))
        ctx.has_w = w is not None
        ctx.b_meta = (b.shape, b.dtype) if b is not None else None

    def backward(ctx, gy, gh=None):
        saved = ctx.saved_tensors
        x, res = saved[0], saved[1]
        w = saved[2] if ctx.has_w else None
        need = ctx.needs_input_grad
        if not layer:
            fused = _rms_kernel_backward(x, res, w, gy, gh, ctx.eps, need[2])
            if fused is not None:
                return fused[0], fused[0], fused[1], None
        else:
            want_gb = ctx.b_meta is not None and need[3]
            if not want_gb or _bias_is_one_row(ctx.b_meta, x):
                fused = _ln_kernel_backward(x, res, w, gy, gh, ctx.eps, need[2], ctx.b_meta, want_gb)
                if fused is not None:
                    return fused[0], fused[0], fused[1], fused[2], None
        hf, gf = x.float() + res.float(), gy.float()
        hc = hf - hf.mean(-1, keepdim=True) if layer else hf
        r = torch.rsqrt(hc.pow(2).mean(-1, keepdim=True) + ctx.eps)
        hhat = hc * r
        ghat = gf * w.float() if w is not None else gf
        g_sum = ghat - hhat * (ghat * hhat).mean(-1, keepdim=True)
        if layer:
            g_sum = g_sum - ghat.mean(-1, keepdim=True)
        g_sum = r * g_sum
        if gh is not None:
            g_sum = g_sum + gh.float()
        g_sum = g_sum.to(x.dtype)
        gw = _reduce_to(gf * hhat, w.shape).to(w.dtype) if w is not None and need[2] else None
        if layer:
            gb = _reduce_to(gf, ctx.b_meta[0]).to(ctx.b_meta[1]) if ctx.b_meta is not None and need[3] else None
            return g_sum, g_sum, gw, gb, None
        return g_sum, g_sum, gw, None

    return setup, backward


def register():
    global _REGISTERED
    if _REGISTERED:
        return
    reg = torch.library.register_autograd
    reg("xpu_ops::rms_norm", _rms_backward, setup_context=_rms_setup)
    reg("xpu_ops::layer_norm", _ln_backward, setup_context=_ln_setup)
    reg("xpu_ops::silu_mul2", _silu_mul2_backward, setup_context=_silu_mul2_setup)
    reg("xpu_ops::act", _act_backward, setup_context=_act_setup)
    reg("xpu_ops::silu_mul", _silu_mul_backward, setup_context=_silu_mul_setup)
    reg("xpu_ops::dense", _dense_backward, setup_context=_dense_setup)
    reg("xpu_ops::dense_glu", _dense_glu_backward, setup_context=_dense_glu_setup)
    reg("xpu_ops::dense_glu_save", _dense_glu_save_backward, setup_context=_dense_glu_save_setup)
    reg("xpu_ops::rope", _rope_backward, setup_context=_rope_setup)
    reg("xpu_ops::sdpa", _sdpa_backward, setup_context=_sdpa_setup)
    reg("xpu_ops::sdpa_lse", _sdpa_lse_backward, setup_context=_sdpa_lse_setup)
    reg("xpu_ops::sdpa_masked", _sdpa_masked_backward, setup_context=_sdpa_masked_setup)
    reg("xpu_ops::sdpa_masked_lse", _sdpa_masked_lse_backward, setup_context=_sdpa_masked_lse_setup)
    for op, layer, with_sum in (("add_rms_norm", False, True), ("add_rms_norm_only", False, False),
                                ("add_layer_norm", True, True), ("add_layer_norm_only", True, False)):
        setup, backward = _add_norm_formulas(layer, with_sum)
        reg(f"xpu_ops::{op}", backward, setup_context=setup)
    # An op that was traced before (an inference compile earlier in the process) has its dispatch decisions cached
    # on the Python side; a stale entry for the Autograd key would keep sending traces to the "no formula" fallback.
    for name in ("rms_norm", "layer_norm", "silu_mul2", "silu_mul", "act", "dense", "dense_glu", "dense_glu_save", "rope", "sdpa", "sdpa_lse",
                 "sdpa_masked", "sdpa_masked_lse", "add_rms_norm", "add_rms_norm_only", "add_layer_norm", "add_layer_norm_only"):
        packet = getattr(torch.ops.xpu_ops, name)
        for overload in packet.overloads():
            getattr(packet, overload)._dispatch_cache.clear()
    _REGISTERED = True
