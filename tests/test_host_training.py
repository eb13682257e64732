"""Training path: the Dynamo graph is lowered to pre-dispatch Aten IR and rewritten in the `pregrad` stage before
AOT differentiates it (reference tests/common/test_fuse_rmsnorm.py:66-157, test_fuse_layernorm.py training cases):
the pattern fires, values and gradients agree with eager."""
import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig
from xpu_graph_amd.fx_utils import dispatch_pregrad
from xpu_graph_amd.test_utils import need_xpu_graph_logs


def naive_rmsnorm(inputs, weight):
    square = torch.square(inputs)
    mean = torch.mean(square, dim=-1, keepdim=True)
    root = torch.sqrt(mean + 1e-6)
    return inputs / root * weight


def naive_rmsnorm_variant(inputs, weight):
    iroot = torch.rsqrt(torch.mean(inputs**2, dim=-1, keepdim=True) + 1e-6)
    return weight * (inputs * iroot)


def naive_rmsnorm_noweight(inputs, weight):
    return inputs / (torch.mean(inputs * inputs, dim=-1, keepdim=True) + 1e-3) ** 0.5


def naive_rmsnorm_liftdtype(inputs, weight):
    return naive_rmsnorm(inputs.to(torch.float32), weight).to(inputs.dtype)


def naive_layernorm(x, w, b):
    mean = x.mean(-1, keepdim=True)
    var = x.var(-1, keepdim=True, unbiased=False)
    return (x - mean) * torch.rsqrt(var + 1e-5) * w + b


def train_backend(**kw):
    return XpuGraph(XpuGraphConfig(is_training=True, opt_level=OptLevel.level2, enable_cache=False, **kw))


@pytest.mark.parametrize(
    "fn,in_dtype,w_dtype",
    [
        (naive_rmsnorm, torch.float32, torch.float32),
        (naive_rmsnorm_variant, torch.float32, torch.float32),
        (naive_rmsnorm_noweight, torch.float32, torch.float32),
        (naive_rmsnorm_liftdtype, torch.bfloat16, torch.float32),
    ],
)
def test_rmsnorm_with_loss_and_grad(caplog, fn, in_dtype, w_dtype):
    x = torch.randn(8, 1024, dtype=in_dtype, requires_grad=True)
    w = torch.randn(1024, dtype=w_dtype, requires_grad=True)
    dy = torch.randn(8, 1024, dtype=in_dtype)
    backend = train_backend()  # before the log context: constructing a backend resets the logger's level
    with need_xpu_graph_logs():
        y0 = torch.compile(fn, backend=backend)(x, w)
    gx0, gw0 = torch.autograd.grad((y0,), (x, w), (dy,), allow_unused=True)
    y1 = fn(x, w)
    gx1, gw1 = torch.autograd.grad((y1,), (x, w), (dy,), allow_unused=True)
    tol = dict(rtol=1e-4, atol=1e-4) if in_dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(y0, y1, **tol)
    torch.testing.assert_close(gx0, gx1, **tol)
    if gw1 is None:
        assert gw0 is None
    else:
        torch.testing.assert_close(gw0, gw1, rtol=1e-3, atol=1e-3 if in_dtype == torch.float32 else 0.5)
    assert "xpu_graph passes start FxStage.pregrad" in caplog.text
    assert "Pattern.FusedRMSNorm changed graph" in caplog.text


def test_layernorm_with_loss_and_grad(caplog):
    x = torch.randn(6, 256, requires_grad=True)
    w, b = torch.randn(256, requires_grad=True), torch.randn(256, requires_grad=True)
    dy = torch.randn(6, 256)
    backend = train_backend()
    with need_xpu_graph_logs():
        y0 = torch.compile(naive_layernorm, backend=backend)(x, w, b)
    g0 = torch.autograd.grad((y0,), (x, w, b), (dy,))
    g1 = torch.autograd.grad((naive_layernorm(x, w, b),), (x, w, b), (dy,))
    for a, c in zip(g0, g1):
        torch.testing.assert_close(a, c, rtol=1e-4, atol=1e-4)
    assert "Pattern.FusedLayerNorm changed graph" in caplog.text


def test_pregrad_is_skipped_for_input_mutation(caplog):
    def fn(x, buf):
        buf.add_(1.0)
        return (x * buf).sum(-1)

    x = torch.randn(4, 8, requires_grad=True)
    buf_c, buf_e = torch.zeros(4, 8), torch.zeros(4, 8)
    backend = train_backend()
    with need_xpu_graph_logs():
        y0 = torch.compile(fn, backend=backend)(x, buf_c)
    y1 = fn(x, buf_e)
    torch.testing.assert_close(y0, y1)
    torch.testing.assert_close(buf_c, buf_e)
    (g0,) = torch.autograd.grad(y0.sum(), x)
    torch.testing.assert_close(g0, torch.ones(4, 8))
    assert "pregrad stage skipped" in caplog.text and "xpu_graph passes start FxStage.forward" in caplog.text


def test_dispatch_pregrad_keeps_composites_and_signature():
    def fn(x, w, b):
        return (F.layer_norm(F.linear(x, w), (16,), None, b),)  # Dynamo graphs return tuples

    gm = torch.fx.symbolic_trace(fn)
    out = dispatch_pregrad(gm, [torch.randn(4, 8), torch.randn(16, 8), torch.randn(16)])
    targets = [str(n.target) for n in out.graph.nodes if n.op == "call_function"]
    assert targets == ["aten.linear.default", "aten.layer_norm.default"]
    assert len([n for n in out.graph.nodes if n.op == "placeholder"]) == 3

    class Holder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w = torch.nn.Parameter(torch.randn(3))

        def forward(self, x):
            return (x * self.w,)

    with pytest.raises(NotImplementedError, match="parameters"):
        dispatch_pregrad(torch.fx.symbolic_trace(Holder()), [torch.randn(3)])


def test_mi355x_training_graphs_use_the_custom_ops(caplog):
    """On the mi355x target the pregrad stage puts the HIP-backed norm and gate ops in; AOT differentiates through
    their registered backward formulas (the forward graph below calls xpu_ops, which refuse CPU tensors)."""

    def block(x, w, g, b, up):
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
        h = F.layer_norm(h, (64,), g, b, 1e-5)
        return F.silu(h) * up

    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(8, 64, requires_grad=True), torch.randn(64, requires_grad=True), torch.randn(64, requires_grad=True),
            torch.randn(64, requires_grad=True), torch.randn(8, 64, requires_grad=True)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(block, backend=backend)(*args)
    pregrad, forward = backend.compiled_graphs[-2:]
    assert [n.target for n in pregrad.graph.nodes if n.op == "call_module"] == ["custom_rms_norm", "custom_layer_norm", "mi355x_silu_mul2"]
    fwd_ops = [str(n.target) for n in forward.graph.nodes if n.op == "call_function"]
    assert fwd_ops[:3] == ["xpu_ops.rms_norm.default", "xpu_ops.layer_norm.default", "xpu_ops.silu_mul2.default"]
    for p in ("FusedRMSNorm", "CustomRMSNorm", "NativeNormToDefault", "CustomLayerNorm", "FusedSwiGLU"):
        assert f"Pattern.{p} changed graph" in caplog.text, p


def test_linear_is_decomposed_for_the_dense_pattern_in_pregrad(caplog):
    """Pre-dispatch graphs keep aten.linear whole; DecomposeLinear turns it into (add)mm so that the dense
    pattern fires before autograd is traced (the dense op has a backward formula)."""

    def mlp(x, w1, b1, w2):
        return F.linear(F.relu(F.linear(x, w1, b1)), w2)

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 8, 64).to(bf).requires_grad_(True), torch.randn(128, 64).to(bf).requires_grad_(True),
            torch.randn(128).to(bf).requires_grad_(True), torch.randn(64, 128).to(bf).requires_grad_(True)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(mlp, backend=backend)(*args)
    pregrad = backend.compiled_graphs[-2]
    calls = [n for n in pregrad.graph.nodes if n.op == "call_module"]
    assert [n.target for n in calls] == ["custom_dense_layer_replacement"] * 2
    assert calls[0].args[2] is True and calls[0].args[3] is not None  # [N, K] weight, bias kept
    assert not any("linear" in str(n.target) or "aten.mm" in str(n.target) for n in pregrad.graph.nodes)
    assert "Pattern.DecomposeLinear changed graph" in caplog.text and "Pattern.CustomDenseLayer changed graph" in caplog.text


def test_gated_mlp_becomes_one_gated_dense_call_in_pregrad(caplog):
    """silu(linear(x, Wg)) * linear(x, Wu) -> linear: the gate and up projections leave the pregrad stage as ONE
    gated dense module (it has a backward formula), the down projection as a dense module."""

    def mlp(x, wg, wu, wd):
        return F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 8, 64).to(bf).requires_grad_(True), torch.randn(128, 64).to(bf).requires_grad_(True),
            torch.randn(128, 64).to(bf).requires_grad_(True), torch.randn(64, 128).to(bf).requires_grad_(True)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(mlp, backend=backend)(*args)
    pregrad = backend.compiled_graphs[-2]
    assert [n.target for n in pregrad.graph.nodes if n.op == "call_module"] == ["mi355x_dense_glu", "custom_dense_layer_replacement"]
    assert "Pattern.FusedDenseGLU changed graph" in caplog.text


def test_rotary_embedding_is_one_module_in_pregrad(caplog):
    """x * cos + rotate_half(x) * sin on a [B, H, S, D] tensor leaves the pregrad stage as the rotary module."""

    def rot(x, cos, sin):
        d = x.shape[-1] // 2
        return (x * cos + torch.cat([-x[..., d:], x[..., :d]], dim=-1) * sin) * 2.0

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 4, 16, 64).to(bf).requires_grad_(True), torch.randn(16, 64).to(bf), torch.randn(16, 64).to(bf)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(rot, backend=backend)(*args)
    pregrad = backend.compiled_graphs[-2]
    assert [n.target for n in pregrad.graph.nodes if n.op == "call_module"] == ["mi355x_rope"]
    assert "Pattern.FusedRoPE changed graph" in caplog.text


def test_causal_attention_is_one_module_in_pregrad(caplog):
    """F.scaled_dot_product_attention(is_causal=True) on 16-bit [B, H, S, D] operands leaves the pregrad stage as
    the attention module of the target (the op has a backward formula)."""

    def attn(q, k, v):
        return F.scaled_dot_product_attention(q, k, v, is_causal=True) * 2.0

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 4, 32, 64).to(bf).requires_grad_(True) for _ in range(3)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(attn, backend=backend)(*args)
    pregrad = backend.compiled_graphs[-2]
    calls = [n for n in pregrad.graph.nodes if n.op == "call_module"]
    assert [n.target for n in calls] == ["mi355x_sdpa"] and calls[0].args[3] is True
    assert "Pattern.FusedCausalSDPA changed graph" in caplog.text


def test_backward_formulas_reach_ops_that_were_traced_before_registration():
    """An inference compile that traces xpu_ops::dense BEFORE any training backend exists must not hide the
    backward formula registered later: the joint graph then saves the dense operands for the backward pass (in a
    fresh process: registration happens once per process)."""
    import subprocess
    import sys

    code = r'''
import warnings, torch, torch.nn.functional as F
from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig
def mlp(x, w1, b1, w2):
    return F.linear(F.silu(F.linear(x, w1, b1)), w2)
bf = torch.bfloat16
args = [torch.randn(16, 64).to(bf), torch.randn(128, 64).to(bf), torch.randn(128).to(bf), torch.randn(64, 128).to(bf)]
first = XpuGraph(XpuGraphConfig(False, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
try:
    with torch.no_grad():
        torch.compile(mlp, backend=first, dynamic=False)(*args)
except NotImplementedError:
    pass  # the kernels refuse CPU tensors; the trace is what matters
assert any("dense" in str(n.target) for n in first.compiled_graphs[-1].graph.nodes)
torch._dynamo.reset()
train = XpuGraph(XpuGraphConfig(True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
with warnings.catch_warnings(record=True) as seen:
    warnings.simplefilter("always")
    try:
        torch.compile(mlp, backend=train, dynamic=False)(*[a.clone().requires_grad_(True) for a in args])
    except NotImplementedError:
        pass
assert not [w for w in seen if "autograd kernel was not registered" in str(w.message)], [str(w.message)[:80] for w in seen]
forward = train.compiled_graphs[-1]
outs = list(forward.graph.nodes)[-1].args[0]
print("FORWARD_OUTPUTS", len(outs))
'''
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    n_out = int(proc.stdout.split("FORWARD_OUTPUTS")[1].split()[0])
    assert n_out >= 5, n_out  # y + the operands both dense backward formulas keep (x, weights, outputs, bias)


def test_written_out_attention_reaches_the_attention_kernel_in_pregrad(caplog):
    """matmul -> / sqrt(D) -> + causal mask -> softmax in fp32 -> cast -> matmul on [B, H, S, D] operands, as a
    hand-written decoder block spells it, becomes aten.scaled_dot_product_attention before autograd is traced
    (beyond the reference, whose FusedSDPA is inference-only); the target pattern recognises the constant causal
    mask, and the differentiated forward graph runs the attention that saves the row statistics."""
    import math

    def attn(q, k, v):
        S, D = q.shape[-2], q.shape[-1]
        s = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(D)
        s = s + torch.full((S, S), float("-inf"), dtype=q.dtype).triu(1)
        p = torch.softmax(s, dim=-1, dtype=torch.float32).to(q.dtype)
        return torch.matmul(p, v)

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 4, 32, 64).to(bf).requires_grad_(True) for _ in range(3)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(attn, backend=backend)(*args)
    pregrad, forward = backend.compiled_graphs[-2:]
    calls = [n for n in pregrad.graph.nodes if n.op == "call_module"]
    assert [n.target for n in calls] == ["mi355x_sdpa"]
    assert calls[0].args[3] is True and abs(calls[0].args[4] - 0.125) < 1e-9  # causal by index, scale 1 / sqrt(64)
    assert not any("softmax" in str(n.target) or "matmul" in str(n.target) for n in pregrad.graph.nodes)
    fwd_ops = [str(n.target) for n in forward.graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.sdpa_lse.default") == 1 and "xpu_ops.sdpa.default" not in fwd_ops, fwd_ops
    assert "Pattern.FusedSDPA changed graph" in caplog.text


def test_masked_attention_in_pregrad_depends_on_who_needs_a_gradient(caplog):
    """The attn_mask form in a training graph: a mask computed from inputs that need no gradient (padding) goes to the
    masked attention module, whose op has backward kernels for q, k, v; a mask computed from a parameter (a learned
    bias) would lose its gradient there, so that attention stays as the Aten op."""

    def attn(q, k, v, pad, bias):
        a = F.scaled_dot_product_attention(q, k, v, attn_mask=pad * 2.0)
        b = F.scaled_dot_product_attention(q, k, v, attn_mask=bias + pad)
        return a + b

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(2, 4, 32, 64).to(bf).requires_grad_(True) for _ in range(3)]
    args += [torch.zeros(2, 1, 32, 32).to(bf), torch.zeros(1, 4, 32, 32).to(bf).requires_grad_(True)]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(attn, backend=backend)(*args)
    pregrad, forward = backend.compiled_graphs[-2:]
    assert [n.target for n in pregrad.graph.nodes if n.op == "call_module"] == ["mi355x_sdpa_masked"]
    assert sum(1 for n in pregrad.graph.nodes if "scaled_dot_product_attention" in str(n.target)) == 1
    fwd_ops = [str(n.target) for n in forward.graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.sdpa_masked_lse.default") == 1 and "xpu_ops.sdpa_masked.default" not in fwd_ops, fwd_ops
