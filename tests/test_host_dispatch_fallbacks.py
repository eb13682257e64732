"""What the backend does with graphs a flat Aten rewrite cannot take apart, and the guard filter option
(reference tests/common/test_custom_op.py:13-188, test_guard_filter.py:13-35): custom ops pass through; in training,
autograd.Function applications and activation checkpoints are higher-order operators, which are reported and sent to
AOT as they are; inference decomposes all of them."""
import pytest
import torch
import torch.nn as nn
from torch.utils.checkpoint import checkpoint

import xpu_graph_amd
from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs


@torch.library.custom_op("xg_test_ops::scale_by", mutates_args=())
def scale_by(x: torch.Tensor, factor: float) -> torch.Tensor:
    return torch.from_numpy(x.numpy(force=True) * factor).to(x.device)  # opaque to tracing


@scale_by.register_fake
def _(x, factor):
    return torch.empty_like(x)


def _scale_setup(ctx, inputs, output):
    ctx.factor = inputs[1]


scale_by.register_autograd(lambda ctx, g: (g * ctx.factor, None), setup_context=_scale_setup)


class ScaleFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, factor):
        ctx.save_for_backward(torch.tensor(factor))
        return torch.from_numpy(x.numpy(force=True) * factor).to(x.device)

    @staticmethod
    def backward(ctx, g):
        (factor,) = ctx.saved_tensors
        return g * factor, None


class WithCustomOp(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.fc = nn.Linear(d, d)

    def forward(self, x):
        return scale_by(self.fc(x), 0.1).sum(dim=-1)


class WithAutogradFunction(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.fc = nn.Linear(d, d)

    def forward(self, x):
        return ScaleFn.apply(ScaleFn.apply(self.fc(x), 0.1), 0.1).sum(dim=-1)


class CheckpointedSwiGLU(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.d = d
        self.proj = nn.Linear(d, 2 * d)

    def _gate(self, x):
        a, b = self.proj(x).split(self.d, dim=-1)
        return nn.functional.silu(a) * b

    def forward(self, x):
        y = checkpoint(self._gate, x, use_reentrant=False) if self.training else self._gate(x)
        return y.sum(dim=-1)


MODULES = [WithCustomOp, WithAutogradFunction, CheckpointedSwiGLU]


@pytest.mark.parametrize("cls", MODULES)
def test_training_with_opaque_pieces(caplog, cls):
    backend = XpuGraph(XpuGraphConfig(is_training=True, opt_level=OptLevel.level2, freeze=False, enable_cache=False))
    golden, compiled = cls(16), cls(16)
    compiled.load_state_dict(golden.state_dict())
    compiled.forward = torch.compile(compiled.forward, backend=backend, dynamic=False)
    x, target = torch.randn(8, 16), torch.randn(8)
    opt_g, opt_c = torch.optim.AdamW(golden.parameters()), torch.optim.AdamW(compiled.parameters())
    opt_c.load_state_dict(opt_g.state_dict())
    loss_fn = nn.MSELoss()
    with need_xpu_graph_logs():
        for _ in range(4):
            opt_g.zero_grad()
            loss_g = loss_fn(golden(x), target)
            loss_g.backward()
            opt_g.step()
            opt_c.zero_grad()
            loss_c = loss_fn(compiled(x), target)
            loss_c.backward()
            opt_c.step()
            assert is_similar(loss_g, loss_c)
            for name, p in golden.named_parameters():
                assert is_similar(p, compiled.get_parameter(name))
    if cls is WithCustomOp:
        assert "Higher order operators detected" not in caplog.text
    else:
        assert "Higher order operators detected" in caplog.text
    torch._dynamo.reset()


@pytest.mark.parametrize("cls", MODULES)
def test_inference_with_opaque_pieces(caplog, cls):
    backend = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, freeze=False, enable_cache=False))
    golden, compiled = cls(16).eval(), cls(16).eval()
    compiled.load_state_dict(golden.state_dict())
    compiled.forward = torch.compile(compiled.forward, backend=backend, dynamic=False)
    with need_xpu_graph_logs(), torch.no_grad():
        for _ in range(4):
            x = torch.randn(8, 16)
            assert is_similar(golden(x), compiled(x))
    assert "Higher order operators detected" not in caplog.text
    assert "decompose graph complete" in caplog.text
    torch._dynamo.reset()


def test_guard_filter_drops_the_shape_guards(caplog):
    """With every guard filtered out a static-shape compile serves other batch sizes too: one pass-pipeline run."""
    backend = XpuGraph(XpuGraphConfig(is_training=False, enable_cache=False))

    def foo(x):
        return x + 1

    compiled = torch.compile(foo, backend=backend, dynamic=False, options={"guard_filter_fn": xpu_graph_amd.skip_all_guards_unsafe})
    with need_xpu_graph_logs():
        for bsz in (8, 10, 12):
            x = torch.randn(bsz, 32)
            assert is_similar(compiled(x), foo(x))
    assert caplog.text.count("xpu_graph passes start ") == 1  # (this torch applies the filter itself before the backend runs)
    torch._dynamo.reset()
