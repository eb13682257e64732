"""Ready-made plugin patterns for the mi355x target.

The fp8 dense layer has no counterpart in the reference and no canonical eager
spelling, so it is offered the way the reference offers user-defined fusions:
as a plugin pattern (reference src/xpu_graph/passes/patterns/plugin_pattern.py:114-284;
real use: targets/mlu/linear_to_matmul.py:7-35).  The user registers THEIR
eager function -- operands already quantised to e4m3, activations per tensor,
weights per output channel -- and every occurrence of that exact subgraph is
replaced by one `torch.ops.xpu_ops.dense_fp8` call.

    from xpu_graph_amd import plugins
    plugins.register_fp8_dense(my_fp8_linear, example_inputs, act="silu")      # before building the backend
    backend = mi355x_compiler()
"""
import torch
import torch.nn.functional as F

from .config import Target
from .passes.patterns.plugin_pattern import register_plugin_pattern

_ACTS = ("none", "relu", "gelu", "silu", "sigmoid")


def fp8_linear_silu_eager(x_q, w_q, x_scale, w_scale, bias):
    """One eager spelling of the fp8 dense layer: x_q [M, K] and w_q [N, K] in float8_e4m3fn, x_scale [1],
    w_scale [N] and bias [N]; dequantise, fp32 matmul, scales and bias in fp32, SiLU, bf16 result."""
    acc = torch.mm(x_q.float(), w_q.float().t())
    return F.silu(acc * x_scale * w_scale + bias.float()).to(torch.bfloat16)


def fp8_linear_eager(x_q, w_q, x_scale, w_scale, bias):
    acc = torch.mm(x_q.float(), w_q.float().t())
    return (acc * x_scale * w_scale + bias.float()).to(torch.bfloat16)


def _replacement(act, out_dtype):
    def fp8_dense(x_q, w_q, x_scale, w_scale, bias):
        return torch.ops.xpu_ops.dense_fp8(x_q, w_q, True, x_scale, w_scale, bias, act, out_dtype)

    return fp8_dense


def _operands_fit(x_q, w_q, x_scale, w_scale, bias):
    """Match-time veto (receives FakeTensors): shapes the kernel takes, otherwise the subgraph stays as it is."""
    ok = x_q.dim() == 2 and w_q.dim() == 2 and x_q.dtype == torch.float8_e4m3fn and w_q.dtype == torch.float8_e4m3fn
    ok = ok and all(isinstance(d, int) for d in (*x_q.shape, *w_q.shape))
    return bool(ok and x_q.shape[1] == w_q.shape[1] and x_q.shape[1] % 16 == 0 and w_q.shape[0] % 8 == 0 and x_scale.numel() == 1 and w_scale.numel() == w_q.shape[0])


def example_fp8_inputs(m=32, n=64, k=128, bias_dtype=torch.bfloat16):
    """Example inputs that trace the eager spelling (shapes are irrelevant to the match)."""
    return (
        torch.zeros(m, k).to(torch.float8_e4m3fn),
        torch.zeros(n, k).to(torch.float8_e4m3fn),
        torch.ones(1),
        torch.ones(n),
        torch.zeros(n, dtype=bias_dtype),
    )


def register_fp8_dense(eager_func, example_inputs=None, act="none", out_dtype=torch.bfloat16, target=Target.mi355x):
    """Register `eager_func(x_q, w_q[N, K], x_scale, w_scale, bias)` as a pattern that lowers to the fp8 MFMA kernel."""
    if act not in _ACTS:
        raise ValueError(f"unknown activation {act!r}")
    from . import ops as _register_ops  # noqa: F401  (defines torch.ops.xpu_ops before the replacement is traced)

    register_plugin_pattern(eager_func, example_inputs or example_fp8_inputs(), _replacement(act, out_dtype), target, extra_checks=[_operands_fit])
