"""Host tests of freezing (parameters unlifted into graph constants, reference fx_utils.py `_unlift_params`), of what
constant folding and CSE may NOT do to tensors the caller receives, and of the bounded attention backward."""
import logging

import pytest
import torch
import torch.nn as nn

from xpu_graph_amd import XpuGraph, XpuGraphConfig
from xpu_graph_amd.config import OptLevel


class ScaledLinear(nn.Module):
    def __init__(self):
        super().__init__()
        self.w = nn.Parameter(torch.randn(8, 8))
        self.register_buffer("b", torch.randn(8))

    def forward(self, x):
        return x @ (self.w.t() * 2.0) + self.b


def _compile(mod, freeze):
    be = XpuGraph(XpuGraphConfig(is_training=False, freeze=freeze, opt_level=OptLevel.level2))
    return torch.compile(mod, backend=be, dynamic=False), be


def test_freeze_unlifts_parameters_and_folds_the_weight_side():
    mod = ScaledLinear().eval()
    x = torch.randn(4, 8)
    fn, be = _compile(mod, freeze=True)
    with torch.no_grad():
        got = fn(x)
        torch.testing.assert_close(got, mod(x))
    gm = be.compiled_graphs[-1]
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    assert len(placeholders) == 1  # only the user input: the weight and the buffer are constants of the graph
    targets = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
    assert not any("aten.t." in t or "aten.mul." in t for t in targets), targets  # w.t() * 2.0 was folded
    with torch.no_grad():  # a second call runs the frozen graph with the user input only
        torch.testing.assert_close(fn(x + 1), mod(x + 1))


def test_without_freeze_the_weight_stays_an_input():
    mod = ScaledLinear().eval()
    fn, be = _compile(mod, freeze=False)
    with torch.no_grad():
        fn(torch.randn(4, 8))
    gm = be.compiled_graphs[-1]
    assert len([n for n in gm.graph.nodes if n.op == "placeholder"]) == 3


def test_freeze_keeps_a_parameter_that_is_returned_or_written():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.w = nn.Parameter(torch.randn(4))
            self.register_buffer("count", torch.zeros(()))

        def forward(self, x):
            self.count.add_(1)
            return x * self.w, self.w

    mod = M().eval()
    fn, be = _compile(mod, freeze=True)
    with torch.no_grad():
        y, w = fn(torch.ones(4))
        y2, _ = fn(torch.ones(4))
    torch.testing.assert_close(y, mod.w.detach())
    assert mod.count.item() == 2  # the in-place update still reaches the module's buffer
    assert w.data_ptr() == mod.w.data_ptr()  # returning a parameter returns the parameter, as eager does


def test_freeze_warns_when_parameters_arrive_as_inputs(caplog):
    w = torch.randn(8, 8)

    def fn(x, w):
        return x @ w

    be = XpuGraph(XpuGraphConfig(is_training=False, freeze=True, opt_level=OptLevel.level1))
    logging.getLogger("xpu_graph").propagate = True
    try:
        with caplog.at_level(logging.WARNING, logger="xpu_graph"):
            torch.compile(fn, backend=be, dynamic=False)(torch.randn(2, 8), w)
    finally:
        logging.getLogger("xpu_graph").propagate = False
    assert any("freeze=True has no effect" in r.getMessage() for r in caplog.records)


def test_a_folded_factory_that_is_returned_is_a_fresh_tensor_every_call():
    def f(x):
        z = torch.zeros(4)
        return z, x + 1

    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))
    c = torch.compile(f, backend=be, dynamic=False)
    x = torch.ones(4)
    a, _ = c(x)
    a.add_(1)
    b, _ = c(x)
    assert b.data_ptr() != a.data_ptr()
    torch.testing.assert_close(b, torch.zeros(4))


def test_two_returned_factories_do_not_alias_each_other():
    def f(x):
        return torch.zeros(4), torch.zeros(4), x * 2

    for level in (OptLevel.level1, OptLevel.level2):
        for folding in (True, False):
            be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=level, constant_folding=folding))
            a, b, _ = torch.compile(f, backend=be, dynamic=False)(torch.ones(4))
            a.add_(1)
            torch.testing.assert_close(b, torch.zeros(4))
            torch._dynamo.reset()


def test_a_view_of_a_folded_constant_is_returned_as_a_copy():
    def f(x):
        t = torch.arange(8.0).reshape(2, 4)
        return t[0], x + t.sum()

    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))
    c = torch.compile(f, backend=be, dynamic=False)
    a, _ = c(torch.ones(4))
    a.mul_(0)
    b, y = c(torch.ones(4))
    torch.testing.assert_close(b, torch.arange(4.0))
    torch.testing.assert_close(y, torch.ones(4) + 28.0)


def test_graph_runner_refreshes_its_inputs_outside_an_assert():
    import inspect

    from xpu_graph_amd import device_graph_runner

    src = inspect.getsource(device_graph_runner.HIPGraphRunner.forward)
    assert "assert self._copy_param_callback" not in src
