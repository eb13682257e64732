"""The run-time parity guard (reference tests/common/test_interceptor.py:18-140): a faulty pattern is caught at the
first call, a sound pipeline stays silent, and `use_golden` decides whose results the caller sees."""
import os

import pytest
import torch

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.fx_utils import FxStage
from xpu_graph_amd.interceptor import OpInterceptor, parse_config
from xpu_graph_amd.passes.patterns.pattern import Pattern
from xpu_graph_amd.test_utils import need_xpu_graph_logs

aten = torch.ops.aten


def test_op_monitor_passes_and_fails(caplog, tmp_path, monkeypatch):
    monkeypatch.setattr("xpu_graph_amd.config._dump_dir", str(tmp_path))

    def slow_add(a, b):
        return torch.from_numpy(a.numpy(force=True) + b.numpy(force=True))

    x, y = torch.randn(2, 2), torch.randn(2, 2)
    with need_xpu_graph_logs():
        with OpInterceptor({aten.add.Tensor: slow_add}, check_device=False, check_dtype=False):
            c = x + y
        assert f"Monitored op: {aten.add.Tensor}" in caplog.text and "diverges" not in caplog.text
        with OpInterceptor({aten.add.Tensor: aten.sub.Tensor}, check_device=False, check_dtype=False):
            d = x + y
    torch.testing.assert_close(c, d)  # the real op's result is what the program sees
    assert "The op diverges" in caplog.text
    (case,) = os.listdir(tmp_path)
    dump = torch.load(os.path.join(tmp_path, case, "dump_glob_op.pt"), weights_only=True)
    torch.testing.assert_close(dump["golden_outputs"], x - y)


def test_parse_config():
    checks, golden = parse_config("rtol=1e-3,atol=1e-4,use_golden=1,check_dtype=false,bogus=3")
    assert checks == {"rtol": 1e-3, "atol": 1e-4, "check_dtype": False} and golden is True
    assert parse_config("") == ({}, False)


class AddBecomesSub(Pattern):
    _support_stages = [FxStage.inference, FxStage.forward, FxStage.backward]

    def process(self, gm):
        changed = False
        for node in gm.graph.nodes:
            if node.op == "call_function" and node.target == aten.add.Tensor:
                node.target = aten.sub.Tensor
                changed = True
        return changed


class InplaceModel(torch.nn.Module):
    def forward(self, x, buf):
        buf.add_(x)  # an input mutation: the guard must hand each function its own copy
        return buf * 2 + x


@pytest.mark.parametrize("use_golden", [True, False])
def test_inference_guard_catches_a_faulty_pattern(caplog, tmp_path, monkeypatch, use_golden):
    monkeypatch.setattr("xpu_graph_amd.config._dump_dir", str(tmp_path))
    cfg = XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, enable_cache=False, enable_interceptor=f"rtol=1e-6,atol=1e-5,use_golden={int(use_golden)}")
    backend = XpuGraph(cfg)
    backend.get_pattern_manager().register_pattern(AddBecomesSub())
    model = InplaceModel()
    x = torch.randn(4, 8)
    buf_c, buf_e = torch.ones(4, 8), torch.ones(4, 8)
    with need_xpu_graph_logs(), torch.no_grad():
        got = torch.compile(model, backend=backend)(x, buf_c)
    want = model(x, buf_e)
    assert "Monitored inference" in caplog.text and "The inference pass diverges" in caplog.text
    if use_golden:  # the caller got the golden function's results, mutation included
        torch.testing.assert_close(got, want)
        torch.testing.assert_close(buf_c, buf_e)
    else:
        assert not torch.allclose(got, want)
    (case,) = os.listdir(tmp_path)
    assert case.startswith("case_0_inference_") and os.path.isfile(os.path.join(tmp_path, case, "golden_mod.py"))
    dump = torch.load(os.path.join(tmp_path, case, "dump_glob_inf.pt"), weights_only=True)
    torch.testing.assert_close(dump["golden_outputs"][0], want)
    torch.testing.assert_close(dump["inputs"][0], torch.ones(4, 8))  # graph order (buf, x): inputs as they were before the call


def test_inference_guard_silent_when_sound(caplog, tmp_path, monkeypatch):
    monkeypatch.setattr("xpu_graph_amd.config._dump_dir", str(tmp_path))
    cfg = XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, enable_cache=False, enable_interceptor="rtol=1e-5,atol=1e-5")
    backend = XpuGraph(cfg)

    def fn(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

    x, w = torch.randn(8, 64), torch.randn(64)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend)(x, w)
    torch.testing.assert_close(got, fn(x, w))
    assert "Monitored inference" in caplog.text and "diverges" not in caplog.text and os.listdir(tmp_path) == []


def test_training_guard_checks_forward_and_backward(caplog, tmp_path, monkeypatch):
    monkeypatch.setattr("xpu_graph_amd.config._dump_dir", str(tmp_path))

    def fn(x, w):
        return torch.tanh(x @ w + x)

    def run(faulty):
        cfg = XpuGraphConfig(is_training=True, opt_level=OptLevel.level1, enable_cache=False, enable_interceptor="rtol=1e-5,atol=1e-5,use_golden=1")
        backend = XpuGraph(cfg)
        if faulty:
            backend.get_pattern_manager().register_pattern(AddBecomesSub())
        x = torch.randn(4, 4, requires_grad=True)
        w = torch.randn(4, 4, requires_grad=True)
        out = torch.compile(fn, backend=backend)(x, w)
        out.sum().backward()
        xe, we = x.detach().clone().requires_grad_(True), w.detach().clone().requires_grad_(True)
        fn(xe, we).sum().backward()
        torch.testing.assert_close(x.grad, xe.grad)  # use_golden: the golden gradients reach the leaves
        torch.testing.assert_close(w.grad, we.grad)

    with need_xpu_graph_logs():
        run(faulty=False)
        assert "Monitored forward" in caplog.text and "Monitored backward" in caplog.text and "diverges" not in caplog.text
        run(faulty=True)
    assert "The forward pass diverges" in caplog.text and "The backward pass diverges" in caplog.text
