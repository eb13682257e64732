"""Device-graph partitioning on the host: which nodes a recording may hold, how a region's inputs are split
into owned and per-call tensors, one recording per input signature.  A stand-in runner with the GraphRunner
interface executes the region eagerly on the recorded buffers, so everything but the HIP capture itself is
exercised here (the capture runs in tests/test_gpu_hip_graph.py).
Reference behaviour: tests/mlu/test_mlu_graph.py:31-120, src/xpu_graph/backends/device_graph.py:14-130."""
import pytest
import torch
from torch.fx.experimental.proxy_tensor import make_fx

from xpu_graph_amd import GraphRunner, HIPGraphRunner, Target, XpuGraph, XpuGraphConfig
from xpu_graph_amd.backends import vendor_compiler
from xpu_graph_amd.backends.device_graph import DeviceGraphOperatorSupport, _LazyXPUGraph, device_graph_compiler


class ReplayOnBuffers(GraphRunner):
    """capture: keep the buffers the callback names, run nothing.  forward: refresh the buffers, then run the
    callable on the CAPTURED arguments -- a result that follows new inputs proves the buffers were refreshed."""

    captures = 0

    def capture(self, *args, memory_pool=None, clone_args=False, **kwargs):
        assert self._graph is None
        type(self).captures += 1
        self._graph = "recorded"
        self._args = args
        self._input_buffers = self._init_param_callback(*args, **kwargs)

    def forward(self, *args, **kwargs):
        assert self._copy_param_callback(self._input_buffers, *args, **kwargs)
        return self._callable_target(*self._args)


def _regions(gm):
    return [m for _, m in gm.named_children() if isinstance(m, _LazyXPUGraph)]


def test_runner_class_by_target():
    assert GraphRunner[Target.mi355x] is HIPGraphRunner
    assert GraphRunner[Target.none] is GraphRunner


def test_support_predicate():
    def f(x, n):
        y = torch.relu(x) * 2.0
        idx = torch.nonzero(y)  # data-dependent shape
        s = y.sum().item()  # synchronises
        z = y + n
        return z, idx, s

    gm = make_fx(f, tracing_mode="symbolic")(torch.randn(4, 4), torch.randn(4, 4))
    sup = DeviceGraphOperatorSupport("cpu")
    verdict = {str(n.target): sup.is_node_supported({}, n) for n in gm.graph.nodes if n.op == "call_function"}
    assert verdict["aten.relu.default"] and verdict["aten.mul.Tensor"] and verdict["aten.add.Tensor"]
    assert not verdict["aten.nonzero.default"]
    assert not verdict["aten._local_scalar_dense.default"]
    other = DeviceGraphOperatorSupport("cuda")
    assert not any(other.is_node_supported({}, n) for n in gm.graph.nodes if n.op == "call_function")
    assert not any(sup.is_node_supported({}, n) for n in gm.graph.nodes if n.op in ("placeholder", "output"))


def test_writes_into_arguments_stay_outside():
    def f(x, buf):
        y = x * 2.0
        buf.copy_(y)
        return y + 1.0

    gm = make_fx(f)(torch.randn(4), torch.zeros(4))
    out = device_graph_compiler(gm, [], "cpu", runner_cls=ReplayOnBuffers)
    top = [str(n.target) for n in out.graph.nodes if n.op == "call_function"]
    assert "aten.copy_.default" in top
    for _ in range(3):  # unrecorded first call, then recorded ones
        x, buf = torch.randn(4), torch.zeros(4)
        res = out(x, buf)
        torch.testing.assert_close(buf, x * 2.0)  # the caller's tensor was written, not a private copy
        torch.testing.assert_close(res, x * 2.0 + 1.0)


def test_mixed_graph_splits_around_the_unrecordable_node_and_replays_with_new_inputs():
    class Mixed(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.l1 = torch.nn.Linear(32, 32)
            self.l2 = torch.nn.Linear(32, 32)

        def forward(self, x):
            x = self.l1(x)
            keep = torch.nonzero(x.sum(dim=1) > -1e30).squeeze(1)  # a host-visible shape: breaks the recording
            x = x[keep]
            return self.l2(x)

    model = Mixed()
    x1 = torch.randn(16, 32)
    gm = make_fx(model)(x1)
    before = ReplayOnBuffers.captures
    out = device_graph_compiler(gm, [x1], "cpu", runner_cls=ReplayOnBuffers)
    regions = _regions(out)
    assert len(regions) >= 2
    torch.testing.assert_close(out(x1), model(x1))  # the first call runs unrecorded
    assert ReplayOnBuffers.captures == before
    x2, x3 = torch.randn(16, 32), torch.randn(16, 32)
    torch.testing.assert_close(out(x2), model(x2))
    torch.testing.assert_close(out(x3), model(x3))
    torch.testing.assert_close(out(x1), model(x1))
    first = regions[0]
    assert first.recorded == 1  # recorded once, replayed afterwards
    # parameters are owned by the outer module: recorded in place, not among the per-call buffers
    runner = next(iter(first._runners.values()))
    assert len(first._owned) == 2 and len(runner._input_buffers) == 1
    assert runner._input_buffers[0].data_ptr() not in (x1.data_ptr(), x2.data_ptr())  # clone_args: a private buffer


def test_one_recording_per_signature_with_eviction():
    def f(x, w):
        return torch.relu(x @ w)

    gm = make_fx(f, tracing_mode="symbolic")(torch.randn(4, 8), torch.randn(8, 8))
    out = device_graph_compiler(gm, [], "cpu", runner_cls=ReplayOnBuffers, max_graphs=2)
    (region,) = _regions(out)
    w = torch.randn(8, 8)
    for rows in (4, 6, 4, 6):
        x = torch.randn(rows, 8)
        torch.testing.assert_close(out(x, w), f(x, w))
    assert region.recorded == 2
    x = torch.randn(9, 8)
    torch.testing.assert_close(out(x, w), f(x, w))
    assert region.recorded == 2  # the least recently used recording made room


def test_clone_outputs_and_caller_buffers():
    def f(x):
        return x * 3.0

    gm = make_fx(f)(torch.randn(4))
    shared = device_graph_compiler(gm, [], "cpu", runner_cls=ReplayOnBuffers, clone_args=False)
    (region,) = _regions(shared)
    x, y = torch.randn(4), torch.randn(4)
    shared(x)
    shared(y)
    assert next(iter(region._runners.values()))._input_buffers[0].data_ptr() == y.data_ptr()  # the caller's own tensor
    gm2 = make_fx(f)(torch.randn(4))
    cloned = device_graph_compiler(gm2, [], "cpu", runner_cls=ReplayOnBuffers, clone_outputs=True)
    ins = [torch.full((4,), float(v)) for v in (1, 2, 3)]
    a, b, c = (cloned(t) for t in ins)
    for got, v in zip((a, b, c), (3.0, 6.0, 9.0)):
        torch.testing.assert_close(got, torch.full((4,), v))  # a later replay did not overwrite an earlier result


def test_tensors_that_keep_their_address_are_recorded_in_place():
    """Weights handed in as graph inputs (no get_attr) are not copied per call; one that moves later is."""

    def f(x, w):
        return x @ w

    gm = make_fx(f)(torch.randn(4, 8), torch.randn(8, 8))
    out = device_graph_compiler(gm, [], "cpu", runner_cls=ReplayOnBuffers)
    (region,) = _regions(out)
    w = torch.randn(8, 8)
    xs = [torch.randn(4, 8) for _ in range(5)]
    for x in xs[:3]:
        torch.testing.assert_close(out(x, w), f(x, w))
    runner = next(iter(region._runners.values()))
    assert region.recorded == 1 and len(runner._input_buffers) == 1  # x only: w is read where it lives
    w2 = torch.randn(8, 8)
    torch.testing.assert_close(out(xs[3], w2), f(xs[3], w2))  # w moved: recorded again, refreshed per call from now on
    w3 = torch.randn(8, 8)
    torch.testing.assert_close(out(xs[4], w3), f(xs[4], w3))
    runner = next(iter(region._runners.values()))
    assert region.recorded == 1 and len(runner._input_buffers) == 2


def test_vendor_compiler_hook_dispatches_by_target():
    def f(x):
        return x + 1

    gm = make_fx(f)(torch.randn(4))
    assert vendor_compiler(gm, [], Target.none, is_inference=True, mode="default") is gm  # no backend module
    assert vendor_compiler(gm, [], Target.mi355x, is_inference=True, mode="default") is gm  # nothing to compile with
    # training graphs are never recorded (saved activations would live in a pool the next replay overwrites): an
    # explicit error, not an assert that python -O drops
    with pytest.raises(ValueError, match="inference"):
        vendor_compiler(gm, [], Target.mi355x, is_inference=False, compiler="device_graph")


def test_backend_runs_the_hook_after_the_passes(monkeypatch):
    seen = []

    def fake_compile(gm, fake_inputs, *, is_inference=False, is_backward=False, **cfg):
        seen.append((is_inference, is_backward, cfg, [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]))
        return gm

    import xpu_graph_amd.backends.mi355x as backend_mod

    monkeypatch.setattr(backend_mod, "mi355x_compile", fake_compile)
    backend = XpuGraph(XpuGraphConfig(False, target=Target.mi355x, enable_cache=False, vendor_compiler_config={"compiler": "device_graph"}))

    def f(x):
        return x.expand(4, 4) * 2.0

    compiled = torch.compile(f, backend=backend, dynamic=False)
    x = torch.randn(4, 4)
    torch.testing.assert_close(compiled(x), f(x))
    assert len(seen) == 1
    is_inference, is_backward, cfg, targets = seen[0]
    assert is_inference and not is_backward and cfg == {"compiler": "device_graph"}
    assert targets == ["aten.mul.Tensor"]  # the hook sees the REWRITTEN graph (the same-shape expand is gone)
