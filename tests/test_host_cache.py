"""Compile-artifact cache (reference tests/common/test_cache.py:14-55): artifacts are saved once per distinct
graph, re-used after Dynamo's own caches are dropped, and what is loaded computes what the original computed."""
import operator
import os
import pickle

import pytest
import torch

from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig, XpuGraphLocalCache, mi355x_compiler, no_cache
from xpu_graph_amd.cache import SerializableGraphModule, graph_module_from_data, graph_module_to_data
from xpu_graph_amd.test_utils import need_xpu_graph_logs, skip_xpu_graph_cache


class SimpleModel(torch.nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.fc = torch.nn.Linear(dim, dim)
        self.w = torch.nn.Parameter(torch.randn(dim))

    def forward(self, x):
        h = torch.relu(self.fc(x))
        return h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6) * self.w


@pytest.mark.parametrize("freezing", [False, True])
def test_cache_saves_once_and_reuses(caplog, tmp_path, freezing):
    backend = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, freeze=freezing), XpuGraphLocalCache(tmp_path))
    model = SimpleModel(16).eval()
    with need_xpu_graph_logs(), torch.no_grad():
        for _ in range(2):
            compiled = torch.compile(model, backend=backend, dynamic=False)
            for bsz in (8, 10):
                x = torch.randn(bsz, 16)
                torch.testing.assert_close(compiled(x), model(x))
            torch._dynamo.reset()
    if freezing:
        # a frozen graph holds this model's parameters as constants, which the key (the graph's text) does not cover
        assert "Save cache in location" not in caplog.text and caplog.text.count("frozen graph: not cached") == 4
        return
    assert caplog.text.count("Save cache in location") == 2  # one artifact per batch size
    assert caplog.text.count("Use cache in location") == 2   # the second round compiles nothing
    assert len([f for f in os.listdir(tmp_path) if f.startswith("xpugraph_") and f.endswith(".pt")]) == 2


def test_cache_disabled_by_config_or_skip(caplog, tmp_path):
    off = XpuGraph(XpuGraphConfig(is_training=False, enable_cache=False), XpuGraphLocalCache(tmp_path / "a"))
    assert off._cache is None
    on = XpuGraph(XpuGraphConfig(is_training=False), XpuGraphLocalCache(tmp_path / "b"))
    fn = lambda x: torch.relu(x) + 1  # noqa: E731
    with need_xpu_graph_logs():
        torch.compile(fn, backend=off)(torch.randn(4))
        with skip_xpu_graph_cache(on):
            torch.compile(fn, backend=on)(torch.randn(4))
        assert isinstance(on._cache, XpuGraphLocalCache)  # restored
    assert "Save cache in location" not in caplog.text and os.listdir(tmp_path / "b") == []
    assert no_cache().load_artifact("anything") is None


def _signature(gm):
    ref = lambda a: a.name if isinstance(a, torch.fx.Node) else a  # noqa: E731
    return [(n.op, str(n.target), torch.fx.node.map_aggregate(n.args, ref), torch.fx.node.map_aggregate(n.kwargs, ref)) for n in gm.graph.nodes]


def test_mi355x_graph_round_trip(tmp_path):
    """A graph full of target modules and xpu_ops survives the file: same nodes, same module state."""
    backend = mi355x_compiler(cache=tmp_path)
    offs = [7, 100, 40, 200]

    def fn(src, x, r, w, cube, *ts):
        cat = torch.cat([src[:, o : o + 8] for o in offs], dim=1)
        acc = ts[0]
        for t in ts[1:]:
            acc = acc + t
        h = x + r
        y = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6) * w
        gathered = [src[:, s : s + 4] * 2 for s in (1, 9, 33)]
        sums = torch.cat([cube[:, 0:a, :].sum(1) for a in (2, 4, 6)], dim=1)
        return cat, acc, y, h, gathered, sums

    args = [torch.randn(6, 256), torch.randn(6, 64), torch.randn(6, 64), torch.randn(64), torch.randn(6, 8, 16)] + [torch.randn(6, 16) for _ in range(5)]
    with pytest.raises(NotImplementedError):  # CPU tensors: the custom ops refuse to run
        torch.compile(fn, backend=backend)(*args)
    gm = backend.compiled_graphs[-1]
    (path,) = [os.path.join(tmp_path, f) for f in os.listdir(tmp_path)]
    with open(path, "rb") as f:
        loaded = pickle.load(f).artifact
    assert _signature(loaded) == _signature(gm)
    mods = {n.target for n in gm.graph.nodes if n.op == "call_module"}
    assert {"fuse_slice_cat", "mi355x_addn", "mi355x_fused_add_norm", "fused_slice_0", "mi355x_slice_sum_cat_0"} <= mods
    assert loaded.get_submodule("fused_slice_0").slices_index == [1, 9, 33]
    assert loaded.get_submodule("mi355x_slice_sum_cat_0").slice_param == [(0, 2), (0, 4), (0, 6)]
    # the same compile again is a hit
    torch._dynamo.reset()
    with pytest.raises(NotImplementedError):
        torch.compile(fn, backend=backend)(*args)
    assert len(os.listdir(tmp_path)) == 1 and _signature(backend.compiled_graphs[-1]) == _signature(gm)


def test_graph_data_has_no_code_and_rejects_local_targets():
    def local_fn(x):
        return x + 1

    g = torch.fx.Graph()
    x = g.placeholder("x")
    y = g.call_function(torch.ops.aten.relu.default, (x,))
    z = g.call_function(operator.getitem, ((y, y), 0))
    g.output(z)
    gm = torch.fx.GraphModule(torch.nn.Module(), g)
    state, records = graph_module_to_data(gm)
    assert "_code" not in state and [r[2][0] for r in records] == ["name", "op", "py", "name"]
    back = graph_module_from_data(state, records)
    t = torch.randn(5)
    torch.testing.assert_close(back(t), gm(t))
    wrapped = SerializableGraphModule(gm)
    assert SerializableGraphModule(wrapped) is wrapped  # wrapping a wrapper is the identity
    torch.testing.assert_close(pickle.loads(pickle.dumps(wrapped))(t), gm(t))

    g2 = torch.fx.Graph()
    x2 = g2.placeholder("x")
    g2.output(g2.call_function(local_fn, (x2,)))
    with pytest.raises(NotImplementedError):
        graph_module_to_data(torch.fx.GraphModule(torch.nn.Module(), g2))
