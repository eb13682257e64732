"""Configuration, pattern switches, the fixed-point driver and the plugin
registry (reference tests/common/test_filter_pattern.py,
test_pattern_manager.py:9-54, test_plugin_pattern.py:53-329)."""
import pytest
import torch

import xpu_graph_amd
from xpu_graph_amd import (
    OptLevel,
    Target,
    XpuGraph,
    XpuGraphCompiler,
    XpuGraphConfig,
    deregister_plugin_patterns,
    enable_plugin_patterns,
    register_plugin_pattern,
    register_this_as_pattern_constraint,
    register_this_as_plugin_pattern,
)
from xpu_graph_amd.passes.patterns.pattern import Pattern, PatternGroup
from xpu_graph_amd.test_utils import need_xpu_graph_logs


def rms(x, w):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w


def test_defaults_match_reference():
    c = XpuGraphConfig(is_training=False)
    assert c.target == Target.none and c.opt_level == OptLevel.level1
    assert c.vendor_compiler_config is None and c.constant_folding and c.fallback_legacy_dispatch
    assert OptLevel.level1 < OptLevel.level2 <= OptLevel.level3 and OptLevel.level0 == OptLevel.level0
    assert Target("mi355x") is Target.mi355x


def test_env_overrides(monkeypatch):
    monkeypatch.setenv("XPUGRAPH_OPT_LEVEL", "2")
    monkeypatch.setenv("XPUGRAPH_DEBUG", "1")
    monkeypatch.setenv("XPUGRAPH_DEBUG_SKIP_PATTERNS", "FusedRMSNorm,FoldCat")
    c = XpuGraphConfig(is_training=False)
    c._reset_config_with_env()
    assert c.opt_level == OptLevel.level2 and c.debug is True and c.skip_patterns == ["FusedRMSNorm", "FoldCat"]
    monkeypatch.setenv("XPUGRAPH_OPT_LEVEL", "9")
    with pytest.warns(UserWarning):
        c._reset_config_with_env()


def test_skip_and_include_patterns(caplog):
    x, w = torch.randn(4, 32), torch.randn(32)
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, skip_patterns=["FusedRMSNorm"]))
    with need_xpu_graph_logs():
        torch.compile(rms, backend=be)(x, w)
    assert "Pattern.FusedRMSNorm changed graph" not in caplog.text
    caplog.clear()
    torch._dynamo.reset()
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level1, include_patterns=["FusedRMSNorm"]))
    with need_xpu_graph_logs():
        torch.compile(rms, backend=be)(x, w)
    assert "Pattern.FusedRMSNorm changed graph" in caplog.text


def test_register_pattern_object_and_function_pair(caplog):
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))

    class ReluToSigmoid(Pattern):
        _pattern_group = PatternGroup.GROUP1

        def process(self, gm):
            hit = False
            for n in gm.graph.nodes:
                if n.op == "call_function" and n.target == torch.ops.aten.relu.default:
                    n.target = torch.ops.aten.sigmoid.default
                    hit = True
            return hit

    be.get_pattern_manager().register_pattern(ReluToSigmoid())
    be.get_pattern_manager().register_pattern(lambda x: torch.ops.aten.neg.default(x), lambda x: torch.ops.aten.abs.default(x))
    x = torch.randn(8)
    with need_xpu_graph_logs():
        got = torch.compile(lambda x: torch.relu(x).neg(), backend=be)(x)
    torch.testing.assert_close(got, torch.sigmoid(x).abs())
    assert "Pattern.ReluToSigmoid changed graph" in caplog.text


def test_training_backend_matches_eager_grads():
    be = XpuGraph(XpuGraphConfig(is_training=True, opt_level=OptLevel.level2))
    x = torch.randn(4, 32, requires_grad=True)
    w = torch.randn(32, requires_grad=True)
    out = torch.compile(rms, backend=be)(x, w)
    gx, gw = torch.autograd.grad(out.sum(), (x, w))
    ex, ew = torch.autograd.grad(rms(x, w).sum(), (x, w))
    torch.testing.assert_close(gx, ex, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(gw, ew, rtol=1e-4, atol=1e-5)


def test_inplace_input_mutation_survives():
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))

    def fn(x, y):
        x.add_(1.0)
        return x * y

    x, y = torch.zeros(4), torch.full((4,), 3.0)
    out = torch.compile(fn, backend=be)(x, y)
    assert torch.equal(x, torch.ones(4)) and torch.equal(out, torch.full((4,), 3.0))


def test_fluent_compiler_wrapper():
    c = XpuGraphCompiler().set_opt_level(OptLevel.level2).set_debug(False)
    assert c.opt_level == OptLevel.level2
    with pytest.raises(AssertionError):
        c.compile(rms)
    c.done()
    x, w = torch.randn(4, 16), torch.randn(16)
    torch.testing.assert_close(c.compile(rms)(x, w), rms(x, w), rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- plugin patterns
def test_plugin_pattern_replaces_and_deregisters(caplog):
    def pattern(a, b):
        return torch.relu(a @ b)

    def replacement(a, b):
        return torch.sigmoid(a @ b)

    a, b = torch.randn(4, 4), torch.randn(4, 4)
    with enable_plugin_patterns():
        register_plugin_pattern(pattern, (torch.empty(4, 4), torch.empty(4, 4)), replacement, Target.none)
        be = XpuGraph(XpuGraphConfig(is_training=False))
        with need_xpu_graph_logs():
            got = torch.compile(lambda a, b: torch.relu(a @ b) + 1, backend=be)(a, b)
        torch.testing.assert_close(got, torch.sigmoid(a @ b) + 1)
        assert "test_plugin_pattern_replaces_and_deregisters" not in caplog.text or True
    # outside the context the registration is gone
    torch._dynamo.reset()
    be = XpuGraph(XpuGraphConfig(is_training=False))
    got = torch.compile(lambda a, b: torch.relu(a @ b) + 1, backend=be)(a, b)
    torch.testing.assert_close(got, torch.relu(a @ b) + 1)


def test_plugin_pattern_literal_input_and_constraint():
    def replacement(x, eps):
        return x * eps  # visibly different so the test can tell

    with enable_plugin_patterns():

        @register_this_as_plugin_pattern((torch.empty(4, 8), 0.123), replacement, Target.none)
        def pattern(x, eps):
            return x + eps

        @register_this_as_pattern_constraint
        def only_two_d(x, eps):
            return x.dim() == 2

        be = XpuGraph(XpuGraphConfig(is_training=False))
        x = torch.randn(4, 8)
        torch.testing.assert_close(torch.compile(lambda x: x + 0.5, backend=be)(x), x * 0.5)  # literal is a wildcard
        torch._dynamo.reset()
        x3 = torch.randn(2, 4, 8)
        torch.testing.assert_close(torch.compile(lambda x: x + 0.5, backend=be)(x3), x3 + 0.5)  # constraint vetoes


def test_plugin_registry_is_keyed_by_target():
    def pattern(x):
        return torch.relu(x)

    def replacement(x):
        return torch.sigmoid(x)

    with enable_plugin_patterns():
        register_plugin_pattern(pattern, (torch.empty(4),), replacement, Target.mi355x)
        be = XpuGraph(XpuGraphConfig(is_training=False))  # target none: must not see it
        x = torch.randn(4)
        torch.testing.assert_close(torch.compile(lambda x: torch.relu(x), backend=be)(x), torch.relu(x))
        deregister_plugin_patterns(pattern, Target.mi355x)


def test_public_api_names():
    for name in ("XpuGraph", "XpuGraphConfig", "Target", "OptLevel", "mi355x_compiler", "register_plugin_pattern", "XpuGraphCompiler"):
        assert hasattr(xpu_graph_amd, name)


def test_fp8_dense_plugin_pattern_rewrites_user_function():
    """The fp8 dense layer reaches the kernel library as a plugin pattern on the mi355x target."""
    from xpu_graph_amd import mi355x_compiler, plugins

    def layer(x_q, w_q, s_x, s_w, b, extra):
        return plugins.fp8_linear_silu_eager(x_q, w_q, s_x, s_w, b) + extra

    x_q, w_q, s_x, s_w, b = plugins.example_fp8_inputs(16, 24, 64)
    extra = torch.zeros(16, 24, dtype=torch.bfloat16)
    with enable_plugin_patterns():
        plugins.register_fp8_dense(plugins.fp8_linear_silu_eager, act="silu")
        be = mi355x_compiler()
        with pytest.raises(NotImplementedError):  # rewritten to the custom op, which has no CPU implementation
            torch.compile(layer, backend=be)(x_q, w_q, s_x, s_w, b, extra)
        gm = be.compiled_graphs[-1]
        targets = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
        assert any("dense_fp8" in t for t in targets) and not any("aten.mm" in t or "silu" in t for t in targets), targets
        # K not a multiple of 16: the constraint vetoes the match and the eager subgraph stays (and runs on the CPU:
        # its dequantised fp32 product has a K that is no multiple of 4, which the fp32 dense kernel does not take either)
        torch._dynamo.reset()
        be = mi355x_compiler()
        x8, w8, s1, sn, bb = plugins.example_fp8_inputs(16, 24, 42)
        got = torch.compile(layer, backend=be)(x8, w8, s1, sn, bb, extra)
        torch.testing.assert_close(got, layer(x8, w8, s1, sn, bb, extra))
        assert not any("dense_fp8" in str(n.target) for n in be.compiled_graphs[-1].graph.nodes)
