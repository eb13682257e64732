"""User-registered patterns: an eager function is traced to Aten IR once and
every occurrence of that subgraph is replaced by a (symbolically traced)
replacement function.  API of the reference's plugin registry
(src/xpu_graph/passes/patterns/plugin_pattern.py:114-284): patterns are keyed
by target and by "<module>-<function name>", run before the built-in patterns,
and can carry extra checks over the FakeTensors bound to the pattern's inputs.
The registry is process-global and not thread safe.
"""
import contextlib
import inspect
from typing import Callable, Union

import torch
from torch import fx
from torch.fx import subgraph_rewriter, symbolic_trace
from torch.fx.experimental.proxy_tensor import make_fx
from torch.utils import _pytree as pytree

from ...config import Target
from ...fx_utils import FxStage
from ...utils import logger
from .pattern import Pattern

__all__ = [
    "register_plugin_pattern",
    "register_this_as_plugin_pattern",
    "register_this_as_pattern_constraint",
    "deregister_plugin_patterns",
    "enable_plugin_patterns",
]

_LITERALS = (float, int, bool)
aten = torch.ops.aten


def _trace_to_aten(fn, example_inputs):
    """Aten-IR graph of `fn` with one placeholder per parameter (python-number inputs included)."""
    gm = make_fx(fn, tracing_mode="fake", _allow_non_fake_inputs=True)(*example_inputs)
    for n in gm.graph.nodes:
        if n.op == "call_function" and n.target in (aten.view.default, aten._unsafe_view.default):
            n.target = aten.reshape.default  # the graphs being searched have had this rewrite applied
    gm.graph.eliminate_dead_code()
    gm.recompile()
    return gm


class PluginPattern(Pattern):
    def __init__(self, eager_func, example_inputs, replacement, filter_list=None, is_training=False, name=None, ignore_literal=False):
        super().__init__()
        self.set_current_stage(FxStage.pregrad if is_training else FxStage.inference)
        self._support_stages = [self._current_stage]
        self._eager_pattern = _trace_to_aten(eager_func, example_inputs)
        self._replacement = symbolic_trace(replacement)
        self._filter_list = list(filter_list) if filter_list else []
        self._bind_literal_inputs(example_inputs)
        self.name = name
        self.ignore_literal = ignore_literal
        logger.debug(
            "Pattern %s-%s : %s\n with Replacement %s", eager_func.__module__, eager_func.__name__, self._eager_pattern.graph, self._replacement.graph
        )

    def _bind_literal_inputs(self, example_inputs):
        """Tracing bakes python-number inputs into the graph as constants; put the placeholder back
        wherever such a (unique) value occurs, so the number becomes a wildcard of the pattern."""
        where = {}
        for i, v in enumerate(example_inputs):
            if isinstance(v, _LITERALS):
                if v in where:
                    raise ValueError(
                        "You should make sure that all the literal example inputs are unique. You should also make sure that the literal "
                        "example inputs MUST be different from thoes non-input literals in pattern and replacement!"
                    )
                where[v] = i
        if not where:
            return
        graph = self._eager_pattern.graph
        placeholders = graph.find_nodes(op="placeholder")

        def swap(a):
            return placeholders[where[a]] if isinstance(a, _LITERALS) and a in where else a

        for n in graph.nodes:
            n.args = pytree.tree_map(swap, n.args)
            n.kwargs = pytree.tree_map(swap, n.kwargs)
        graph.lint()
        self._eager_pattern.recompile()

    @property
    def filter_list(self):
        return self._filter_list

    def process(self, gm):
        hits = subgraph_rewriter.replace_pattern_with_filters(
            gm, self._eager_pattern, self._replacement, self._filter_list, ignore_literals=self.ignore_literal
        )
        return len(hits) > 0

    def __str__(self):
        return self.name or super().__str__()


__PLUGIN_PATTERN_GROUP__ = {}
_last_registered = None
_recorder = []


def _as_match_filter(check):
    def match_filter(match, gm, pattern_graph):
        ok = check(*[p.meta["val"] if isinstance(p, fx.Node) else p for p in match.placeholder_nodes])  # literals bind as values
        assert isinstance(ok, bool)
        return ok

    return match_filter


def register_plugin_pattern(eager_func, example_inputs, replacement, target: Target, extra_checks=None, is_training=False, postfix=None, ignore_literal=False):
    key = f"{eager_func.__module__}-{eager_func.__name__}"
    sig = inspect.signature(eager_func)
    assert len(example_inputs) == len(sig.parameters), (
        f"You should provide the same number of example inputs as the number of parameters in the function {key}"
    )
    assert inspect.signature(replacement) == sig, (
        f"The signature of the replacement function {replacement.__name__} should be the same as the signature of the function {key}."
    )
    filters = [_as_match_filter(c) for c in extra_checks] if extra_checks else None
    if isinstance(_recorder, list):
        _recorder.append(eager_func)
    pat = PluginPattern(eager_func, example_inputs, replacement, filters, is_training, f"{key}-{postfix}" if postfix else key, ignore_literal)
    __PLUGIN_PATTERN_GROUP__.setdefault(target, {}).setdefault(key, []).append(pat)
    global _last_registered
    _last_registered = (key, sig, target)


def _with_fewer_args(func, argument_elimination):
    """A function with the signature of `argument_elimination` that forwards func(*args, **kwargs) of its result
    (symbolic tracing needs a fixed signature, hence the generated def)."""
    sig = inspect.signature(argument_elimination)
    assert len(sig.parameters) <= len(inspect.signature(func).parameters)
    scope = {"_elim": argument_elimination, "_func": func}
    exec(f"def _new{sig}:\n    a, k = _elim{sig}\n    return _func(*a, **k)\n", scope)
    new = scope["_new"]
    new.__name__, new.__module__, new.__signature__ = func.__name__, func.__module__, sig
    return new


def register_this_as_plugin_pattern(example_inputs, replacement, target, extra_checks=None, is_training=False, argument_elimination=None, postfix=None, ignore_literal=False):
    def decorate(func):
        f, r = func, replacement
        if argument_elimination:
            f, r = _with_fewer_args(func, argument_elimination), _with_fewer_args(replacement, argument_elimination)
        register_plugin_pattern(f, example_inputs, r, target, extra_checks, is_training, postfix, ignore_literal)
        return func

    return decorate


def register_this_as_pattern_constraint(func):
    assert _last_registered is not None
    key, sig, target = _last_registered
    assert inspect.signature(func) == sig
    for pat in __PLUGIN_PATTERN_GROUP__.get(target, {}).get(key, []):
        pat.filter_list.append(_as_match_filter(func))
    logger.debug("Register constraint %s for %s successfully.", func.__name__, key)
    return func


def deregister_plugin_patterns(func_or_func_name: Union[Callable, str], target=None):
    if callable(func_or_func_name):
        key = f"{func_or_func_name.__module__}-{func_or_func_name.__name__}"
    elif isinstance(func_or_func_name, str):
        key = func_or_func_name
    else:
        raise ValueError("func_or_func_name should be Callable or str")
    groups = [__PLUGIN_PATTERN_GROUP__.get(target, {})] if target else list(__PLUGIN_PATTERN_GROUP__.values())
    for g in groups:
        if key in g:
            del g[key]
            logger.debug("Deregister pattern %s successfully.", key)


@contextlib.contextmanager
def enable_plugin_patterns():
    """Patterns registered inside the block are removed again when it exits."""
    global _recorder
    saved, _recorder = _recorder, []
    try:
        yield
    finally:
        for f in _recorder:
            deregister_plugin_patterns(f)
        _recorder = saved
