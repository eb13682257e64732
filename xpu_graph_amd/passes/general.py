"""Target-independent clean-up passes that keep graphs canonical for the matchers:
assertion removal, view->reshape, dead-code elimination, common-subexpression
elimination and folding of constant subgraphs.

Behaviour follows the reference's passes of the same names
(src/xpu_graph/passes/{remove_runtime_assertions,view_to_reshape,dce,cse,constant_folding}.py).
"""
import torch
import torch.fx as fx
import torch.utils._pytree as pytree

from ..fx_utils import FxStage, outside_fake_mode
from ..utils import logger
from .optimizer import Optimizer

aten = torch.ops.aten
_ALL_STAGES = [FxStage.inference, FxStage.pregrad, FxStage.forward, FxStage.backward]


class RemoveAssertions(Optimizer):
    """Drops aten._assert_tensor_metadata nodes: they add users that defeat single-use checks."""

    _support_stages = _ALL_STAGES

    def process(self, gm):
        if not hasattr(aten, "_assert_tensor_metadata"):
            return False
        victims = list(gm.graph.find_nodes(op="call_function", target=aten._assert_tensor_metadata.default))
        for n in victims:
            gm.graph.erase_node(n)
        return bool(victims)


class ViewToReshape(Optimizer):
    """view/_unsafe_view -> reshape: later rewrites may change input strides, reshape stays valid."""

    _support_stages = _ALL_STAGES

    def process(self, gm):
        changed = False
        for n in gm.graph.nodes:
            if n.op == "call_function" and n.target in (aten.view.default, aten._unsafe_view.default):
                n.target = aten.reshape.default
                changed = True
        return changed


class Dce(Optimizer):
    _support_stages = _ALL_STAGES

    def process(self, gm):
        changed = gm.graph.eliminate_dead_code()
        used = {n.target for n in gm.graph.nodes if n.op == "get_attr"}
        for name in [k for k in getattr(gm, "_xg_constants", ()) if k not in used]:
            delattr(gm, name)
            gm._xg_constants.remove(name)
            changed = True
        return changed


def _hashable(x):
    if isinstance(x, (list, tuple)):
        return tuple(_hashable(i) for i in x)
    if isinstance(x, dict):
        return tuple(sorted((k, _hashable(v)) for k, v in x.items()))
    if isinstance(x, fx.Node):
        return ("node", id(x))
    if isinstance(x, (torch.dtype, torch.device, torch.layout, torch.memory_format, str, int, float, bool, type(None), slice)):
        return (type(x).__name__, x if not isinstance(x, slice) else (x.start, x.stop, x.step))
    return ("obj", id(x))


class Cse(Optimizer):
    """Merges repeated pure call_function nodes with identical targets and arguments."""

    _support_stages = _ALL_STAGES

    @staticmethod
    def _mergeable(node):
        if node.op != "call_function" or node.is_impure():
            return False
        tgt = node.target
        if isinstance(tgt, torch._ops.OpOverload):
            if torch.Tag.nondeterministic_seeded in tgt.tags or tgt._schema.is_mutable:
                return False
            name = tgt._schema.name
            # factories and copies return fresh storage that later in-place ops may write
            if name.startswith("aten::empty") or name in ("aten::clone", "aten::_to_copy", "aten::copy"):
                return False
            # a call with no tensor input (zeros, full, arange, ...) makes a fresh tensor each time: two of them are
            # two tensors, which the caller may go on to write separately
            flat, _ = pytree.tree_flatten((node.args, node.kwargs))
            if not any(isinstance(a, fx.Node) for a in flat):
                return False
            return True
        return tgt.__module__ == "_operator"

    def process(self, gm):
        seen = {}
        changed = False
        for node in list(gm.graph.nodes):
            if not self._mergeable(node):
                continue
            key = (node.target, _hashable(node.args), _hashable(node.kwargs))
            prev = seen.get(key)
            if prev is None:
                seen[key] = node
            else:
                node.replace_all_uses_with(prev)
                gm.graph.erase_node(node)
                changed = True
        return changed


def is_constant(arg, include_params=True):
    """Python scalars, and get_attr nodes (graph constants; parameters when include_params)."""
    if isinstance(arg, fx.Node):
        if arg.op != "get_attr":
            return False
        if include_params:
            return True
        return arg.target in getattr(arg.graph.owning_module, "_xg_constants", ())
    return True


class ConstantFolding(Optimizer):
    """Evaluates call_function nodes whose inputs are all constants and stores the
    result as a module attribute read through get_attr."""

    def __init__(self, folding_params=False):
        super().__init__()
        self.folding_params = folding_params

    @staticmethod
    def _foldable_factory(node):
        """A call with no tensor input (arange, full, ...) folds like any other constant expression -- position
        tables and masks are built from them -- unless its value is not a function of its arguments."""
        tgt = node.target
        if not isinstance(tgt, torch._ops.OpOverload):
            return False
        name = tgt._schema.name
        if torch.Tag.nondeterministic_seeded in tgt.tags or name.startswith("aten::empty") or name.startswith("aten::new_empty"):
            return False
        val = node.meta.get("val")
        return isinstance(val, torch.Tensor) and all(isinstance(d, int) for d in val.shape)

    def process(self, gm):
        graph = gm.graph
        anchor = None
        for anchor in graph.nodes:
            if anchor.op not in ("placeholder", "get_attr"):
                break
        changed = False
        for node in list(graph.nodes):
            if node.op != "call_function" or node.is_impure():
                continue
            flat, _ = pytree.tree_flatten((node.args, node.kwargs))
            if not all(is_constant(a, self.folding_params) for a in flat):
                continue
            if not any(isinstance(a, fx.Node) for a in flat) and not self._foldable_factory(node):
                continue
            if node.target is torch.ops.aten.clone.default and node.users and all(u.op == "output" for u in node.users):
                continue  # the copy that keeps a constant from being handed to the caller (see _protect_outputs)
            args, kwargs = pytree.tree_map(lambda a: getattr(gm, a.target) if isinstance(a, fx.Node) else a, (node.args, node.kwargs))
            logger.info(f"start constant folding: {node.name} {node.target}")
            with outside_fake_mode():
                value = node.target(*args, **kwargs)
            if not isinstance(value, torch.Tensor):
                continue
            name = f"_xg_folded_{node.name}"
            gm.register_buffer(name, value, persistent=False)
            if not hasattr(gm, "_xg_constants"):
                gm._xg_constants = []
            gm._xg_constants.append(name)
            with graph.inserting_before(anchor):
                const = graph.get_attr(name)
            node.replace_all_uses_with(const)
            changed = True
        return self._protect_outputs(gm) or changed

    _VIEW_OPS = (
        "aten::view", "aten::reshape", "aten::_unsafe_view", "aten::expand", "aten::permute", "aten::transpose", "aten::t",
        "aten::slice", "aten::select", "aten::unsqueeze", "aten::squeeze", "aten::alias", "aten::detach", "aten::as_strided",
    )

    @classmethod
    def _folded_base(cls, gm, node):
        """The folded constant `node` is (a view of), or None."""
        while isinstance(node, fx.Node):
            if node.op == "get_attr":
                return node if node.target in getattr(gm, "_xg_constants", ()) else None
            tgt = node.target
            if node.op == "call_function" and isinstance(tgt, torch._ops.OpOverload) and tgt._schema.name in cls._VIEW_OPS and node.args:
                node = node.args[0]
                continue
            return None
        return None

    def _protect_outputs(self, gm):
        """A folded constant lives in the module and would be handed to the caller again on every call: whoever writes
        into a result (a freshly initialised cache or accumulator) would change the next call's result, and two
        outputs folded to one constant would alias each other.  Every output that is (a view of) a folded constant is
        returned as a copy, which is what eager and the unfolded graph return: a fresh tensor."""
        out_node = next(n for n in reversed(gm.graph.nodes) if n.op == "output")
        changed = False

        def fix(arg):
            nonlocal changed
            if isinstance(arg, fx.Node) and self._folded_base(gm, arg) is not None:
                with gm.graph.inserting_before(out_node):
                    fresh = gm.graph.call_function(torch.ops.aten.clone.default, (arg,))
                if "val" in arg.meta:
                    fresh.meta["val"] = arg.meta["val"]
                changed = True
                return fresh
            return arg

        new_args = fx.map_arg(out_node.args, fix)
        if changed:
            out_node.args = new_args
        return changed
