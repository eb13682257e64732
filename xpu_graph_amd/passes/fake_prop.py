"""Shape/dtype re-propagation after rewrites.

Only nodes that have no `meta["val"]` yet, and the nodes downstream of them whose
value changes as a result, are evaluated (under the graph's FakeTensorMode),
which is what makes freshly inserted call_module / call_function nodes visible
to the next matcher.  Target modules therefore run
their `forward` on FakeTensors here, and every custom op needs a Meta kernel.
Same contract as the reference's FakeTensorProp
(src/xpu_graph/passes/fake_tensor_prop.py:17-79).
"""
import torch
import torch.fx as fx
from torch._dispatch.python import enable_python_dispatcher
from torch._subclasses.fake_tensor import FakeTensor
from torch.fx.node import map_aggregate

_SYM = (torch.SymInt, torch.SymFloat, torch.SymBool)


def _snapshot(mode, obj):
    if isinstance(obj, FakeTensor):
        return obj.detach()
    if isinstance(obj, torch.Tensor):
        return mode.from_tensor(obj, static_shapes=True)
    if isinstance(obj, _SYM) or isinstance(obj, (int, float, bool)):
        return obj
    return None


def _same_layout(a, b):
    """Do two meta values describe the same tensors (shape, stride, dtype), element by element?"""
    if isinstance(a, (list, tuple)) and isinstance(b, (list, tuple)):
        return len(a) == len(b) and all(_same_layout(x, y) for x, y in zip(a, b))
    if isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor):
        return a.dtype == b.dtype and a.shape == b.shape and a.stride() == b.stride()
    return type(a) is type(b) and (a is b or a == b)


def _layout_sig(val):
    if isinstance(val, (list, tuple)):
        return tuple(_layout_sig(v) for v in val)
    if isinstance(val, torch.Tensor):
        return (str(tuple(val.shape)), str(tuple(val.stride())), str(val.dtype))
    return None


def _input_sig(node):
    """Which nodes feed `node`, and in which layout: a value computed for other inputs is stale."""
    return tuple((i.name, _layout_sig(i.meta.get("val"))) for i in node.all_input_nodes)


def propagate_missing(gm: fx.GraphModule, fake_mode):
    """Evaluate nodes without a fake value or whose inputs were rewired, and re-evaluate the nodes downstream of
    them for as long as the result changes: a replacement may return a different memory layout than the subgraph
    it stands for, and the strides recorded on its users (views, copies) would otherwise be stale."""

    def val_of(n):
        return n.meta["val"]

    changed_nodes = set()
    with enable_python_dispatcher(), fake_mode:
        for node in gm.graph.nodes:
            if node.op == "output":
                continue
            missing = "val" not in node.meta
            sig = _input_sig(node)
            rewired = node.meta.get("xg_in_sig", sig) != sig  # a pass gave this node other inputs since its value was computed
            if not missing and not rewired and not any(i in changed_nodes for i in node.all_input_nodes):
                node.meta["xg_in_sig"] = sig
                continue
            if node.op == "placeholder":
                raise RuntimeError(f"placeholder {node.name} carries no fake value")
            if node.op == "get_attr":
                obj = gm
                for part in node.target.split("."):
                    obj = getattr(obj, part)
                out = obj
            else:
                args = fx.map_arg(node.args, val_of)
                kwargs = fx.map_arg(node.kwargs, val_of)
                if node.op == "call_function":
                    out = node.target(*args, **kwargs)
                elif node.op == "call_module":
                    out = gm.get_submodule(node.target)(*args, **kwargs)
                elif node.op == "call_method":
                    out = getattr(args[0], node.target)(*args[1:], **kwargs)
                else:
                    raise RuntimeError(f"unexpected node op {node.op}")
            meta = map_aggregate(out, lambda o: _snapshot(fake_mode, o))
            if meta is None:
                continue
            if missing or not _same_layout(node.meta["val"], meta):
                changed_nodes.add(node)
            node.meta["val"] = meta
            node.meta["xg_in_sig"] = sig
