"""Shape/dtype re-propagation after rewrites.

Only nodes that have no `meta["val"]` yet are evaluated (under the graph's
FakeTensorMode), which is what makes freshly inserted call_module /
call_function nodes visible to the next matcher.  Target modules therefore run
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


def propagate_missing(gm: fx.GraphModule, fake_mode):
    def val_of(n):
        return n.meta["val"]

    with enable_python_dispatcher(), fake_mode:
        for node in gm.graph.nodes:
            if "val" in node.meta or node.op == "output":
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
            if meta is not None:
                node.meta["val"] = meta
