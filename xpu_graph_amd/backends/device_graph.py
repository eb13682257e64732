"""Split a rewritten graph into the parts a HIP graph can record and run each of them through a graph runner.

Interface of the reference (src/xpu_graph/backends/device_graph.py:14-130): `DeviceGraphOperatorSupport` says
which nodes may be recorded, `device_graph_compiler(module, example_inputs, target, **config)` returns the
module with every recordable region replaced by a `_LazyXPUGraph` that captures on its first call and replays
afterwards.  Configuration keys: `memory_pool`, `clone_args` (both as in the reference), `clone_outputs`,
`max_graphs`.

What is recorded: nodes whose tensors all live on the target device (everything in the `xpu_ops` namespace
does), minus the nodes a recording cannot hold -- results whose shape or value depends on data (they
synchronise), host arithmetic on sizes, and operators that write into one of their arguments (a recording
runs on private copies of its inputs, so the write would miss the caller's tensor).

How a region runs: the first call runs it unrecorded.  From the second call on its inputs are split into
tensors recorded in place -- those the outer module owns (parameters and constants reached by get_attr) and those
that kept their address since the first call (weights passed as graph inputs, a fixed input buffer) -- and
per-call tensors, copied into buffers the recording reads.  One recording is kept per input signature (shapes,
strides, dtypes, integer arguments, addresses of the tensors recorded in place), so a region reached with several
batch sizes records once per size.
The tensors a region returns live in the recording's memory pool and are overwritten by its next replay unless
`clone_outputs` is set.
"""
import operator
from collections import OrderedDict
from typing import Dict

import torch
import torch.fx
from torch.fx.node import Node
from torch.fx.passes.operator_support import OperatorSupport
from torch.utils import _pytree

from ..utils import logger

__all__ = ["DeviceGraphOperatorSupport", "device_graph_compiler"]

_CALLABLE = ("call_function", "call_method", "call_module")
_RECORDABLE_NAMESPACES = ("xpu_ops",)
_UNRECORDABLE_TAGS = tuple(
    t for t in (getattr(torch.Tag, "data_dependent_output", None), getattr(torch.Tag, "dynamic_output_shape", None)) if t is not None
)


def _meta_value(node):
    return node.meta.get("val", node.meta.get("fake_result", None))


def _tensors_in(value):
    return [t for t in _pytree.tree_leaves(value) if isinstance(t, torch.Tensor)]


def _writes_an_argument(target):
    schema = getattr(target, "_schema", None)
    return schema is not None and schema.is_mutable


class DeviceGraphOperatorSupport(OperatorSupport):
    def __init__(self, target_device: str):
        super().__init__()
        self.target_device = torch.device(target_device).type

    def is_node_supported(self, submodules, node: Node) -> bool:
        if node.op not in _CALLABLE:
            return False
        if node.target is operator.getitem:
            # follows its producer: a tuple result taken apart inside the recording costs nothing
            return all(self.is_node_supported(submodules, p) for p in node.all_input_nodes if p.op in _CALLABLE)
        if getattr(node.target, "namespace", None) in _RECORDABLE_NAMESPACES:
            return True
        tags = getattr(node.target, "tags", ())
        if any(t in tags for t in _UNRECORDABLE_TAGS) or _writes_an_argument(node.target):
            return False
        produced = _tensors_in(_meta_value(node))
        if not produced:
            return False  # size arithmetic and other host values stay on the host
        consumed = [t for p in node.all_input_nodes for t in _tensors_in(_meta_value(p))]
        return all(t.device.type == self.target_device for t in produced + consumed)


def _signature(args, owned):
    sig = []
    for i, a in enumerate(args):
        if isinstance(a, torch.Tensor):
            sig.append((tuple(a.shape), tuple(a.stride()), a.dtype, a.data_ptr() if i in owned else None))
        elif isinstance(a, (int, float, bool, str, type(None), torch.dtype, torch.device)):
            sig.append(a)
        else:
            sig.append(repr(a))
    return tuple(sig)


class _LazyXPUGraph(torch.nn.Module):
    """One recordable region.

    The first call runs the region as it is: operators before the region may change state it reads, modules inside
    it may build tables on first use, and only a later call can tell which arguments keep their address from call
    to call (weights handed in as graph inputs, a caller's fixed input buffer).  Such tensors are recorded where
    they are, like the owned ones; the others get buffers that every call refreshes.  A tensor that was taken for
    fixed and then moves is refreshed like the others from then on (all recordings are made again, once)."""

    def __init__(self, region: torch.nn.Module, runner_cls, owned_positions=(), memory_pool=None, clone_args=True,
                 clone_outputs=False, max_graphs=8):
        super().__init__()
        self.region = region
        self._runner_cls = runner_cls
        self._owned = frozenset(owned_positions)
        self._memory_pool = memory_pool
        self._clone_args = bool(clone_args)
        self._clone_outputs = bool(clone_outputs)
        self._max_graphs = max(1, int(max_graphs))
        self._runners = OrderedDict()  # signature -> runner, least recently used first
        self._first_ptrs = None  # addresses of the tensor arguments of the first call
        self._fixed = None  # positions recorded in place (owned + those that kept their address) -> address

    @property
    def recorded(self):
        return len(self._runners)

    @staticmethod
    def _ptrs(args):
        return [a.data_ptr() if isinstance(a, torch.Tensor) else None for a in args]

    def _per_call(self, args):
        return [a for i, a in enumerate(args) if isinstance(a, torch.Tensor) and i not in self._fixed]

    def _settle_fixed(self, args):
        now = self._ptrs(args)
        if self._fixed is None:
            keep = [
                i
                for i, (was, is_) in enumerate(zip(self._first_ptrs, now))
                if is_ is not None and (i in self._owned or was == is_ or isinstance(args[i], torch.nn.Parameter))
            ]
            self._fixed = {i: now[i] for i in keep}
            return
        moved = [i for i, ptr in self._fixed.items() if i not in self._owned and now[i] != ptr]
        if moved:
            logger.debug(f"device graph: arguments {moved} moved, they are refreshed per call from now on")
            for i in moved:
                del self._fixed[i]
            self._drop_recordings()
        for i in self._owned:  # a replaced parameter: its address is part of the signature
            if i in self._fixed:
                self._fixed[i] = now[i]

    def _drop_recordings(self):
        for runner in self._runners.values():
            runner.reset()
        self._runners.clear()

    def _new_runner(self, args):
        def init_param_callback(*a):
            return self._per_call(a)

        def copy_param_callback(buffers, *a):
            fresh = self._per_call(a)
            if len(fresh) != len(buffers):
                return False
            for dst, src in zip(buffers, fresh):
                if dst.data_ptr() != src.data_ptr():
                    dst.copy_(src)
            return True

        runner = self._runner_cls(self.region, init_param_callback=init_param_callback, copy_param_callback=copy_param_callback)
        if self._clone_args:
            # private buffers for the per-call tensors (the caller may free or overwrite its own between calls)
            args = [a.detach().clone() if isinstance(a, torch.Tensor) and i not in self._fixed else a for i, a in enumerate(args)]
        runner.capture(*args, memory_pool=self._memory_pool, clone_args=False)
        return runner

    def forward(self, *args):
        if self._first_ptrs is None:
            self._first_ptrs = self._ptrs(args)
            return self.region(*args)
        self._settle_fixed(args)
        key = _signature(args, self._fixed)
        runner = self._runners.get(key)
        if runner is None:
            if len(self._runners) >= self._max_graphs:
                _, oldest = self._runners.popitem(last=False)
                oldest.reset()
            logger.debug(f"device graph: recording for signature {key}")
            runner = self._new_runner(args)
            self._runners[key] = runner
        else:
            self._runners.move_to_end(key)
        # a recording holds no results: what the caller reads always comes from a replay
        out = runner(*args)
        if self._clone_outputs:
            out = _pytree.tree_map(lambda t: t.clone() if isinstance(t, torch.Tensor) else t, out)
        return out


def _owned_positions(outer: torch.fx.GraphModule, call_node: Node):
    """Argument positions of a region call that are fed by get_attr nodes of the outer module."""
    return [i for i, a in enumerate(call_node.args) if isinstance(a, Node) and a.op == "get_attr"]


def device_graph_compiler(module: torch.nn.Module, example_inputs, target, *, runner_cls=None, **config_dict: Dict) -> torch.nn.Module:
    from torch.fx.passes.infra.partitioner import CapabilityBasedPartitioner

    if runner_cls is None:
        from ..device_graph_runner import HIPGraphRunner

        runner_cls = HIPGraphRunner
    total = sum(1 for n in module.graph.nodes if n.op in _CALLABLE)
    partitioner = CapabilityBasedPartitioner(module, DeviceGraphOperatorSupport(target), allows_single_node_partition=True)
    partitions = partitioner.propose_partitions()
    inside = sum(len(p.nodes) for p in partitions)
    fused = partitioner.fuse_partitions(partitions)

    regions = 0
    for node in list(fused.graph.nodes):
        if node.op != "call_module":
            continue
        region = fused.get_submodule(node.target)
        if not isinstance(region, torch.fx.GraphModule) or not node.target.startswith("fused_"):
            continue  # a replacement module of the target that stayed outside every region
        lazy = _LazyXPUGraph(
            region,
            runner_cls,
            owned_positions=_owned_positions(fused, node),
            memory_pool=config_dict.get("memory_pool", None),
            clone_args=config_dict.get("clone_args", True),
            clone_outputs=config_dict.get("clone_outputs", False),
            max_graphs=config_dict.get("max_graphs", 8),
        )
        setattr(fused, node.target, lazy)
        regions += 1
    logger.info(f"device graph: {inside} of {total} calls recorded in {regions} region(s)")
    return fused
