"""Record a compiled callable into a HIP graph once and replay it.

Interface of the reference's GraphRunner (src/xpu_graph/device_graph_runner.py:11-141):
construct with the callable and two callbacks (which tensors are the static input
buffers; how to refresh them from new arguments), `capture(*args)` once, then call
the runner like the original function.  Every kernel behind `torch.ops.xpu_ops`
only enqueues work on the current stream (no allocation, no synchronisation, no
memset), so a compiled mi355x graph records as it is; the outputs of a replay live
in the graph's private memory pool and are overwritten by the next replay.
"""
from typing import Callable, Dict, List, Tuple

import torch
import torch.utils._pytree as pytree


_RUNNERS = {}  # target name -> runner class


class GraphRunner(torch.nn.Module):
    def __init__(
        self,
        callable_target: Callable,
        init_param_callback: Callable[[Tuple, Dict], List[torch.Tensor]] = None,
        copy_param_callback: Callable[[List[torch.Tensor], Tuple, Dict], bool] = None,
    ):
        super().__init__()
        self._callable_target = callable_target
        self._init_param_callback = init_param_callback or _tensors_of
        self._copy_param_callback = copy_param_callback or _copy_tensors
        self._stream = None
        self._graph = None
        self._input_buffers = None
        self._output = None
        self._mempool = None

    @property
    def mempool(self):
        return self._mempool

    def __class_getitem__(cls, target):
        """`GraphRunner[Target.mi355x]` is the runner class of that target (reference utils.py:252-256); a target
        with no runner of its own gets the class itself."""
        return _RUNNERS.get(getattr(target, "value", target), cls)

    def clone(self):
        return type(self)(self._callable_target, self._init_param_callback, self._copy_param_callback)

    def reset(self):
        self.__init__(self._callable_target, self._init_param_callback, self._copy_param_callback)
        return self


def _tensors_of(*args, **kwargs):
    """Default: every tensor argument is a static input buffer, in flattening order."""
    return [a for a in pytree.tree_leaves((args, kwargs)) if isinstance(a, torch.Tensor)]


def _copy_tensors(buffers, *args, **kwargs):
    new = [a for a in pytree.tree_leaves((args, kwargs)) if isinstance(a, torch.Tensor)]
    if len(new) != len(buffers):
        return False
    for dst, src in zip(buffers, new):
        if dst.shape != src.shape or dst.dtype != src.dtype:
            return False
        if dst.data_ptr() != src.data_ptr():
            dst.copy_(src)
    return True


class HIPGraphRunner(GraphRunner):
    """GraphRunner over torch.cuda.CUDAGraph, which is a hipGraph on ROCm."""

    def capture(self, *args, memory_pool=None, clone_args=False, warmup=2, **kwargs) -> None:
        assert self._graph is None, "Device graph has been recorded."
        if clone_args:
            args, kwargs = pytree.tree_map(lambda x: x.detach().clone() if isinstance(x, torch.Tensor) else x, (args, kwargs))
        self._input_buffers = self._init_param_callback(*args, **kwargs)
        assert self._input_buffers is not None
        self._stream = torch.cuda.Stream()  # default priority
        self._graph = torch.cuda.CUDAGraph()
        self._mempool = memory_pool if memory_pool else torch.cuda.graph_pool_handle()
        # run a few times outside the capture: lazy one-time work (function attributes, compile caches, allocator
        # growth) must not happen while the stream is recording
        self._stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self._stream), torch.no_grad():
            for _ in range(warmup):
                self._callable_target(*args, **kwargs)
        torch.cuda.current_stream().wait_stream(self._stream)
        torch.cuda.synchronize()
        with torch.cuda.graph(self._graph, stream=self._stream, pool=self._mempool), torch.no_grad():
            self._output = self._callable_target(*args, **kwargs)

    def forward(self, *args, **kwargs):
        if self._graph is None:
            raise RuntimeError("capture() first")
        # the refresh of the recorded input buffers is work, not a check: it must also happen under `python -O`
        if not self._copy_param_callback(self._input_buffers, *args, **kwargs):
            raise RuntimeError("arguments do not fit the recorded buffers")
        self._graph.replay()
        return self._output


_RUNNERS["mi355x"] = HIPGraphRunner
