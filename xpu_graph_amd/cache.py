"""Compile-artifact cache: a rewritten GraphModule is stored under a key made of the incoming graph, its
(fake) inputs, the configuration and the stage, and loaded instead of running the pass pipeline again.

Public surface and behaviour follow the reference (src/xpu_graph/cache.py:40-335): `SerializableArtifact`
wraps the callable and pickles through `convert_to_bytes` / `rebuild_from_bytes`; `XpuGraphCache` is the
do-nothing base, `XpuGraphLocalCache(path)` keeps one `xpugraph_<key>.pt` per artifact, `save_artifact`
returns the RE-LOADED artifact (so that what runs is what a later process would load), `no_cache()` /
`default_cache()` are the factories.  The artifact of this backend is always an FX GraphModule whose
call_function targets are Aten / xpu_ops overloads or importable Python callables, so only that case exists.

The graph is stored as plain data: one record per node (name, opcode, target reference, arguments with node
references replaced by names) next to the module's own state (parameters, buffers, submodules -- the target's
replacement modules pickle by class reference).  Cache files are written and read by this package only.
"""
import hashlib
import importlib
import io
import os
import pickle
from abc import ABC, abstractmethod
from contextlib import contextmanager, nullcontext
from os import PathLike
from typing import Union

import torch
from torch import fx
from torch.fx.node import map_aggregate

from .config import XpuGraphConfig, get_cache_dir
from .fx_utils import FxStage
from .utils import logger

__all__ = ["SerializableArtifact", "SerializableGraphModule", "XpuGraphCache", "XpuGraphLocalCache", "no_cache", "default_cache"]

_FORMAT = 1


class _NodeRef:
    """Stands for an fx.Node inside stored arguments."""

    __slots__ = ("name",)

    def __init__(self, name):
        self.name = name

    def __reduce__(self):
        return (_NodeRef, (self.name,))


def _target_ref(node):
    """A picklable description of node.target that `_resolve_target` turns back into the object."""
    t = node.target
    if node.op != "call_function":
        return ("name", t)
    if isinstance(t, torch._ops.OpOverload):
        ns, op = t._schema.name.split("::")
        return ("op", ns, op, t._overloadname or "default")
    if isinstance(t, torch._ops.OpOverloadPacket):
        ns, op = t._qualified_op_name.split("::")
        return ("packet", ns, op)
    mod, qual = getattr(t, "__module__", None), getattr(t, "__qualname__", None)
    if mod is None or qual is None or "<locals>" in qual:
        raise NotImplementedError(f"call_function target {t!r} cannot be stored by reference")
    return ("py", mod, qual)


def _resolve_target(ref):
    kind = ref[0]
    if kind == "name":
        return ref[1]
    if kind in ("op", "packet"):
        ns = ref[1]
        if ns == "xpu_ops":
            from . import ops as _register_ops  # noqa: F401  (defines torch.ops.xpu_ops)
        packet = getattr(getattr(torch.ops, ns), ref[2])
        return packet if kind == "packet" else getattr(packet, ref[3])
    if kind == "py":
        obj = importlib.import_module(ref[1])
        for part in ref[2].split("."):
            obj = getattr(obj, part)
        if not callable(obj):
            raise NotImplementedError(f"stored target {ref[1]}.{ref[2]} is not callable")
        return obj
    raise NotImplementedError(f"unknown target reference {ref!r}")


def graph_module_to_data(gm: fx.GraphModule):
    """(module state, node records): everything needed to rebuild `gm`, with no code object in it."""
    state = {k: v for k, v in gm.__dict__.items() if k not in ("_graph", "_code", "_lineno_map", "_prologue_start")}
    state = dict(state)
    mods = dict(state.get("_modules", {}))
    for k, v in mods.items():
        if isinstance(v, fx.GraphModule):
            mods[k] = ("__graph_module__",) + graph_module_to_data(v)
    state["_modules"] = mods
    wrap = lambda a: _NodeRef(a.name) if isinstance(a, fx.Node) else a  # noqa: E731
    records = []
    for n in gm.graph.nodes:
        records.append((n.name, n.op, _target_ref(n), map_aggregate(n.args, wrap), map_aggregate(n.kwargs, wrap), n.type))
    return state, records


def graph_module_from_data(state, records):
    state = dict(state)
    mods = dict(state.get("_modules", {}))
    for k, v in mods.items():
        if isinstance(v, tuple) and v and v[0] == "__graph_module__":
            mods[k] = graph_module_from_data(v[1], v[2])
    state["_modules"] = mods
    root = torch.nn.Module()
    root.__dict__.update(state)
    graph = fx.Graph()
    by_name = {}
    unwrap = lambda a: by_name[a.name] if isinstance(a, _NodeRef) else a  # noqa: E731
    for name, op, tref, args, kwargs, typ in records:
        if op == "output":
            node = graph.output(map_aggregate(args, unwrap)[0], typ)
        else:
            node = graph.create_node(op, _resolve_target(tref), map_aggregate(args, unwrap), map_aggregate(kwargs, unwrap), name, typ)
        by_name[name] = node
    gm = fx.GraphModule(root, graph)
    # GraphModule copies only the attributes the graph refers to; bring the rest of the stored state along
    for k, v in state.items():
        if k not in ("_modules", "_parameters", "_buffers") and k not in gm.__dict__:
            gm.__dict__[k] = v
    return gm


@contextmanager
def _outside_tracing():
    """Loading must produce REAL tensors (parameters, tables), whatever tracing context the compile runs in."""
    from torch._guards import TracingContext
    from torch.utils._python_dispatch import _disable_current_modes

    with _disable_current_modes():
        ctx = TracingContext.try_get()
        with ctx.patch(fake_mode=None) if ctx is not None else nullcontext():
            yield


class SerializableArtifact(ABC):
    def __new__(cls, artifact):
        # wrapping a wrapper is the identity (reference cache.py:54-58)
        if isinstance(artifact, SerializableArtifact):
            return artifact
        return super().__new__(cls)

    def __init__(self, artifact):
        if isinstance(artifact, SerializableArtifact):
            return
        assert callable(artifact), f"artifact must be callable, but got {type(artifact)}"
        self._artifact = artifact
        if getattr(artifact, "_boxed_call", False):
            self._boxed_call = True

    def __call__(self, *args, **kwargs):
        return self._artifact(*args, **kwargs)

    @property
    def artifact(self):
        return self._artifact

    def __reduce__(self):
        return self.rebuild_from_bytes, (self.convert_to_bytes(),)

    @abstractmethod
    def convert_to_bytes(self) -> bytes: ...

    @staticmethod
    @abstractmethod
    def rebuild_from_bytes(byte_s: bytes): ...


class SerializableGraphModule(SerializableArtifact):
    def __init__(self, artifact):
        if isinstance(artifact, SerializableArtifact):
            return
        assert isinstance(artifact, fx.GraphModule)
        super().__init__(artifact)

    def convert_to_bytes(self) -> bytes:
        with _outside_tracing():
            state, records = graph_module_to_data(self._artifact)
            buf = io.BytesIO()
            pickle.dump((_FORMAT, state, records), buf)
            return buf.getvalue()

    @staticmethod
    def rebuild_from_bytes(byte_s: bytes):
        with _outside_tracing():
            fmt, state, records = pickle.loads(byte_s)
            if fmt != _FORMAT:
                raise NotImplementedError(f"cache artifact format {fmt}, this package reads {_FORMAT}")
            return SerializableGraphModule(graph_module_from_data(state, records))


class XpuGraphCache:
    """The base cache stores nothing."""

    def cache_key(self, gm: fx.GraphModule, fake_inputs, config: XpuGraphConfig, stage: FxStage):
        from . import __version__ as pkg_version

        text = gm.print_readable(print_output=False, include_stride=True, include_device=True)
        key = f"{text}-{fake_inputs}-{config}-{stage}-{pkg_version}"
        logger.debug(f"Cache Key readable: \n{key}")
        digest = hashlib.md5(key.encode()).hexdigest()
        logger.info(f"Cache Key: {digest}")
        return digest

    def save_artifact(self, key, value, expire=None):
        return value

    def load_artifact(self, key):
        return None

    def delete_artifact(self, key):
        return None

    def _set_cache_ctx(self):
        return None

    def _restore_cache_ctx(self, orig_ctx):
        pass


class XpuGraphLocalCache(XpuGraphCache):
    def __init__(self, cache_path: Union[str, PathLike]):
        super().__init__()
        cache_path = os.path.abspath(cache_path)
        os.makedirs(cache_path, exist_ok=True)
        self._path = cache_path

    def _artifact_path(self, key):
        return os.path.join(self._path, f"xpugraph_{key}.pt")

    def save_artifact(self, key, value, expire=None):
        assert isinstance(value, SerializableArtifact)
        path = self._artifact_path(key)
        logger.info(f"Save cache in location: {path}")
        tmp = f"{path}.{os.getpid()}.tmp"
        with open(tmp, "wb") as f:
            pickle.dump(value, f)
        os.replace(tmp, path)  # readers never see a half-written file
        with open(path, "rb") as f:
            return pickle.load(f)

    def load_artifact(self, key):
        path = self._artifact_path(key)
        if not os.path.isfile(path):
            return None
        logger.info(f"Use cache in location: {path}")
        with open(path, "rb") as f:
            return pickle.load(f)

    def delete_artifact(self, key):
        path = self._artifact_path(key)
        if os.path.isfile(path):
            os.remove(path)


def no_cache():
    return XpuGraphCache()


def default_cache():
    return XpuGraphLocalCache(get_cache_dir())
