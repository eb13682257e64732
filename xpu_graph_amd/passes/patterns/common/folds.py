"""Level-1 canonicalisers the fusion matchers rely on: no-op expand / view
removal, view-of-view merging, one-input cat -> clone, removal of clones and
same-dtype copies that do not feed graph outputs.

Behaviour of the reference's fold_expand.py:9-33, fold_view.py:9-112,
fold_cat.py:9-70, fold_clone.py:9-42 and fold_to_copy.py:9-59.
"""
import torch
import torch.fx as fx
from torch.multiprocessing.reductions import StorageWeakRef

from ....fx_utils import FxStage
from ..pattern import Pattern, PatternGroup
from ..utils.node_utils import VIEW_OPS, aten, cat_axis, is_call, is_getitem, same_shape

_ALL = [FxStage.inference, FxStage.pregrad, FxStage.forward, FxStage.backward]
_SHAPE_ONLY_OPS = VIEW_OPS + (aten.squeeze.default, aten.squeeze.dim, aten.squeeze.dims, aten.unsqueeze.default)


def _storage_key(node):
    v = node.meta.get("val")
    if isinstance(v, torch.Tensor) and v.layout == torch.strided:
        try:
            return StorageWeakRef(v.untyped_storage())
        except Exception:
            return None
    return None


def _same_storage(a, b):
    """Keys of _storage_key; a node without storage (a size-valued placeholder of a dynamic graph) shares none."""
    return a is not None and b is not None and a == b


def _output_storages(gm):
    out = list(gm.graph.nodes)[-1]
    assert out.op == "output"
    keys = {_storage_key(n) for n in out.all_input_nodes}
    keys.discard(None)
    return keys


class FoldExpand(Pattern):
    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, aten.expand.default)]:
            src = n.args[0]
            if same_shape(n.meta["val"].shape, src.meta["val"].shape):
                n.replace_all_uses_with(src)
                gm.graph.erase_node(n)
                changed = True
        return changed


class FoldView0(Pattern):
    """view/reshape to the shape the input already has."""

    _support_stages = _ALL

    def process(self, gm):
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, *VIEW_OPS)]:
            src = n.args[0]
            if same_shape(n.meta["val"].shape, src.meta["val"].shape):
                n.replace_all_uses_with(src)
                gm.graph.erase_node(n)
                changed = True
        return changed


class FoldView1(Pattern):
    """reshape(reshape(x)) -> reshape(x); reshape(squeeze/unsqueeze(x)) -> reshape(x)."""

    _support_stages = [FxStage.inference, FxStage.pregrad, FxStage.forward]

    @staticmethod
    def _merged_shape(inner, outer):
        def neg(shape):
            return any(isinstance(d, int) and d < 0 for d in shape)

        if neg(inner) or not neg(outer):
            return outer
        # the inner shape was fully specified (it asserts the element count), the outer one
        # has a -1: resolve it from the inner shape so the assertion is not lost

        def split(shape):
            syms, prod = [], 1
            for d in shape:
                if isinstance(d, fx.Node):
                    syms.append(d)
                elif d > 0:
                    prod *= d
            return sorted(syms), prod

        isym, iprod = split(inner)
        osym, oprod = split(outer)
        if isym == osym:
            fill = iprod // oprod
        elif iprod == oprod:
            fill = next((a for a, b in zip(isym, osym + [None]) if a != b), None)
            if fill is None:
                return None
        else:
            return None
        return tuple(fill if d == -1 else d for d in outer)

    def process(self, gm):
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, *VIEW_OPS)]:
            src = n.args[0]
            if not is_call(src, *_SHAPE_ONLY_OPS):
                continue
            if src.target in VIEW_OPS:
                merged = self._merged_shape(src.args[1], n.args[1])
                if merged is not None:
                    n.args = (src.args[0], merged)
                    changed = True
            else:
                n.replace_input_with(src, src.args[0])
                changed = True
        return changed


class FoldCat(Pattern):
    """cat([x]) -> clone(x); cat(split_with_sizes(x, dim) pieces in order, same dim) -> clone(x)."""

    _support_stages = _ALL

    @staticmethod
    def _whole_split_source(pieces):
        src = None
        for i, p in enumerate(pieces):
            if not (is_getitem(p) and p.args[1] == i):
                return None
            if i == 0:
                if not is_call(p.args[0], aten.split_with_sizes.default):
                    return None
                src = p.args[0]
            elif p.args[0] is not src:
                return None
        if src is not None and len(src.meta["val"]) == len(pieces):
            return src
        return None

    def process(self, gm):
        changed = False
        for cat in reversed([n for n in gm.graph.nodes if cat_axis(n) is not None]):
            pieces = cat.args[0]
            repl_src = None
            if len(pieces) == 1:
                repl_src = pieces[0]
            else:
                split = self._whole_split_source(pieces)
                if split is not None:
                    sdim = split.args[2] if len(split.args) > 2 else split.kwargs.get("dim", 0)
                    cdim = cat_axis(cat)
                    sdim += len(split.args[0].meta["val"].shape) if sdim < 0 else 0
                    cdim += len(cat.meta["val"].shape) if cdim < 0 else 0
                    if sdim == cdim:
                        repl_src = split.args[0]
            if repl_src is None:
                continue
            with gm.graph.inserting_before(cat):
                clone = gm.graph.call_function(aten.clone.default, args=(repl_src,))
            cat.replace_all_uses_with(clone)
            gm.graph.erase_node(cat)
            changed = True
        return changed


class FoldClone(Pattern):
    """clone(x, preserve_format) -> x unless the clone's storage reaches a graph output.

    One case beyond the reference: a clone that IS a graph output is still dropped when x is a contiguous
    intermediate with storage of its own (not an input's, not a parameter's) that reaches no other output;
    nobody can then tell the copy from the original.  This is what is left of cat([fused]) once a whole
    slice/cat group has become a single kernel call, and the copy would double that kernel's memory traffic.
    """

    _support_stages = [FxStage.inference]

    @staticmethod
    def _private_intermediate(gm, clone, out_nodes):
        src = clone.args[0]
        key = _storage_key(src)
        if key is None or src.op not in ("call_module", "call_function"):
            return False
        for n in gm.graph.nodes:
            if n.op in ("placeholder", "get_attr") and _same_storage(_storage_key(n), key):
                return False
        if any(o is not clone and _same_storage(_storage_key(o), key) for o in out_nodes):
            return False
        fmt = clone.kwargs.get("memory_format", torch.preserve_format)
        return fmt in (torch.preserve_format, torch.contiguous_format) and src.meta["val"].is_contiguous()

    def process(self, gm):
        outs = _output_storages(gm)
        out_nodes = list(list(gm.graph.nodes)[-1].all_input_nodes)
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, aten.clone.default)]:
            key = _storage_key(n)
            if key is None:
                continue
            src = n.args[0]
            if not isinstance(src.meta.get("val"), torch.Tensor):
                continue
            if key in outs:
                if n in out_nodes and self._private_intermediate(gm, n, out_nodes):
                    n.replace_all_uses_with(src)
                    gm.graph.erase_node(n)
                    out_nodes = list(list(gm.graph.nodes)[-1].all_input_nodes)
                    changed = True
                continue
            fmt = n.kwargs.get("memory_format", torch.preserve_format)
            # also: a copy into the contiguous format of something that already is contiguous (one case beyond the
            # reference; it is what remains of transpose(1, 2).contiguous() once a kernel writes [B, S, H, D] directly)
            if fmt == torch.preserve_format or (fmt == torch.contiguous_format and src.meta["val"].is_contiguous()):
                n.replace_all_uses_with(src)
                gm.graph.erase_node(n)
                changed = True
        return changed


class FoldToCopy(Pattern):
    """_to_copy that changes neither dtype, device nor layout -> its input."""

    _support_stages = _ALL
    _pattern_group = PatternGroup.GROUP1

    @staticmethod
    def _is_noop(n):
        src = n.args[0]
        a, b = src.meta.get("val"), n.meta.get("val")
        if a is None or b is None or a.dtype != b.dtype or a.device != b.device:
            return False
        if any(k in n.kwargs for k in ("layout", "pin_memory", "non_blocking")):
            return False
        return n.kwargs.get("memory_format", torch.preserve_format) == torch.preserve_format

    def process(self, gm):
        outs = _output_storages(gm)
        changed = False
        for n in [n for n in gm.graph.nodes if is_call(n, aten._to_copy.default)]:
            key = _storage_key(n)
            if key is None or key in outs:
                continue
            if self._is_noop(n):
                n.replace_all_uses_with(n.args[0])
                gm.graph.erase_node(n)
                changed = True
        return changed
