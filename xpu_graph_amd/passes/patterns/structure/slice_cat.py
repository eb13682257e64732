"""Column-slice gathers.

    FusedCatSlice          cat([..., x[:, a:b], x[:, c:d], ...], 1) -> fuse_slice_cat(x, [(a,b),(c,d)])
    FusedMultipleSliceCat  several fuse_slice_cat on one source     -> one multi-output module
    FusedSliceStackSum     stack(slices) [+ sum(0)]                 -> fuse_slice_cat + reshape [+ sum(1)]

Behaviour of the reference's structure/fuse_slice_cat.py:30-116,
fuse_multiple_slice_cat.py:11-105 and fuse_slice_stack.py:32-151: 2-D tensors
only, slices literally along dim 1, the longest consecutive run of slice
inputs of one cat/stack, at least two slices, `end` may be INT64_MAX or
negative.
"""
import operator

import torch
from torch import fx, nn

from ....config import OptLevel
from ..pattern import Pattern
from ..utils.node_utils import aten, cat_axis, fresh_submodule_name, has_val, is_call, longest_run, rank
from ....fx_utils import outside_fake_mode

INT64_MAX = 9223372036854775807
SLICE_CAT_NAME = "fuse_slice_cat"
SLICE_CAT_V2 = "fuse_slice_cat_v2"


def _is_2d_slice(n):
    return is_call(n, aten.slice.Tensor) and has_val(n) and rank(n) == 2


def slice_run_params(nodes):
    """(source, [(start, end), ...]) when `nodes` are >= 2 dim-1 slices of one source, else None."""
    if len(nodes) < 2:
        return None
    src = nodes[0].args[0]
    width = src.meta["val"].shape[-1]
    if not isinstance(width, int):
        return None  # a symbolic width: the column table cannot be built at compile time
    params = []
    for n in nodes:
        if n.args[0] is not src or len(n.args) < 4 or n.args[1] != 1:
            return None
        if len(n.args) > 4 and n.args[4] != 1:
            return None
        start, end = n.args[2], n.args[3]
        start = 0 if start is None else start
        if not isinstance(start, int) or not isinstance(end, (int, type(None))):
            return None
        if end is None or end == INT64_MAX:
            end = width
        elif end < 0:
            end = width + end
        if start < 0:
            start = width + start
        # eager slicing clamps bounds to the source (x[:, 5:10000] is x[:, 5:]; an empty range stays empty)
        start = max(0, min(start, width))
        end = max(start, min(end, width))
        params.append((start, end))
    return src, params


def _drop_dead(graph, nodes):
    for n in nodes:
        if isinstance(n, fx.Node) and len(n.users) == 0:
            graph.erase_node(n)


class FusedCatSlice(Pattern):
    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def process(self, gm):
        if not hasattr(gm, SLICE_CAT_NAME):
            gm.add_submodule(SLICE_CAT_NAME, self.target_mod())
        g = gm.graph
        changed = False
        for node in reversed(g.nodes):
            axis = cat_axis(node)
            if axis is None or axis == 0 or not has_val(node) or rank(node) != 2:
                continue
            pieces = list(node.args[0])
            lo, hi = longest_run(pieces, _is_2d_slice)
            m = slice_run_params(pieces[lo : hi + 1]) if lo >= 0 else None
            if m is None:
                continue
            src, params = m
            with g.inserting_before(node):
                fused = g.call_module(SLICE_CAT_NAME, args=(src, params))
                new_cat = g.create_node(
                    "call_function", aten.cat.default, (pieces[:lo] + [fused] + pieces[hi + 1 :], -1), name=node.name + "_replacement"
                )
            node.replace_all_uses_with(new_cat)
            g.erase_node(node)
            _drop_dead(g, pieces)
            changed = True
        return changed


class FusedMultipleSliceCat(Pattern):
    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def _new_module(self, gm, slice_lists):
        name = fresh_submodule_name(gm, SLICE_CAT_V2)
        with outside_fake_mode():
            gm.add_submodule(name, self.target_mod(slice_lists))
        return name

    def _merge_singles(self, gm):
        g = gm.graph
        by_src = {}
        for n in g.nodes:
            if n.op == "call_module" and n.target == SLICE_CAT_NAME:
                by_src.setdefault(n.args[0], []).append(n)
        changed = False
        for src, nodes in by_src.items():
            if len(nodes) < 2:
                continue
            lists = [n.args[1] for n in nodes]
            with g.inserting_before(nodes[0]):
                multi = g.call_module(self._new_module(gm, lists), args=(src, lists))
            for i, old in enumerate(nodes):
                with g.inserting_before(old):
                    item = g.call_function(operator.getitem, (multi, i))
                old.replace_all_uses_with(item)
                g.erase_node(old)
            changed = True
        return changed

    def _merge_multis(self, gm):
        g = gm.graph
        by_src = {}
        for n in g.nodes:
            if n.op == "call_module" and isinstance(n.target, str) and n.target.startswith(SLICE_CAT_V2):
                by_src.setdefault(n.args[0], []).append(n)
        changed = False
        for src, nodes in by_src.items():
            if len(nodes) < 2:
                continue
            lists, items = [], []
            for n in nodes:
                lists += list(n.args[1])
                got = sorted((u for u in n.users if is_call(u, operator.getitem)), key=lambda u: u.args[1])
                # every output position must map to the merged table, used or not
                base = len(lists) - len(n.args[1])
                items += [(u, base + u.args[1]) for u in got]
            with g.inserting_before(nodes[0]):
                multi = g.call_module(self._new_module(gm, lists), args=(src, lists))
            for old_item, idx in items:
                with g.inserting_after(multi):
                    new_item = g.call_function(operator.getitem, (multi, idx))
                old_item.replace_all_uses_with(new_item)
            changed = True
        return changed

    def process(self, gm):
        changed = self._merge_singles(gm)
        changed = self._merge_multis(gm) or changed
        return changed


class _StackPieces(nn.Module):
    """cat of 3-D pieces along dim 0; 2-D pieces count as one slab."""

    def forward(self, pieces, axis=0):
        return torch.cat([p if p.dim() == 3 else p.unsqueeze(0) for p in pieces], dim=0)


class FusedSliceStackSum(Pattern):
    _opt_level = OptLevel.level2

    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    @staticmethod
    def _retarget_sum(gm, stack):
        """stack feeding only sum(dim 0): rewrite that sum to dim 1 of the [rows, n, w] layout."""
        if len(stack.users) != 1:
            return False
        s = next(iter(stack.users))
        if not is_call(s, aten.sum.dim_IntList) or s.args[1] != [0] or len(s.args) > 2:
            return False
        with gm.graph.inserting_before(s):
            new = gm.graph.call_function(aten.sum.dim_IntList, (s.args[0], [1]))
        s.replace_all_uses_with(new)
        gm.graph.erase_node(s)
        return True

    def process(self, gm):
        if not hasattr(gm, SLICE_CAT_NAME):
            gm.add_submodule(SLICE_CAT_NAME, self.target_mod())
        if not hasattr(gm, "reshape_cat_module"):
            gm.add_submodule("reshape_cat_module", _StackPieces())
        g = gm.graph
        changed = False
        for node in reversed(g.nodes):
            if not is_call(node, aten.stack.default):
                continue
            if len(node.args) > 1 and node.args[1] != 0:
                continue
            pieces = list(node.args[0])
            lo, hi = longest_run(pieces, _is_2d_slice)
            m = slice_run_params(pieces[lo : hi + 1]) if lo >= 0 else None
            if m is None:
                continue
            src, params = m
            if len({e - s for s, e in params}) != 1:
                continue  # stack needs equal widths; unequal ones would have failed in eager too
            with g.inserting_before(node):
                fused = g.call_module(SLICE_CAT_NAME, args=(src, params))
                rows = g.call_method("size", args=(fused, 0))
                slab = g.call_function(aten.reshape.default, (fused, (rows, len(params), -1)))
                whole = lo == 0 and hi + 1 == len(pieces)
                if not (whole and self._retarget_sum(gm, node)):
                    slab = g.call_function(aten.transpose.int, (slab, 0, 1))
                new_in = pieces[:lo] + [slab] + pieces[hi + 1 :]
                if len(new_in) == 1:
                    out = g.create_node("call_function", aten.cat.default, (new_in, 0), name=node.name + "_replacement")
                else:
                    out = g.call_module("reshape_cat_module", args=(new_in, -1))
            node.replace_all_uses_with(out)
            g.erase_node(node)
            _drop_dead(g, pieces)
            changed = True
        return changed
