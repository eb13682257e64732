"""Many equally wide slices of one tensor along its last dim -> one gather.

    FusedSlice   a = x[..., s0:s0+w]; b = x[..., s1:s1+w]; c = ... (>= 3 of one width, each used by something other
                 than the graph output)  ->  g = fused_slice(x, w) : [n, *x.shape[:-1], w];  a = g[0]; b = g[1]; ...

Behaviour of the reference's structure/fuse_slice.py:30-121: only slices with literal integer bounds along the last
dim, grouped per source and per width, at least three per group; a slice that only feeds the graph output is left
alone (it is a view, the gather would be a copy).  Unlike the reference, bounds are normalised first (negative or
open ends), a slice with a step is skipped, and the slabs are taken with aten.select, which later passes understand.
"""
import torch
from torch import fx

from ..pattern import Pattern, PatternGroup
from ..utils.node_utils import aten, fresh_submodule_name, has_val, is_call
from ....fx_utils import outside_fake_mode

INT64_MAX = 9223372036854775807
FUSED_SLICE_NAME = "fused_slice"


def last_dim_slice(node):
    """(source, start, end) of a unit-step slice along the last dim with literal bounds inside the source, else None."""
    if not is_call(node, aten.slice.Tensor) or not has_val(node) or len(node.args) < 2:
        return None
    src = node.args[0]
    if not isinstance(src, fx.Node) or not has_val(src):
        return None
    shape = src.meta["val"].shape
    if len(shape) < 2 or not isinstance(shape[-1], int):
        return None
    dim = node.args[1]
    if not isinstance(dim, int) or dim not in (-1, len(shape) - 1):
        return None
    if len(node.args) > 4 and node.args[4] != 1:
        return None
    width = shape[-1]
    start = node.args[2] if len(node.args) > 2 else None
    end = node.args[3] if len(node.args) > 3 else None
    start = 0 if start is None else start
    end = width if end is None or end == INT64_MAX else end
    if not isinstance(start, int) or not isinstance(end, int):
        return None
    if start < 0:
        start += width
    if end < 0:
        end += width
    end = min(end, width)
    if not (0 <= start < end):
        return None
    return src, start, end


class FusedSlice(Pattern):
    _pattern_group = PatternGroup.GROUP1

    def __init__(self, target_mod: torch.nn.Module):
        super().__init__()
        self.target_mod = target_mod

    def process(self, gm):
        g = gm.graph
        groups = {}  # (source, width) -> [(slice node, start)]
        for node in g.nodes:
            m = last_dim_slice(node)
            if m is None:
                continue
            users = list(node.users)
            if len(users) == 0 or (len(users) == 1 and users[0].op == "output"):
                continue
            src, start, end = m
            groups.setdefault((src, end - start), []).append((node, start))
        changed = False
        for (src, width), members in groups.items():
            if len(members) < 3:
                continue
            starts = [s for _, s in members]
            first = members[0][0]
            name = fresh_submodule_name(gm, FUSED_SLICE_NAME)
            with outside_fake_mode():
                gm.add_submodule(name, self.target_mod(starts))
            with g.inserting_before(first):
                fused = g.call_module(name, args=(src, width))
                slabs = [g.call_function(aten.select.int, (fused, 0, i)) for i in range(len(members))]
            for (node, _), slab in zip(members, slabs):
                node.replace_all_uses_with(slab)
                g.erase_node(node)
            changed = True
        return changed
