"""cat([..., x[:, a0:b0, :].sum(1), x[:, a1:b1, :].sum(1), x[:, a2:b2, :].sum(1), ...], -1) -> one kernel.

The reference's MLU pattern (targets/mlu/fuse_sum_cat.py:118-252, FusedCatSum / SliceSumCatOperation): sums over
dim 1 (no keepdim) of row slices of ONE 3-D tensor, each sum and each slice used once, at least three of them in a
row among the inputs of a cat along the last dim; literal integer bounds.  The run is replaced by a module call
that yields [batch, n * cols]; other cat inputs stay.  Where the reference still requires every slice to start at
row 0, any start is taken here (the kernel sums each slice on its own).
"""
import torch
from torch import fx, nn

from .....config import OptLevel
from ...pattern import Pattern
from ...utils.node_utils import aten, cat_axis, fresh_submodule_name, has_val, is_call, rank

INT64_MAX = 9223372036854775807
NAME = "mi355x_slice_sum_cat"
_DTYPES = (torch.float32, torch.bfloat16, torch.float16)
_MAX = 64


class SliceSumCatModule(nn.Module):
    def __init__(self, slice_param):
        super().__init__()
        self.slice_param = [(int(a), int(b)) for a, b in slice_param]

    def forward(self, x):
        return torch.ops.xpu_ops.slice_sum_cat(x, [a for a, _ in self.slice_param], [b for _, b in self.slice_param])


def _slice_sum(node):
    """(source, start, end) when node is sum(slice(source3d, 1, start, end), [1]) with single-use links, else None."""
    if not is_call(node, aten.sum.dim_IntList) or not has_val(node) or rank(node) != 2:
        return None
    if len(node.args) != 2 or list(node.args[1]) != [1] or node.kwargs or len(node.users) != 1:
        return None
    sl = node.args[0]
    if not is_call(sl, aten.slice.Tensor) or len(sl.users) != 1 or len(sl.args) < 2 or sl.args[1] != 1:
        return None
    if len(sl.args) > 4 and sl.args[4] != 1:
        return None
    src = sl.args[0]
    if not isinstance(src, fx.Node) or not has_val(src) or rank(src) != 3:
        return None
    val = src.meta["val"]
    rows = val.shape[1]
    if val.dtype not in _DTYPES or not isinstance(rows, int):
        return None
    start = sl.args[2] if len(sl.args) > 2 else None
    end = sl.args[3] if len(sl.args) > 3 else None
    start = 0 if start is None else start
    end = rows if end is None or end == INT64_MAX else end
    if not isinstance(start, int) or not isinstance(end, int):
        return None
    if start < 0:
        start += rows
    if end < 0:
        end += rows
    end = min(end, rows)
    if not (0 <= start <= end):
        return None
    return src, start, end


class FusedCatSum(Pattern):
    _opt_level = OptLevel.level2

    def process(self, gm):
        g = gm.graph
        changed = False
        for node in list(g.nodes):
            axis = cat_axis(node)
            if axis is None or not has_val(node) or rank(node) != 2 or axis not in (1, -1):
                continue
            pieces = list(node.args[0])
            infos = [_slice_sum(p) if isinstance(p, fx.Node) else None for p in pieces]
            # first run of >= 3 consecutive slice-sums of one source
            best = None
            i = 0
            while i < len(pieces) and best is None:
                if infos[i] is None:
                    i += 1
                    continue
                j = i
                while j + 1 < len(pieces) and infos[j + 1] is not None and infos[j + 1][0] is infos[i][0] and j + 1 - i < _MAX:
                    j += 1
                if j - i >= 2:
                    best = (i, j)
                i = j + 1
            if best is None:
                continue
            lo, hi = best
            src = infos[lo][0]
            params = [(a, b) for _, a, b in infos[lo : hi + 1]]
            name = fresh_submodule_name(gm, NAME)
            gm.add_submodule(name, SliceSumCatModule(params))
            with g.inserting_before(node):
                fused = g.call_module(name, args=(src,))
                rest = pieces[:lo] + [fused] + pieces[hi + 1 :]
                new_cat = g.call_function(aten.cat.default, (rest, -1)) if len(rest) > 1 else fused
            node.replace_all_uses_with(new_cat)
            g.erase_node(node)
            for p in pieces[lo : hi + 1]:
                if len(p.users) == 0:
                    sl = p.args[0]
                    g.erase_node(p)
                    if len(sl.users) == 0:
                        g.erase_node(sl)
            changed = True
        return changed
