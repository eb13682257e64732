"""Rotary position embedding in the rotate-half convention -> one kernel.

    x * cos + cat([-x[..., D/2:], x[..., :D/2]], -1) * sin        -> rope(x, cos, sin)

x is a [B, H, S, D] tensor (usually the transposed view of a projection's
[B, S, H, D] output: the kernel takes strides and writes in the same layout,
so no copy is made), cos / sin are [S, D] tables in x's dtype, possibly with
leading dimensions of size 1, or one row [D] shared by every position (a
decode step's).  The reference has no rotary pattern; unfused,
the subgraph is seven elementwise / copy kernels per tensor in the Llama block
of benchmark config 5.
"""
import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern, PatternGroup
from ...utils.node_utils import aten, cat_axis, is_call
from .swiglu import _last_dim_slice

ROPE_NAME = "mi355x_rope"
_DTYPES = (torch.bfloat16, torch.float16)


class RoPEModule(nn.Module):
    def forward(self, x, cos, sin):
        return torch.ops.xpu_ops.rope(x, cos, sin)


def _val(node):
    v = node.meta.get("val") if isinstance(node, fx.Node) else None
    return v if isinstance(v, torch.Tensor) else None


def _is_table(node, x_val):
    """[S, D] in x's dtype, possibly with leading dimensions of size 1 -- or a single row ([D], [1, D]) that every
    position shares, which is what a decode step passes for its one position."""
    v = _val(node)
    if v is None or v.dtype != x_val.dtype or v.dim() < 1:
        return False
    shape = list(v.shape)
    if not all(isinstance(d, int) for d in shape) or shape[-1] != x_val.shape[-1]:
        return False
    rows_ok = v.dim() == 1 or shape[-2] in (1, x_val.shape[-2])
    return rows_ok and all(d == 1 for d in shape[:-2])


def _rotate_half_source(node):
    """x when node is cat([neg(x[..., h:]), x[..., :h]], last dim) with h = D / 2, else None."""
    if cat_axis(node) is None:
        return None
    pieces = node.args[0]
    v = _val(node)
    if v is None or len(pieces) != 2 or cat_axis(node) not in (-1, v.dim() - 1):
        return None
    neg, lo = pieces
    if not is_call(neg, aten.neg.default):
        return None
    hi_s, lo_s = _last_dim_slice(neg.args[0]), _last_dim_slice(lo)
    if hi_s is None or lo_s is None or hi_s[0] is not lo_s[0]:
        return None
    x = hi_s[0]
    d = _val(x).shape[-1] if _val(x) is not None else None
    if not isinstance(d, int) or d % 2 != 0:
        return None
    if (hi_s[1], hi_s[2]) != (d // 2, d) or (lo_s[1], lo_s[2]) != (0, d // 2):
        return None
    return x


def match_rope(add):
    """(x, cos, sin) when `add` is x * cos + rotate_half(x) * sin, else None."""
    if not is_call(add, aten.add.Tensor) or len(add.args) != 2 or add.kwargs.get("alpha", 1) != 1:
        return None
    for direct, rotated in ((add.args[0], add.args[1]), (add.args[1], add.args[0])):
        if not (is_call(direct, aten.mul.Tensor) and is_call(rotated, aten.mul.Tensor)):
            continue
        for rot, sin in ((rotated.args[0], rotated.args[1]), (rotated.args[1], rotated.args[0])):
            x = _rotate_half_source(rot) if isinstance(rot, fx.Node) else None
            if x is None:
                continue
            xv = _val(x)
            if xv is None or xv.dim() != 4 or xv.dtype not in _DTYPES or not isinstance(xv.shape[-1], int) or xv.shape[-1] % 16 != 0:
                continue
            for x2, cos in ((direct.args[0], direct.args[1]), (direct.args[1], direct.args[0])):
                if x2 is x and _is_table(cos, xv) and _is_table(sin, xv):
                    out = _val(add)
                    if out is not None and out.dtype == xv.dtype and tuple(out.shape) == tuple(xv.shape):
                        return x, cos, sin
    return None


class FusedRoPE(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP1
    _support_stages = [FxStage.inference, FxStage.pregrad]  # rope carries a backward formula

    def process(self, gm):
        changed = False
        for node in list(gm.graph.nodes):
            m = match_rope(node)
            if m is None:
                continue
            if not hasattr(gm, ROPE_NAME):
                gm.add_submodule(ROPE_NAME, RoPEModule())
            with gm.graph.inserting_before(node):
                new = gm.graph.call_module(ROPE_NAME, args=m)
            node.replace_all_uses_with(new)
            gm.graph.erase_node(node)
            changed = True
        return changed
