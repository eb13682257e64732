"""silu(gate) * up -> one SwiGLU kernel.

    silu(x[..., :d]) * x[..., d:]   (both halves of one tensor)  -> silu_mul(x)
    silu(a) * b                      (two tensors, same shape)    -> silu_mul2(a, b)

The first form is what the reference's NPU FusedSwiGLU matches
(passes/patterns/targets/npu/fuse_silu_mul.py:21-69); the second is the
Llama MLP with separate gate and up projections.
"""
import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern
from ...utils.node_utils import aten, is_call, same_shape, sole_user_is

_INT64_MAX = 9223372036854775807
_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


class SiluMulHalves(nn.Module):
    def forward(self, x):
        return torch.ops.xpu_ops.silu_mul(x)


class SiluMulPair(nn.Module):
    def forward(self, gate, up):
        return torch.ops.xpu_ops.silu_mul2(gate, up)


def _last_dim_slice(node):
    """(source, start, end) of a step-1 slice along the last dim, else None."""
    if not is_call(node, aten.slice.Tensor) or len(node.args) < 2:
        return None
    src = node.args[0]
    nd = len(src.meta["val"].shape)
    dim = node.args[1]
    if dim not in (-1, nd - 1):
        return None
    width = src.meta["val"].shape[-1]
    if not isinstance(width, int):
        return None
    start = node.args[2] if len(node.args) > 2 and node.args[2] is not None else 0
    end = node.args[3] if len(node.args) > 3 and node.args[3] is not None else width
    step = node.args[4] if len(node.args) > 4 else 1
    if step != 1 or not isinstance(start, int) or not isinstance(end, int):
        return None
    end = width if end == _INT64_MAX else end
    start = start + width if start < 0 else start
    end = end + width if end < 0 else end
    return src, start, min(end, width)


def match_swiglu(mul):
    if not is_call(mul, aten.mul.Tensor):
        return None
    a, b = mul.args[0], mul.args[1]
    if not (isinstance(a, fx.Node) and isinstance(b, fx.Node)):
        return None
    if is_call(a, aten.silu.default):
        act, up = a, b
    elif is_call(b, aten.silu.default):
        act, up = b, a
    else:
        return None
    gate = act.args[0]
    if not sole_user_is(act, mul):
        return None
    vg, vu = gate.meta.get("val"), up.meta.get("val")
    if not (isinstance(vg, torch.Tensor) and isinstance(vu, torch.Tensor)):
        return None
    if vg.dtype not in _DTYPES or vg.dtype != vu.dtype or mul.meta["val"].dtype != vg.dtype:
        return None
    if not same_shape(vg.shape, vu.shape):
        return None
    sg, su = _last_dim_slice(gate), _last_dim_slice(up)
    if sg is not None and su is not None and sg[0] is su[0]:
        width = sg[0].meta["val"].shape[-1]
        d = width // 2
        if width % 2 == 0 and (sg[1], sg[2]) == (0, d) and (su[1], su[2]) == (d, width):
            return "halves", (sg[0],)
    return "pair", (gate, up)


class FusedSwiGLU(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]  # silu_mul / silu_mul2 carry backward formulas

    def process(self, gm):
        if not hasattr(gm, "mi355x_silu_mul"):
            gm.add_submodule("mi355x_silu_mul", SiluMulHalves())
            gm.add_submodule("mi355x_silu_mul2", SiluMulPair())
        g = gm.graph
        changed = False
        for node in reversed(list(g.nodes)):
            m = match_swiglu(node)
            if m is None:
                continue
            kind, args = m
            with g.inserting_before(node):
                new = g.call_module("mi355x_silu_mul" if kind == "halves" else "mi355x_silu_mul2", args=args)
            node.replace_all_uses_with(new)
            changed = True
        return changed
