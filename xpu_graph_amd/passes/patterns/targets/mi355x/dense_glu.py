"""silu(x Wg^T) * (x Wu^T): two dense calls and the SwiGLU gate -> one gated dense kernel.

    silu_mul2(reshape?(dense(x, Wg, True, None, "none")), reshape?(dense(x, Wu, True, None, "none")))
    mul(reshape?(dense(x, Wg, True, None, "silu")), reshape?(dense(x, Wu, True, None, "none")))
        ->  reshape?(dense_glu(x, Wg, Wu))

(the second spelling is what is left when the dense pattern has already taken the SiLU into the gate projection)

Both projections read the same activations, both weights are [N, K] (torch.nn.Linear layout) of one shape, and each
dense result (and its reshape) has no other user.  The kernel computes both projections in one workgroup -- the A
operand is loaded once for the pair -- and applies the gate in its epilogue, so the two [M, N] intermediates are never
written and the separate gate kernel disappears.  Results are bit-identical to the unfused sequence (each projection
is rounded to the storage type before the gate).  No counterpart in the reference.
"""
import torch
from torch import fx, nn

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern, PatternGroup
from ...structure.dense import DENSE_NAME
from ...utils.node_utils import VIEW_OPS, aten, is_call, same_shape

GLU_NAME = "mi355x_dense_glu"
SILU_MUL2 = "mi355x_silu_mul2"


class DenseGLUModule(nn.Module):
    def forward(self, x, w_gate, w_up):
        if torch.is_grad_enabled() and (x.requires_grad or w_gate.requires_grad or w_up.requires_grad):
            # a graph that will be differentiated: the same launch also writes the two projections, which the backward
            # needs and would otherwise run again (two more dense layers)
            return torch.ops.xpu_ops.dense_glu_save(x, w_gate, w_up)[0]
        return torch.ops.xpu_ops.dense_glu(x, w_gate, w_up)


def _plain_dense(node, want_act="none"):
    """(dense call, reshape or None) for `dense` or `reshape(dense)` with single users, no bias, [N, K] weight and the
    activation `want_act`."""
    view = None
    if is_call(node, *VIEW_OPS) and len(node.users) == 1:
        view, node = node, node.args[0]
    if not (isinstance(node, fx.Node) and node.op == "call_module" and node.target == DENSE_NAME and len(node.users) == 1):
        return None, None
    if len(node.args) != 5 or node.kwargs:
        return None, None
    _, _, weight_trans, bias, act = node.args
    if weight_trans is not True or bias is not None or act != want_act:
        return None, None
    return node, view


def _gate_and_up(node):
    """((gate dense, its reshape), (up dense, its reshape)) for the two spellings of the gated product: the SwiGLU
    module over two plain projections, or a multiplication whose one factor is a projection that already took the
    SiLU into its epilogue."""
    none = ((None, None), (None, None))
    if node.op == "call_module" and node.target == SILU_MUL2 and len(node.args) == 2:
        return _plain_dense(node.args[0]), _plain_dense(node.args[1])
    if is_call(node, aten.mul.Tensor) and len(node.args) == 2 and all(isinstance(a, fx.Node) for a in node.args):
        for a, b in (node.args, node.args[::-1]):
            gate, up = _plain_dense(a, "silu"), _plain_dense(b)
            if gate[0] is not None and up[0] is not None:
                va, vb, vo = (n.meta.get("val") for n in (a, b, node))
                if all(isinstance(v, torch.Tensor) for v in (va, vb, vo)) and va.shape == vb.shape == vo.shape and va.dtype == vb.dtype == vo.dtype:
                    return gate, up
    return none


class FusedDenseGLU(Pattern):
    _opt_level = OptLevel.level2
    _pattern_group = PatternGroup.GROUP2
    _support_stages = [FxStage.inference, FxStage.pregrad]  # dense_glu carries a backward formula

    def process(self, gm):
        from ..... import ops as _xops

        g = gm.graph
        changed = False
        for node in list(g.nodes):
            (dg, vg), (du, vu) = _gate_and_up(node)
            if dg is None or du is None or dg is du or dg.args[0] is not du.args[0]:
                continue
            x, wg, wu = dg.args[0], dg.args[1], du.args[1]
            vals = [n.meta.get("val") if isinstance(n, fx.Node) else None for n in (x, wg, wu)]
            if not all(isinstance(v, torch.Tensor) for v in vals):
                continue
            xv, gv, uv = vals
            if gv.shape != uv.shape or gv.dtype != xv.dtype or uv.dtype != xv.dtype:
                continue
            if not _xops.dense_glu_fits(tuple(xv.shape), tuple(gv.shape), xv.dtype):
                continue
            out_shape = list(node.meta["val"].shape) if "val" in node.meta else None
            if out_shape is None:
                continue
            symbolic = [i for i, d in enumerate(out_shape) if not isinstance(d, int)]
            if len(symbolic) > 1:  # the reshape back can leave one dim (the batch) to be inferred
                continue
            back_shape = [(-1 if i in symbolic else d) for i, d in enumerate(out_shape)]
            if not hasattr(gm, GLU_NAME):
                gm.add_submodule(GLU_NAME, DenseGLUModule())
            with g.inserting_before(node):
                fused = g.call_module(GLU_NAME, args=(x, wg, wu))
                new = fused
                if not same_shape(out_shape, [xv.shape[0], gv.shape[0]]):
                    new = g.call_function(aten.reshape.default, (fused, back_shape))
            node.replace_all_uses_with(new)
            g.erase_node(node)
            for n in (vg, vu, dg, du):
                if n is not None and len(n.users) == 0:
                    g.erase_node(n)
            changed = True
        return changed
