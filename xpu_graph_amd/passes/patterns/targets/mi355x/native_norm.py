"""Library norm ops -> the default norm modules, so that the structure and
residual-fusion patterns see F.layer_norm / F.rms_norm callers exactly like the
hand-written decomposed forms.  (The reference only matches the decomposed
spelling; `aten.native_layer_norm` passes through it untouched.)

    native_layer_norm(x, [N], w, b, eps)[0]  -> fused_layer_norm(x, w, b, eps)
    _fused_rms_norm(x, [N], w, eps)[0]       -> fused_rms_norm(x, w, eps)
    layer_norm(x, [N], w, b, eps, _)         -> fused_layer_norm(x, w, b, eps)     (pre-dispatch graphs: the
    rms_norm(x, [N], w, eps)                 -> fused_rms_norm(x, w, eps)           composite ops are still whole)

Only when the statistics outputs are unused and the norm is over the last axis.
"""

import torch

from .....config import OptLevel
from .....fx_utils import FxStage
from ...common.norms import LN_NAME, RMS_NAME
from ...pattern import Pattern
from ...utils.default_replacements import DefaultLayerNorm, DefaultRMSNorm
from ...utils.node_utils import aten, is_call, is_getitem, same_shape


def _only_output0(node):
    users = list(node.users)
    return len(users) >= 1 and all(is_getitem(u) and u.args[1] == 0 for u in users)


class NativeNormToDefault(Pattern):
    _opt_level = OptLevel.level2
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        if not hasattr(gm, LN_NAME):
            gm.add_module(LN_NAME, DefaultLayerNorm())
        if not hasattr(gm, RMS_NAME):
            gm.add_module(RMS_NAME, DefaultRMSNorm())
        g = gm.graph
        fused_rms = getattr(aten, "_fused_rms_norm", None)
        changed = False
        for node in list(g.nodes):
            if is_call(node, aten.native_layer_norm.default):
                x, nshape, w, b, eps = node.args[:5]
                name, args = LN_NAME, (x, w, b, eps)
            elif fused_rms is not None and is_call(node, fused_rms.default):
                x, nshape, w, eps = node.args[:4]
                if eps is None:
                    eps = torch.finfo(x.meta["val"].dtype).eps
                name, args = RMS_NAME, (x, w, eps)
            elif is_call(node, aten.layer_norm.default):
                x, nshape = node.args[:2]
                w = node.args[2] if len(node.args) > 2 else None
                b = node.args[3] if len(node.args) > 3 else None
                eps = node.args[4] if len(node.args) > 4 else 1e-5
                name, args = LN_NAME, (x, w, b, eps)
            elif hasattr(aten, "rms_norm") and is_call(node, aten.rms_norm.default):
                x, nshape = node.args[:2]
                w = node.args[2] if len(node.args) > 2 else None
                eps = node.args[3] if len(node.args) > 3 else None
                if eps is None:
                    eps = torch.finfo(x.meta["val"].dtype).eps
                name, args = RMS_NAME, (x, w, eps)
            else:
                continue
            single = is_call(node, aten.layer_norm.default) or (hasattr(aten, "rms_norm") and is_call(node, aten.rms_norm.default))
            if len(nshape) != 1 or not same_shape(list(nshape), list(x.meta["val"].shape[-1:])):
                continue
            if not isinstance(eps, (int, float)) or (not single and not _only_output0(node)):
                continue
            with g.inserting_before(node):
                new = g.call_module(name, args)
            if single:  # the composite ops return the normalised tensor itself
                node.replace_all_uses_with(new)
            else:
                for u in list(node.users):
                    u.replace_all_uses_with(new)
                    g.erase_node(u)
            g.erase_node(node)
            changed = True
        return changed
