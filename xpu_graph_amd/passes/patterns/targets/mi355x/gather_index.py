"""A gather index that is a `repeat` of a size-1 axis need not be materialised: `expand` gives the gather the same
index as a stride-0 view, and an [B, N, 1] index repeated to [B, N, D] (row gather through `torch.gather`) costs
D times less memory traffic to build (reference targets/mlu/repeat_to_expand.py:16-48, `FusedGatherToCopy`).
The rewrite is made only where `repeat` really is a broadcast: same rank, and every repeated axis has size 1."""
from torch import fx

from .....config import OptLevel
from .....fx_utils import FxStage
from ...pattern import Pattern
from ...utils.node_utils import aten, is_call, same_shape


def _broadcast_sizes(repeat):
    """expand sizes equivalent to repeat(src, reps), or None when the repeat copies data."""
    src, reps = repeat.args[0], repeat.args[1]
    if not isinstance(src, fx.Node) or "val" not in src.meta:
        return None
    shape = src.meta["val"].shape
    if len(reps) != len(shape):
        return None
    sizes = []
    for dim, rep in zip(shape, reps):
        if isinstance(rep, int) and rep == 1:
            sizes.append(-1)
        elif same_shape(dim, 1):
            sizes.append(rep)
        else:
            return None
    return sizes


class FusedGatherToCopy(Pattern):
    _opt_level = OptLevel.level1
    _support_stages = [FxStage.inference, FxStage.pregrad]

    def process(self, gm):
        changed = False
        for gather in [n for n in gm.graph.nodes if is_call(n, aten.gather.default)]:
            index = gather.args[2]
            if not is_call(index, aten.repeat.default) or len(index.users) != 1:
                continue
            sizes = _broadcast_sizes(index)
            if sizes is None:
                continue
            with gm.graph.inserting_before(index):
                view = gm.graph.call_function(aten.expand.default, (index.args[0], sizes))
            index.replace_all_uses_with(view)
            gm.graph.erase_node(index)
            changed = True
        return changed
