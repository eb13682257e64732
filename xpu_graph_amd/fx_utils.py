"""FX helpers shared by the compiler entry and the passes."""
import enum
from contextlib import nullcontext

import torch
from torch._guards import detect_fake_mode
from torch._subclasses.fake_tensor import FakeTensor, FakeTensorMode, unset_fake_temporarily


class FxStage(enum.Enum):
    """Which graph a pass sees (reference src/xpu_graph/fx_utils.py:36-40)."""

    inference = "inference"
    pregrad = "pregrad"
    forward = "forward"
    backward = "backward"


def fakify_tensors(inputs):
    """Return (fake_mode, inputs as FakeTensors); reuses the mode the inputs already belong to."""
    mode = detect_fake_mode(inputs)
    if mode is None:
        mode = FakeTensorMode(allow_non_fake_inputs=True)
    out = []
    for t in inputs:
        if isinstance(t, torch.Tensor) and not isinstance(t, FakeTensor):
            out.append(mode.from_tensor(t, static_shapes=True))
        else:
            out.append(t)
    return mode, out


def has_storage(node):
    val = node.meta.get("val")
    return isinstance(val, torch.Tensor) and not isinstance(val, torch._subclasses.FakeTensor) or (
        isinstance(val, FakeTensor) and val.layout == torch.strided
    )


def outside_fake_mode():
    """Context in which real tensors can be created even while a FakeTensorMode is active."""
    try:
        return unset_fake_temporarily()
    except Exception:  # pragma: no cover
        return nullcontext()


def node_val(node):
    return node.meta.get("val") if isinstance(node, torch.fx.Node) else None
