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


def find_hop_nodes(gm):
    """{operator: [nodes]} for the higher-order operators of a Dynamo graph (autograd.Function applications,
    activation checkpoints, control flow): their bodies are sub-graphs a flat Aten rewrite cannot see
    (reference fx_utils.py:410-420)."""
    hops = {}
    for n in gm.graph.nodes:
        if n.op == "call_function" and isinstance(n.target, torch._ops.HigherOrderOperator):
            hops.setdefault(n.target, []).append(n)
    return hops


def find_subclass_inputs(inputs):
    """{type: [tensors]} for inputs that are traceable tensor subclasses (reference fx_utils.py:423-436)."""
    from torch.utils._python_dispatch import is_traceable_wrapper_subclass_type

    found = {}
    for t in inputs:
        if isinstance(t, torch.Tensor) and is_traceable_wrapper_subclass_type(type(t)):
            found.setdefault(type(t), []).append(t)
    return found


def dispatch_pregrad(gm, example_inputs):
    """Lower a Dynamo graph to functional PRE-DISPATCH Aten IR (composite ops such as linear or layer_norm stay
    whole, autograd has not been traced) with the same inputs and outputs, ready for the `pregrad` pattern stage
    (reference fx_utils.dispatch_graph(stage=FxStage.pregrad), src/xpu_graph/fx_utils.py:89-121).  Raises
    NotImplementedError for graphs this cannot represent."""
    from torch._functorch.aot_autograd import aot_export_module

    if any(True for _ in gm.parameters()) or any(True for _ in gm.buffers()):
        raise NotImplementedError("the graph owns parameters or buffers (Dynamo did not lift them to inputs)")
    for n in gm.graph.nodes:
        if n.op == "call_function" and isinstance(n.target, torch._ops.HigherOrderOperator):
            raise NotImplementedError(f"higher-order operator {n.target}")
    for t in example_inputs:
        if isinstance(t, torch.Tensor) and type(t) not in (torch.Tensor, torch.nn.Parameter, FakeTensor):
            raise NotImplementedError(f"tensor subclass input {type(t).__name__}")
    try:
        out, sig = aot_export_module(gm, list(example_inputs), trace_joint=False, pre_dispatch=True)
    except Exception as e:  # export refuses some graphs (data-dependent control, unsupported mutation, ...)
        raise NotImplementedError(f"pre-dispatch export failed: {type(e).__name__}: {e}") from e
    if sig.user_inputs_to_mutate or sig.buffers_to_mutate or getattr(sig, "parameters_to_mutate", None) or sig.input_tokens:
        raise NotImplementedError("the graph mutates its inputs")
    return out


def unlift_params(gm, params_flat, fw_metadata):
    """Freezing (reference fx_utils.py `_unlift_params`): AOT hands the inference compiler a graph whose first
    len(params_flat) placeholders are the module's parameters and buffers.  Each of them that the graph neither
    writes nor hands back as (an alias of) an output becomes a `get_attr` constant holding the parameter itself, so
    that ConstantFolding(folding_freezed_params) can fold weight-side subgraphs (a transposed or pre-scaled weight).
    Returns the indices of the placeholders that remain graph inputs, in order."""
    from torch._functorch._aot_autograd.schemas import MutationType

    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    aliased = {info.base_idx for info in fw_metadata.output_info if info.base_idx is not None}
    mutated = {i for i, m in enumerate(fw_metadata.input_info) if m.mutation_type in (MutationType.MUTATED_IN_GRAPH, MutationType.MUTATED_OUT_GRAPH)}
    kept = []
    for i, (node, real) in enumerate(zip(placeholders, params_flat)):
        if i in aliased or i in mutated or not isinstance(real, torch.Tensor):
            kept.append(i)
            continue
        name = f"_xg_frozen_param{i}"
        if isinstance(real, torch.nn.Parameter):
            gm.register_parameter(name, real)  # the parameter itself, not a copy
        else:
            gm.register_buffer(name, real, persistent=False)
        with gm.graph.inserting_before(node):
            const = gm.graph.get_attr(name)
        const.meta.update({k: v for k, v in node.meta.items() if k in ("val", "tensor_meta")})
        node.replace_all_uses_with(const)
        gm.graph.erase_node(node)
    kept.extend(range(len(params_flat), len(placeholders)))
    gm.recompile()
    return kept
