"""Run-time parity guard: every call of a compiled function also runs the function it was compiled from
(the Dynamo graph) and compares inputs after the call, outputs and -- when training -- input gradients; a
divergence is logged and the tensors of the case are dumped under the dump directory.

Switched on by `XpuGraphConfig.enable_interceptor` / XPUGRAPH_INTERCEPTOR, a comma-separated `key=value` list:
rtol, atol, equal_nan, check_device, check_dtype, check_layout, check_stride, allow_subclasses are handed to
`torch.testing.assert_close`; `use_golden=1` makes the golden function's results the ones returned (the compiled
one is then only checked).  Behaviour of the reference's src/xpu_graph/interceptor.py:16-405 (`intercept`,
`FunctionInterceptor`, `AutogradInterceptor`, `OpInterceptor`).
"""
import copy
import itertools
import os
from typing import Callable

import torch
from torch.fx import GraphModule
from torch.utils._python_dispatch import TorchDispatchMode

from .config import get_dump_dir
from .utils import logger

__all__ = ["intercept", "FunctionInterceptor", "AutogradInterceptor", "OpInterceptor", "compare_tensor_list"]

_CASE_IDS = itertools.count()
_FLOAT_KEYS = ("rtol", "atol")
_BOOL_KEYS = ("allow_subclasses", "equal_nan", "check_device", "check_dtype", "check_layout", "check_stride")


def parse_config(config_str):
    """'rtol=1e-3,atol=1e-3,use_golden=1' -> ({'rtol': 1e-3, 'atol': 1e-3}, True)"""
    checks, use_golden = {}, False
    for item in filter(None, (config_str or "").split(",")):
        key, _, val = item.partition("=")
        key = key.strip()
        truth = val.strip().lower() in ("true", "1", "on")
        if key in _FLOAT_KEYS:
            checks[key] = float(val)
        elif key in _BOOL_KEYS:
            checks[key] = truth
        elif key == "use_golden":
            use_golden = truth
        else:
            logger.warning(f"Invalid key: {key}")
    return checks, use_golden


def compare_tensor_list(base_list, trgt_list, **check_configs):
    """Number of positions at which the two lists differ beyond the tolerances; each one is logged."""
    diverged = 0
    for i, (base_t, trgt_t) in enumerate(zip(base_list, trgt_list)):
        try:
            torch.testing.assert_close(trgt_t, base_t, **check_configs)
        except AssertionError as e:
            diverged += 1
            logger.warning(f"Tensor {i} diverges:\n{e}")
    return diverged


def _as_list(out):
    return list(out) if isinstance(out, (tuple, list)) else [out]


def _rng_device_type():
    # fork_rng always forks the CPU generator; with no accelerator present, "cuda" makes it fork nothing else
    return torch._utils._get_available_device_type() or "cuda"


class _Reporter:
    """Names the case, writes the golden graph and the tensors of a divergence."""

    def __init__(self, golden_fn, mark):
        self.golden_fn, self.mark = golden_fn, mark

    def report(self, phase, summary, file_name, payload):
        path = os.path.join(get_dump_dir(), f"case_{self.mark}_{phase}_{next(_CASE_IDS)}")
        logger.warning(f"Summary: The {phase} pass diverges for {self.golden_fn}\n         {summary}\n         cases saved_to: {path}")
        os.makedirs(path, exist_ok=True)
        if isinstance(self.golden_fn, GraphModule):
            with open(os.path.join(path, "golden_mod.py"), "w") as f:
                f.write(self.golden_fn.print_readable(print_output=False, include_stride=True, include_device=True))
        torch.save(payload, os.path.join(path, file_name))


def _forward_both(base_func, trgt_func, base_inputs, impure, grad):
    """Runs the checked function first, inside a forked RNG state, then the one whose results are kept, so that
    random ops see the same stream in both.  Impure functions (input mutation) get their own copy of the inputs."""
    backup = copy.deepcopy(base_inputs) if impure else base_inputs
    trgt_inputs = copy.deepcopy(base_inputs) if impure else base_inputs
    ctx = torch.enable_grad if grad else _null
    with torch.random.fork_rng(device_type=_rng_device_type()):
        with ctx():
            trgt_outputs = trgt_func(*trgt_inputs)
    with ctx():
        base_outputs = base_func(*base_inputs)
    return backup, trgt_inputs, trgt_outputs, base_outputs


class _null:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


def _carry_module_api(src, dst):
    for name in ("zero_grad", "named_parameters", "named_buffers"):
        if hasattr(src, name):
            setattr(dst, name, getattr(src, name))
    return dst


class FunctionInterceptor:
    """Inference: no autograd involved; the golden graph is stateless (Dynamo passes parameters as inputs)."""

    def __init__(self, golden_fn: Callable, mark=0, use_golden=False, impure=True, **check_configs):
        self.golden_fn, self.mark = golden_fn, mark
        self.use_golden, self.impure, self.check_configs = use_golden, impure, check_configs
        self._reporter = _Reporter(golden_fn, mark)

    def guard(self, compiled_fn):
        base_func, trgt_func = (self.golden_fn, compiled_fn) if self.use_golden else (compiled_fn, self.golden_fn)

        def monitored_inference(*inputs):
            logger.info("Monitored inference")
            backup, trgt_inputs, trgt_out, base_out = _forward_both(base_func, trgt_func, inputs, self.impure, grad=False)
            n_in = compare_tensor_list(inputs, trgt_inputs, **self.check_configs) if self.impure else 0
            n_out = compare_tensor_list(_as_list(base_out), _as_list(trgt_out), **self.check_configs)
            if n_in + n_out > 0:
                golden, actual = ((inputs, base_out), (trgt_inputs, trgt_out)) if self.use_golden else ((trgt_inputs, trgt_out), (inputs, base_out))
                self._reporter.report(
                    "inference",
                    f"input_diverge_cnt: {n_in}, output_diverge_cnt: {n_out}",
                    "dump_glob_inf.pt",
                    {"inputs": backup, "golden_inputs": golden[0], "actual_inputs": actual[0], "golden_outputs": golden[1], "actual_outputs": actual[1]},
                )
            return base_out

        return _carry_module_api(compiled_fn, monitored_inference)


def _grads_of(func_inputs, func_outputs, grad_outputs, inputs_requires_grad):
    """d(outputs)/d(inputs that required grad), given the cotangents of [inputs mutated in place..., outputs...]."""
    wrt, heads, cots = [], [], []
    for i, t in enumerate(func_inputs):
        if inputs_requires_grad[i]:
            wrt.append((i, t))
        elif isinstance(t, torch.Tensor) and t.requires_grad:  # became part of the graph through an in-place update
            heads.append(t)
            cots.append(grad_outputs[i])
    for j, t in enumerate(func_outputs):
        if isinstance(t, torch.Tensor) and t.requires_grad:
            heads.append(t)
            cots.append(grad_outputs[len(func_inputs) + j])
    grads = [None] * len(func_inputs)
    if wrt and heads:
        got = torch.autograd.grad(heads, [t for _, t in wrt], cots, allow_unused=True)
        for (i, _), g in zip(wrt, got):
            grads[i] = g
    return tuple(grads)


class AutogradInterceptor:
    """Training: forward of both functions on detached leaves inside one autograd.Function, whose backward
    differentiates both and compares the input gradients."""

    def __init__(self, golden_fn: Callable, mark=0, use_golden=False, impure=True, **check_configs):
        if isinstance(golden_fn, torch.nn.Module):
            assert len(golden_fn.state_dict()) == 0, "the golden graph must be stateless"
        self.golden_fn, self.mark = golden_fn, mark
        self.use_golden, self.impure, self.check_configs = use_golden, impure, check_configs
        self._reporter = _Reporter(golden_fn, mark)

    def guard(self, compiled_fn):
        outer = self
        base_func, trgt_func = (self.golden_fn, compiled_fn) if self.use_golden else (compiled_fn, self.golden_fn)

        class Monitored(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *inputs):
                logger.info("Monitored forward")
                needs = [isinstance(t, torch.Tensor) and t.requires_grad for t in inputs]
                leaves = [t.detach().requires_grad_(t.requires_grad) if isinstance(t, torch.Tensor) else t for t in inputs]
                backup, trgt_inputs, trgt_out, base_out = _forward_both(base_func, trgt_func, leaves, outer.impure, grad=True)
                base_out, trgt_out = _as_list(base_out), _as_list(trgt_out)
                n_in = compare_tensor_list(leaves, trgt_inputs, **outer.check_configs) if outer.impure else 0
                n_out = compare_tensor_list(base_out, trgt_out, **outer.check_configs)
                if n_in + n_out > 0:
                    golden, actual = ((leaves, base_out), (trgt_inputs, trgt_out)) if outer.use_golden else ((trgt_inputs, trgt_out), (leaves, base_out))
                    outer._reporter.report(
                        "forward",
                        f"input_diverge_cnt: {n_in}, output_diverge_cnt: {n_out}",
                        "dump_glob_fwd.pt",
                        {"inputs": backup, "golden_inputs": golden[0], "actual_inputs": actual[0], "golden_outputs": golden[1], "actual_outputs": actual[1]},
                    )
                ctx.saved = (leaves, trgt_inputs, base_out, trgt_out, needs)
                # inputs that entered the graph through an in-place update are handed back so that the caller's
                # tensors can take their values; returning a tuple guarantees that backward is reached
                updated = [
                    t.detach().requires_grad_(True) if isinstance(t, torch.Tensor) and t.requires_grad and not need else None
                    for t, need in zip(leaves, needs)
                ]
                outs = [t.detach().requires_grad_(True) if isinstance(t, torch.Tensor) and t.requires_grad else t for t in base_out]
                return tuple(updated + outs)

            @staticmethod
            def backward(ctx, *grad_outputs):
                logger.info("Monitored backward")
                leaves, trgt_inputs, base_out, trgt_out, needs = ctx.saved
                trgt_grads = _grads_of(trgt_inputs, trgt_out, grad_outputs, needs)
                base_grads = _grads_of(leaves, base_out, grad_outputs, needs)
                n = compare_tensor_list(base_grads, trgt_grads, **outer.check_configs)
                if n > 0:
                    golden, actual = ((leaves, base_grads), (trgt_inputs, trgt_grads)) if outer.use_golden else ((trgt_inputs, trgt_grads), (leaves, base_grads))
                    outer._reporter.report(
                        "backward",
                        f"grad_diverge_cnt: {n}",
                        "dump_glob_bwd.pt",
                        {"golden_inputs": golden[0], "actual_inputs": actual[0], "grad_outputs": grad_outputs, "golden_grad_inputs": golden[1], "actual_grad_inputs": actual[1]},
                    )
                return base_grads

        def monitored_forward(*inputs):
            results = Monitored.apply(*inputs)
            for t, t_after in zip(inputs, results[: len(inputs)]):
                if t_after is not None:
                    t.copy_(t_after)
            return results[len(inputs) :]

        return _carry_module_api(compiled_fn, monitored_forward)


def intercept(target_fn, *, golden_fn, fw_metadata, is_training, mark=0, config_str=""):
    checks, use_golden = parse_config(config_str)
    # Mutations that stay inside the compiled graph (keep_inference_input_mutations) do not show up in
    # num_mutated_inp_runtime_indices, so the per-input records decide; unknown metadata counts as impure.
    if fw_metadata is None:
        impure = True
    else:
        infos = getattr(fw_metadata, "input_info", None) or []
        impure = fw_metadata.num_mutated_inp_runtime_indices > 0 or any(
            getattr(i, "mutates_data", False) or getattr(i, "mutates_metadata", False) for i in infos
        )
    cls = AutogradInterceptor if is_training else FunctionInterceptor
    return cls(golden_fn, mark, use_golden=use_golden, impure=impure, **checks).guard(target_fn)


class OpInterceptor(TorchDispatchMode):
    """`with OpInterceptor({op: golden_fn}, **assert_close options):` checks every dispatch of the listed ops
    against its golden function; results of the real op are what the program sees."""

    def __init__(self, golden_funcs, mark=None, dispatch_key=None, **check_configs):
        super().__init__(dispatch_key)
        self.golden_funcs = golden_funcs
        self.mark = "op" if mark is None else mark
        self.check_configs = check_configs

    def __torch_dispatch__(self, func, types, args, kwargs=None):
        kwargs = kwargs or {}
        golden_fn = self.golden_funcs.get(func)
        if golden_fn is None:
            return func(*args, **kwargs)
        logger.info(f"Monitored op: {func}")
        golden_inputs = copy.deepcopy(args)
        with torch.random.fork_rng(device_type=_rng_device_type()):
            golden_outputs = golden_fn(*golden_inputs, **kwargs)
        actual_outputs = func(*args, **kwargs)
        n_in = compare_tensor_list(_as_list(args), _as_list(golden_inputs), **self.check_configs)
        n_out = compare_tensor_list(_as_list(actual_outputs), _as_list(golden_outputs), **self.check_configs)
        if n_in + n_out > 0:
            path = os.path.join(get_dump_dir(), f"case_{self.mark}_op_{next(_CASE_IDS)}")
            logger.warning(
                f"Summary: The op diverges for {func}\n         input_diverge_cnt: {n_in}, output_diverge_cnt: {n_out}\n         cases saved_to: {path}"
            )
            os.makedirs(path, exist_ok=True)
            torch.save(
                {"golden_inputs": golden_inputs, "actual_inputs": args, "golden_outputs": golden_outputs, "actual_outputs": actual_outputs},
                os.path.join(path, "dump_glob_op.pt"),
            )
        return actual_outputs
