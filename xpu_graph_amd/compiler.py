"""`XpuGraph`: the torch.compile backend.

    compiled = torch.compile(fn, backend=XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x,
                                                               opt_level=OptLevel.level2)))

Dynamo hands over a Torch-IR graph; AOT dispatch lowers it to functional Aten
IR; the pass pipeline rewrites that graph (on the mi355x target: into calls of
the gfx950 kernels) and the rewritten GraphModule is what runs.  Entry points
and their behaviour follow the reference (src/xpu_graph/compiler.py:32-327);
graph capture goes through `aot_autograd` -- the reference's own path for
graphs with subclass inputs (compiler.py:138-154) -- because it is the stable
interface across torch versions.  No vendor compiler is involved: the compiled
artifact is the FX GraphModule itself.
"""
import itertools
import pickle
from typing import Callable

import torch
from torch._dynamo.backends.common import aot_autograd
from torch._functorch.aot_autograd import make_boxed_func

from .cache import SerializableArtifact, SerializableGraphModule, default_cache
from .config import Target, XpuGraphConfig, get_partition_fn
from .fx_utils import FxStage, fakify_tensors
from .passes.pass_manager import PassManager
from .passes.patterns.plugin_pattern import __PLUGIN_PATTERN_GROUP__
from .utils import local_logger, logger, setup_logger

__all__ = ["XpuGraph", "XpuGraphCompiler", "XpuGraphRuntimeArtifact"]


class XpuGraphRuntimeArtifact:
    """What torch.compile calls at run time; honours the boxed calling convention
    (reference src/xpu_graph/runtime/__init__.py:1-9)."""

    def __init__(self, compiled_func, boxed=None):
        self._compiled_func = compiled_func
        # The wrapper AOT returns takes *args yet inherits a `_boxed_call` attribute from the
        # module it wraps, so the convention is stated by the creator when it is known.
        self._boxed = getattr(compiled_func, "_boxed_call", False) if boxed is None else boxed

    def __call__(self, *args):
        if self._boxed:
            return self._compiled_func(list(args))
        return self._compiled_func(*args)


def _node_census(gm):
    counts = {}
    for n in gm.graph.nodes:
        if n.op in ("call_function", "call_module", "call_method"):
            counts[str(n.target)] = counts.get(str(n.target), 0) + 1
    return dict(sorted(counts.items(), key=lambda kv: -kv[1]))


class XpuGraph:
    def __init__(self, config: XpuGraphConfig, cache=None):
        config._reset_config_with_env()
        self._config = config
        setup_logger(config.debug)
        # reference compiler.py:43: a cache object counts only when the configuration enables caching
        self._cache = (cache if cache is not None else default_cache()) if config.enable_cache else None
        self._orig_ctx = {}
        self.compiled_graphs = []  # the last few rewritten GraphModules, newest last (inspection / tests)
        self._set_context()
        if config.is_training and config.target == Target.mi355x:
            from . import ops as _xops

            _xops.enable_autograd()  # the target's norm / gate / dense ops may enter training graphs
        self._pass_manager = PassManager(config)
        # plugin patterns run before the built-in ones of their group
        plugins = __PLUGIN_PATTERN_GROUP__.get(config.target, {})
        self._pass_manager.get_pattern_manager().insert_patterns(list(itertools.chain.from_iterable(plugins.values())))

    # -- compile one Aten graph ------------------------------------------------------
    def _get_compiler(self, stage: FxStage, boxed=True):
        """The function AOT (or, for the pregrad stage, this class) calls with a graph and its sample inputs.
        boxed: return the rewritten GraphModule wrapped for AOT's list calling convention, else the module itself."""

        def compile_stage(gm, sample_inputs):
            with local_logger(stage.name):
                if stage == FxStage.inference:
                    logger.info("decompose graph complete")
                kept = None
                if stage == FxStage.inference and self._config.freeze and not self._config.is_training:
                    kept = self._freeze(gm)
                    if kept is not None:
                        sample_inputs = [sample_inputs[i] for i in kept]
                fake_mode, fake_inputs = fakify_tensors(sample_inputs)
                if stage == FxStage.forward:
                    # a forward graph returns the caller's results first and the values saved for the backward after
                    # them; passes that would make two results share storage only need to look at the former
                    ctx = torch._guards.TracingContext.try_get()
                    meta = getattr(ctx, "fw_metadata", None) if ctx is not None else None
                    if meta is not None and hasattr(meta, "num_forward_returns"):
                        gm.meta["xg_user_outputs"] = int(meta.num_forward_returns)
                hashkey = None
                # a frozen graph carries its parameters as constants: the text of the graph, which is what the cache
                # key is made of, no longer identifies it (two models of one architecture would share an artifact)
                if self._cache is not None and kept is not None:
                    logger.info("frozen graph: not cached (its constants are this model's parameters)")
                if self._cache is not None and kept is None:
                    hashkey = self._cache.cache_key(gm, fake_inputs, self._config, stage)
                    cached = self._cache.load_artifact(hashkey)
                    if cached is not None:
                        assert isinstance(cached, SerializableArtifact)
                        self.compiled_graphs.append(cached.artifact)
                        del self.compiled_graphs[:-8]
                        runnable = self._vendor_compile(cached.artifact, fake_inputs, stage)
                        return make_boxed_func(runnable) if boxed else runnable
                with fake_mode:
                    with local_logger("before"):
                        logger.debug("before xpu_graph, graph like:\n %s", gm.print_readable(print_output=False))
                        logger.info(f"xpu_graph passes start {stage}...")
                    before = _node_census(gm)
                    out = self._pass_manager(gm, fake_inputs, stage)
                    with local_logger("after"):
                        logger.info("xpu_graph passes complete")
                        logger.debug("after xpu_graph, graph like:\n %s", out.print_readable(print_output=False))
                    logger.info(f"node statistic: before {before} after {_node_census(out)}")
                if hashkey is not None:
                    try:
                        # what runs is the re-loaded artifact, i.e. what a later process would get
                        out = self._cache.save_artifact(hashkey, SerializableGraphModule(out)).artifact
                    except (NotImplementedError, TypeError, AttributeError, pickle.PicklingError) as e:
                        logger.warning(f"Artifact is not serializable ({e}), skip cache.")
                self.compiled_graphs.append(out)
                del self.compiled_graphs[:-8]
                # the cache holds the rewritten graph; what the post-pass hook builds around it (recordings of
                # device graphs) is made again, cheaply, in every process
                runnable = self._vendor_compile(out, fake_inputs, stage)
                if kept is not None:
                    return _drop_frozen_args(runnable, kept)
                # AOT's runtime wrappers call the compiled stage with one list of arguments
                return make_boxed_func(runnable) if boxed else runnable

        return compile_stage

    def _freeze(self, gm):
        """Parameters and buffers of an inference graph become constants of the graph (reference
        fx_utils.py:89-350, `dispatch_graph` with freeze).  Returns the placeholder indices that stay inputs, or
        None (with a warning) when AOT did not say which inputs are parameters."""
        from .fx_utils import unlift_params

        ctx = torch._guards.TracingContext.try_get()
        params_flat = getattr(ctx, "params_flat", None) if ctx is not None else None
        fw_metadata = getattr(ctx, "fw_metadata", None) if ctx is not None else None
        if not params_flat or fw_metadata is None:
            logger.warning("freeze=True has no effect on this graph: it received its parameters as ordinary inputs")
            return None
        kept = unlift_params(gm, list(params_flat), fw_metadata)
        logger.info(f"freeze: {len(params_flat) - sum(1 for i in kept if i < len(params_flat))} parameters became constants, {len(kept)} inputs remain")
        return kept

    def __call__(self, dynamo_gm, example_inputs, *args, **kwargs):
        logger.info(f"{self._config}")
        logger.debug("before compile: graph like:\n %s", dynamo_gm.print_readable(print_output=False))
        if self._config.is_training:
            aot_kwargs = {
                "fw_compiler": self._get_compiler(FxStage.forward),
                "bw_compiler": self._get_compiler(FxStage.backward),
                "inference_compiler": self._get_compiler(FxStage.inference),
                "keep_inference_input_mutations": True,
            }
            part = get_partition_fn(self._config.partition_fn)
            if part is not None:
                aot_kwargs["partition_fn"] = part
            # Patterns that replace a differentiable subgraph must run BEFORE autograd is traced: afterwards the
            # forward graph hands the intermediates of that subgraph to the backward graph and nothing matches.
            # So the Dynamo graph is first lowered to pre-dispatch Aten IR, rewritten in the `pregrad` stage, and
            # AOT then differentiates the rewritten module (reference compiler.py:158-182).
            pregrad_gm = None if self._needs_plain_dispatch(dynamo_gm, example_inputs) else self._pregrad(dynamo_gm, example_inputs)
            compiled = aot_autograd(**aot_kwargs)(pregrad_gm if pregrad_gm is not None else dynamo_gm, example_inputs)
        else:
            aot_kwargs = {"fw_compiler": self._get_compiler(FxStage.inference), "keep_inference_input_mutations": True}
            self._needs_plain_dispatch(dynamo_gm, example_inputs)  # for its warnings: AOT handles both cases
            logger.info("decompose graph start...")  # "complete" is logged by the stage that receives the Aten graph
            # an inference compiler: trace without autograd whatever the caller's grad mode is
            with torch.no_grad():
                compiled = aot_autograd(**aot_kwargs)(dynamo_gm, example_inputs)
        artifact = XpuGraphRuntimeArtifact(compiled, boxed=False)
        if self._config.enable_interceptor is not None:
            import os

            from .interceptor import intercept

            logger.info("Wrapping compiled function with interceptor")
            tctx = torch._guards.TracingContext.try_get()
            artifact = intercept(
                artifact,
                golden_fn=dynamo_gm,
                fw_metadata=getattr(tctx, "fw_metadata", None) if tctx is not None else None,
                is_training=self._config.is_training,
                mark=os.environ.get("RANK", "0"),
                config_str=self._config.enable_interceptor,
            )

        opts = kwargs.get("options") or {}
        guard_filter_fn = opts.get("guard_filter_fn")
        ctx = torch._guards.TracingContext.try_get()
        if guard_filter_fn is not None and ctx is not None:
            guards = ctx.guards_context.dynamo_guards
            flags = guard_filter_fn(guards)
            dropped = torch._guards.GuardsSet({g for g, keep in zip(guards, flags) if not keep})
            logger.info(f"Removed guards: {list(dropped)}")
            ctx.guards_context.dynamo_guards = guards - dropped
        return artifact

    def _needs_plain_dispatch(self, dynamo_gm, example_inputs):
        """True when the Dynamo graph must go to AOT as it is (reference compiler.py:125-138): in training, bodies
        of higher-order operators would be lost to a pre-autograd rewrite; tensor-subclass inputs need AOT's own
        unwrapping.  Says which of the two it found."""
        from .fx_utils import find_hop_nodes, find_subclass_inputs

        plain = False
        if self._config.is_training:
            hops = find_hop_nodes(dynamo_gm)
            if hops:
                logger.warning(f"Higher order operators detected: {', '.join(str(op) for op in hops)}.")
                plain = True
        subclasses = find_subclass_inputs(example_inputs)
        if subclasses:
            logger.warning(f"Subclass inputs detected: {', '.join(str(cls) for cls in subclasses)}.")
            plain = True
        return plain

    def _vendor_compile(self, gm, fake_inputs, stage: FxStage):
        """The post-pass hook (reference compiler.py:90-103): with `vendor_compiler_config` set, every stage but
        pregrad goes through `backends.vendor_compiler`."""
        cfg = self._config.vendor_compiler_config
        if cfg is None or stage == FxStage.pregrad:
            return gm
        from .backends import vendor_compiler

        return vendor_compiler(
            gm, fake_inputs, self._config.target, is_inference=stage == FxStage.inference, is_backward=stage == FxStage.backward, **cfg
        )

    def _pregrad(self, dynamo_gm, example_inputs):
        """The Dynamo graph as a rewritten pre-autograd Aten module, or None when it cannot be taken apart that way
        (higher-order operators, tensor-subclass inputs, input mutation, parameters held by the module): the graph
        then goes to AOT as it is and only the forward / backward stages see it."""
        from .fx_utils import dispatch_pregrad

        logger.info("decompose graph start...")
        try:
            dispatched = dispatch_pregrad(dynamo_gm, example_inputs)
        except NotImplementedError as e:
            logger.warning(f"pregrad stage skipped: {e}")
            return None
        logger.info("decompose graph complete")
        logger.debug("after decompose, graph like:\n %s", dispatched.print_readable(print_output=False))
        # The exported graph's metadata does not say which inputs will be differentiated; patterns that may only take
        # operands without a gradient (an attention mask) read it from the placeholders.
        placeholders = [n for n in dispatched.graph.nodes if n.op == "placeholder"]
        if len(placeholders) == len(example_inputs):
            for node, real in zip(placeholders, example_inputs):
                node.meta["xg_requires_grad"] = bool(isinstance(real, torch.Tensor) and real.requires_grad)
        return self._get_compiler(FxStage.pregrad, boxed=False)(dispatched, example_inputs)

    def get_pattern_manager(self):
        return self._pass_manager.get_pattern_manager()

    def _set_context(self):
        import torch._inductor.config as inductor_config

        self._orig_ctx["freezing"] = inductor_config.freezing
        inductor_config.freezing = bool(self._config.freeze and not self._config.is_training)

    def _restore_context(self):
        import torch._inductor.config as inductor_config

        inductor_config.freezing = self._orig_ctx["freezing"]


def _drop_frozen_args(runnable, kept):
    """AOT keeps passing every parameter at run time; the frozen graph takes only the inputs it kept."""

    def call(args):
        live = [args[i] for i in kept]
        args.clear()
        return runnable(*live)

    call._boxed_call = True
    return call


class XpuGraphCompiler:
    """Fluent wrapper: XpuGraphCompiler().set_target(...).set_opt_level(...).done(); .compile(model)
    (reference compiler.py:273-327).  Every config field gets a property and a chained set_<field>."""

    def __init__(self):
        self._config = XpuGraphConfig(is_training=False)
        self._config._reset_config_with_env()
        self._compiler = None
        self.prior_work()

    def __init_subclass__(cls, **kw):
        super().__init_subclass__(**kw)

    def prior_work(self):
        ...

    def done(self):
        self._compiler = XpuGraph(self._config)
        return self

    def compile(self, model, *args, backend=None, **kwargs) -> Callable:
        assert isinstance(self._compiler, XpuGraph), "You should call XpuGraphCompiler.done before XpuGraphCompiler.compile"
        return torch.compile(model, *args, backend=self._compiler, **kwargs)


def _install_config_accessors():
    import dataclasses

    for f in dataclasses.fields(XpuGraphConfig):
        name = f.name

        def getter(self, _n=name):
            return getattr(self._config, _n)

        def setter(self, val, _n=name):
            setattr(self._config, _n, val)
            self._compiler = None

        def chained(self, val, _s=setter):
            _s(self, val)
            return self

        setattr(XpuGraphCompiler, name, property(getter, setter))
        setattr(XpuGraphCompiler, f"set_{name}", chained)


_install_config_accessors()
