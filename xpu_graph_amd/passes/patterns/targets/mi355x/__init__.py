"""The `mi355x` target: patterns that only make sense with the gfx950 kernel
library behind them (residual + norm, SwiGLU, stack+sum -> add-N, causal
attention, native norm ops) and, in `structure_replacements`, the modules the
structure patterns plug in.  Everything here ends in `torch.ops.xpu_ops.*`."""
from ...pattern import collect_patterns


def get_all_patterns(config):
    from ..... import ops as _register_ops  # noqa: F401  (defines torch.ops.xpu_ops)

    return collect_patterns(__name__, __path__, config)
