"""The drop-in boundary: a target is a package `targets/<target.value>/` that
provides

    get_all_patterns(config)          -> {PatternGroup: [Pattern instances]}
    structure_replacements.get_structure_replacements(config)
                                      -> {"<StructurePatternClass>": Module | (Module, constraint_fn)}

A target without such a package contributes nothing
(reference src/xpu_graph/passes/patterns/targets/__init__.py:4-27)."""
import importlib
import importlib.util


def _has_target_package(config):
    return importlib.util.find_spec(f"{__package__}.{config.target.value}") is not None


def get_all_patterns(config) -> dict:
    if not _has_target_package(config):
        return {}
    # a target that exists but fails to import is an error, not "no patterns"
    mod = importlib.import_module(f".{config.target.value}", __package__)
    return mod.get_all_patterns(config)


def get_structure_replacements(config) -> dict:
    if _has_target_package(config):
        mod = importlib.import_module(f".{config.target.value}.structure_replacements", __package__)
        raw = mod.get_structure_replacements(config)
    else:
        raw = {}
    out = {}
    for name, spec in raw.items():
        if isinstance(spec, tuple):
            out[name] = {"target_mod": spec[0], "constraint_fn": spec[1]}
        else:
            out[name] = {"target_mod": spec}
    return out
