"""Structure patterns: target-independent matchers whose replacement is a module
supplied by the target.  A structure pattern is instantiated only when the
target's `get_structure_replacements` has an entry under its class name
(reference src/xpu_graph/passes/patterns/structure/__init__.py:8-34)."""
from ..pattern import collect_patterns


def get_all_patterns(config):
    from ..targets import get_structure_replacements

    repl = get_structure_replacements(config)

    def factory(cls):
        kwargs = repl.get(cls.__name__)
        return cls(**kwargs) if kwargs is not None else None

    return collect_patterns(__name__, __path__, config, factory)
