"""Target-independent patterns: Aten -> Aten canonicalisations (level 1) and the
recognisers that turn norm / addmm / add-N / attention subgraphs into the
default replacement modules or single Aten ops (level 2)."""
from ..pattern import collect_patterns


def get_all_patterns(config):
    return collect_patterns(__name__, __path__, config)
