"""Input mutation and aliasing through the backend (reference tests/common/test_inplace.py:15-92): whatever the
passes fold away -- clones, copies, views -- the compiled function must leave its inputs in the same state as
eager does and return the same values, including when outputs alias the mutated input."""
import pytest
import torch

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar


def scatter_into_fresh(idx, v):
    out = torch.zeros(torch.max(idx) + 1, dtype=v.dtype, device=v.device)
    out.scatter_(0, idx, v)
    return out


def mutate_and_return(idx, v):
    return v.add_(1)


def functional_then_inplace(idx, v):
    a = v.add(1)
    b = v.add_(1)
    return a, b


def clone_between_mutations(idx, v):
    a = v.add_(1)
    b = v.clone()
    c = a.add_(1)
    return a, b, c


def chained_aliases(idx, v):
    a = v.add_(1)
    b = a.add_(1)
    return v, a, b


def copy_back_into_the_input(idx, v):
    a = v.add_(1)
    b = a.add(2)
    c = b.add_(a)
    a.copy_(c)
    d = a + b
    return a, b, c, d


def copy_into_a_clone(idx, v):
    a = v.add(1)
    b = v.clone()
    b.copy_(a)
    a.add_(2)
    return a, b, b + a


CASES = [scatter_into_fresh, mutate_and_return, functional_then_inplace, clone_between_mutations, chained_aliases,
         copy_back_into_the_input, copy_into_a_clone]


@pytest.fixture(scope="module")
def backend():
    return XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, enable_cache=False))


@pytest.mark.parametrize("dynamic", [True, False])
@pytest.mark.parametrize("fn", CASES)
def test_inplace_semantics_survive_the_passes(backend, fn, dynamic):
    idx = torch.tensor([7, 6, 5, 4, 0, 1, 2, 3], dtype=torch.int64)
    v = torch.randn(8)
    v_eager = v.clone()
    want = fn(idx, v_eager)
    got = torch.compile(fn, backend=backend, dynamic=dynamic)(idx, v)
    want = want if isinstance(want, tuple) else (want,)
    got = got if isinstance(got, tuple) else (got,)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert is_similar(g, w)
    assert is_similar(v, v_eager)  # the input was mutated exactly as eager mutates it
    torch._dynamo.reset()
