"""Level-1 algebraic and shape folds on the default (target none) path: each case compiles, matches eager and
reports the pattern that rewrote it (reference tests/common/test_fold_add.py, test_fold_sub.py, test_fold_mul.py,
test_fold_div.py, test_fold_where.py, test_fold_reduce.py, test_fold_stack.py, test_fold_squeeze.py,
test_fold_slice_like.py, test_change_tensor_like.py)."""
import pytest
import torch

from xpu_graph_amd import XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs, skip_xpu_graph_cache


@pytest.fixture(scope="module")
def infer_backend():
    return XpuGraph(XpuGraphConfig(is_training=False, enable_cache=False))


@pytest.fixture(scope="module")
def train_backend():
    return XpuGraph(XpuGraphConfig(is_training=True, enable_cache=False))


def run(backend, fn, *args, dynamic=False, exact=False):
    want = fn(*args)
    got = torch.compile(fn, backend=backend, dynamic=dynamic)(*args)
    want = want if isinstance(want, (tuple, list)) else (want,)
    got = got if isinstance(got, (tuple, list)) else (got,)
    assert len(want) == len(got)
    for w, g in zip(want, got):
        assert w.dtype == g.dtype and w.shape == g.shape
        assert torch.equal(w, g) if exact else is_similar(w.float(), g.float())
    torch._dynamo.reset()


# ---- neutral elements -------------------------------------------------------------------------------------------
NEUTRAL = {
    "FoldAdd0": [lambda x: x + 0, lambda x: x + torch.zeros_like(x), lambda x: 42 + torch.zeros_like(x),
                 lambda x: x + torch.zeros_like(x.unsqueeze(-1)), lambda x: x + torch.zeros_like(x) + 0],
    "FoldSub0": [lambda x: x - 0, lambda x: x - torch.zeros_like(x), lambda x: torch.rsub(torch.zeros_like(x), x),
                 lambda x: x - torch.zeros_like(x.unsqueeze(-1))],
    "FoldMul1": [lambda x: x * 1, lambda x: x * torch.ones_like(x), lambda x: 7 * torch.ones_like(x),
                 lambda x: x * torch.ones_like(x.unsqueeze(-1)), lambda x: x * torch.ones_like(x) * 1],
    "FoldDiv1": [lambda x: x / 1, lambda x: x / torch.ones_like(x), lambda x: x / torch.ones_like(x.unsqueeze(-1))],
}
# case index -> needs a shape written out, which a symbolic shape does not allow
NEEDS_STATIC = {"FoldAdd0": {2, 3}, "FoldSub0": {3}, "FoldMul1": {2, 3}, "FoldDiv1": {2}}


@pytest.mark.parametrize("name,idx", [(k, i) for k, v in NEUTRAL.items() for i in range(len(v))])
def test_neutral_operand_is_folded(caplog, infer_backend, name, idx):
    with need_xpu_graph_logs():
        run(infer_backend, NEUTRAL[name][idx], torch.rand(100))
    assert f"Pattern.{name} changed graph" in caplog.text


@pytest.mark.parametrize("name,idx", [(k, i) for k, v in NEUTRAL.items() for i in range(len(v))])
def test_neutral_operand_with_symbolic_shapes_in_training(caplog, train_backend, name, idx):
    with need_xpu_graph_logs():
        run(train_backend, NEUTRAL[name][idx], torch.rand(100), dynamic=True)
    if idx in NEEDS_STATIC[name]:
        assert f"Pattern.{name} changed graph" not in caplog.text
    else:
        assert f"Pattern.{name} changed graph" in caplog.text


def test_folded_arithmetic_does_not_alias_its_input(infer_backend):
    def fn(x):
        y = x + 0
        y.add_(1)  # must not reach x
        return y

    x = torch.rand(16)
    keep = x.clone()
    got = torch.compile(fn, backend=infer_backend)(x)
    assert torch.equal(x, keep) and torch.equal(got, keep + 1)
    torch._dynamo.reset()


def test_integer_division_with_rounding_is_left_alone(caplog, infer_backend):
    with need_xpu_graph_logs():
        run(infer_backend, lambda x: torch.div(x, 1, rounding_mode="floor"), torch.randn(8) * 5, exact=True)
    assert "Pattern.FoldDiv1 changed graph" not in caplog.text


# ---- where ---------------------------------------------------------------------------------------------------------
def _cond(x):
    return torch.arange(x.numel(), device=x.device).reshape(x.shape) % 3 == 0


WHERE = [
    lambda x: torch.where(_cond(x), x, x),
    lambda x: torch.where(_cond(x), torch.ones_like(x), torch.ones_like(x)),
    lambda x: torch.where(_cond(x), torch.zeros_like(x), torch.zeros_like(x)),
    lambda x: torch.where(_cond(x), torch.zeros_like(x.unsqueeze(0)), torch.zeros_like(x.unsqueeze(1))),
    lambda x: torch.where(_cond(x), torch.where(_cond(x), x, x), torch.where(_cond(x), x, x)),
]


@pytest.mark.parametrize("idx", range(len(WHERE)))
@pytest.mark.parametrize("dynamic", [False, True])
def test_where_with_equal_branches(caplog, infer_backend, idx, dynamic):
    with need_xpu_graph_logs():
        run(infer_backend, WHERE[idx], torch.randn(128, 64), dynamic=dynamic)
    if dynamic and idx == 3:  # the broadcast result shape would have to be written out
        assert "Pattern.FoldWhere changed graph" not in caplog.text
    else:
        assert "Pattern.FoldWhere changed graph" in caplog.text


@pytest.mark.parametrize("dynamic", [False, True])
def test_where_constant_branch_shrinks_to_one_element(caplog, infer_backend, dynamic):
    with need_xpu_graph_logs():
        run(infer_backend, lambda x: torch.where(x <= 0, torch.zeros_like(x), x), torch.randn(128, 64), dynamic=dynamic, exact=True)
        run(infer_backend, lambda x: torch.where(x <= 0, x, torch.full_like(x, 2.5)), torch.randn(128, 64), dynamic=dynamic, exact=True)
    assert caplog.text.count("Pattern.FoldWhere changed graph") >= 2


# ---- reductions over unit dims ------------------------------------------------------------------------------------
REDUCE = [
    lambda a: torch.sum(a, dim=1) + 100,
    lambda a: torch.sum(a.permute(2, 1, 0, 3), dim=1).reshape(-1) + 100,
    lambda a: torch.sum(a, dim=3, keepdim=True),
    lambda a: torch.sum(a, dim=1, keepdim=False),
    lambda a: torch.sum(a, dim=(1, 3), keepdim=False),
    lambda a: torch.sum(a, dim=(1, 3), keepdim=True),
    lambda a: torch.sum(torch.sum(a, dim=1, keepdim=True), dim=3, keepdim=True),
]


@pytest.mark.parametrize("idx", range(len(REDUCE)))
@pytest.mark.parametrize("dynamic", [False, True])
def test_sum_over_unit_dims(caplog, infer_backend, idx, dynamic):
    with need_xpu_graph_logs(), skip_xpu_graph_cache(infer_backend):
        run(infer_backend, REDUCE[idx], torch.randn(128, 1, 64, 1), dynamic=dynamic, exact=True)
    assert "Pattern.FoldReduce changed graph" in caplog.text


def test_sum_over_a_real_dim_is_kept(caplog, infer_backend):
    with need_xpu_graph_logs():
        run(infer_backend, lambda a: torch.sum(a, dim=(1, 2)), torch.randn(8, 1, 16, 1))
        run(infer_backend, lambda a: torch.sum(a, dim=1, dtype=torch.float64), torch.randn(8, 1, 16))
    assert "Pattern.FoldReduce changed graph" not in caplog.text


@pytest.mark.parametrize("dynamic", [False, True])
def test_sum_over_all_dims_of_a_one_element_tensor(caplog, infer_backend, dynamic):
    with need_xpu_graph_logs():
        run(infer_backend, lambda a: torch.sum(a, dim=None, keepdim=True), torch.randn(1, 1, 1, 1), dynamic=dynamic, exact=True)
    assert "Pattern.FoldReduce changed graph" in caplog.text


# ---- stack ---------------------------------------------------------------------------------------------------------
STACK = [
    (lambda a: torch.stack([a], dim=0), True),
    (lambda a: torch.stack([a.T], dim=0).reshape(-1), True),
    (lambda a: torch.stack([a], dim=1), True),
    (lambda a: torch.stack([a], dim=2), True),
    (lambda a: torch.stack(a.unbind()), True),
    (lambda a: torch.stack(a.unbind(dim=1), dim=1), True),
    (lambda a: torch.stack(a.unbind(dim=1)[:4], dim=1), False),  # not all the pieces
    (lambda a: torch.stack(a.unbind(dim=1), dim=0), False),  # put together along another dim
    (lambda a: torch.stack(a.unbind(dim=0)[::-1], dim=0), False),  # out of order
]


@pytest.mark.parametrize("idx", range(len(STACK)))
@pytest.mark.parametrize("dynamic", [False, True])
def test_stack_of_one_and_unbind_round_trips(caplog, infer_backend, idx, dynamic):
    fn, folds = STACK[idx]
    with need_xpu_graph_logs(), skip_xpu_graph_cache(infer_backend):
        run(infer_backend, fn, torch.randn(12, 6), dynamic=dynamic, exact=True)
    assert ("Pattern.FoldStack changed graph" in caplog.text) == folds


# ---- squeeze -------------------------------------------------------------------------------------------------------
SQUEEZE = [
    ("FoldSqueeze0", lambda a: a.squeeze(1).squeeze() + 1),
    ("FoldSqueeze0", lambda a: a.squeeze().squeeze(0) + 1),
    ("FoldSqueeze1", lambda a: a.unsqueeze(0).squeeze() + 1),
    ("FoldSqueeze1", lambda a: a.unsqueeze(2).squeeze(2) + 1),
    ("FoldSqueeze1", lambda a: a.unsqueeze(-1).squeeze(-1) + 1),
]


@pytest.mark.parametrize("idx", range(len(SQUEEZE)))
def test_squeeze_chains(caplog, infer_backend, idx):
    name, fn = SQUEEZE[idx]
    with need_xpu_graph_logs():
        run(infer_backend, fn, torch.randn(8, 1, 5, 1), exact=True)
    assert f"Pattern.{name} changed graph" in caplog.text


def test_squeeze_of_another_dim_is_kept(caplog, infer_backend):
    with need_xpu_graph_logs():
        run(infer_backend, lambda a: a.unsqueeze(0).squeeze(2) + 1, torch.randn(8, 1, 5), exact=True)
    assert "Pattern.FoldSqueeze1 changed graph" not in caplog.text


# ---- slice / slice_scatter / *_like / detach --------------------------------------------------------------------
@pytest.mark.parametrize("dynamic", [False, True])
def test_whole_range_slices(caplog, infer_backend, dynamic):
    def fn(a):
        b = a[:, 0:] + 1  # the whole of dim 1
        c = a[0:12] * 2  # the whole of dim 0 with an explicit end
        d = a[:, 1:]  # a real slice
        return b, c, d

    with need_xpu_graph_logs():
        run(infer_backend, fn, torch.randn(12, 6), dynamic=dynamic, exact=True)
    assert "Pattern.FoldSliceLike changed graph" in caplog.text


def test_slice_scatter_over_the_whole_base(caplog, infer_backend):
    def fn(a, b):
        full = torch.slice_scatter(a, b, dim=1, start=0, end=6)
        part = torch.slice_scatter(a, b[:, :3], dim=1, start=0, end=3)
        return full + 1, part + 1

    with need_xpu_graph_logs():
        run(infer_backend, fn, torch.randn(4, 6), torch.randn(4, 6), exact=True)
    assert "Pattern.FoldSliceLike changed graph" in caplog.text
    final = infer_backend.compiled_graphs[-1]
    assert sum(1 for n in final.graph.nodes if "slice_scatter" in str(n.target)) == 1  # the partial one stays


LIKE = [
    lambda a: torch.ones_like(a),
    lambda a: torch.zeros_like(a),
    lambda a: torch.full_like(a, 42),
    lambda a: torch.full_like(a, 42, dtype=torch.int32),
    lambda a: torch.full_like(a, 42, device="cpu"),
]


@pytest.mark.parametrize("idx", range(len(LIKE)))
def test_like_constructors_become_plain_constructors(caplog, infer_backend, idx):
    with need_xpu_graph_logs(), skip_xpu_graph_cache(infer_backend):
        run(infer_backend, LIKE[idx], torch.randn(128, 64), dynamic=True, exact=True)
    assert "Pattern.ChangeTensorLike changed graph" in caplog.text


def test_like_constructors_of_data_dependent_shapes(caplog, infer_backend):
    def fn(a):
        b = torch.sum(a, dim=1)
        outs = []
        for i in range(3):
            lo, hi = a[b >= i], a[b < i]
            outs.append(torch.concat([torch.zeros_like(lo), torch.ones_like(hi)], dim=0))
        return torch.stack(outs, dim=0)

    # one graph with unbacked sizes (this torch otherwise breaks the graph at every mask index and compiles nothing):
    # a size no graph node carries cannot be written out, so those constructors stay as they are -- values must agree
    with need_xpu_graph_logs(), skip_xpu_graph_cache(infer_backend), torch._dynamo.config.patch(capture_dynamic_output_shape_ops=True):
        run(infer_backend, fn, torch.randn(32, 8), dynamic=True, exact=True)
    assert "xpu_graph passes complete" in caplog.text


def test_constants_keep_the_layout_of_a_permuted_template(infer_backend):
    def fn(a):
        return torch.zeros_like(a.t()) + 1, torch.ones_like(a.t()), a.t() * torch.ones_like(a.t())

    a = torch.randn(6, 4)
    got = torch.compile(fn, backend=infer_backend)(a)
    for g, w in zip(got, fn(a)):
        assert g.stride() == w.stride() and torch.equal(g, w)
    torch._dynamo.reset()


def test_detach_disappears_in_inference(caplog, infer_backend):
    with need_xpu_graph_logs(), torch.no_grad():
        run(infer_backend, lambda a: a.detach() * 2 + a.detach(), torch.randn(8, 8), exact=True)
    assert "Pattern.FoldDetach changed graph" in caplog.text


# ---- hand-written GELU ---------------------------------------------------------------------------------------------
import math  # noqa: E402

GELUS = [
    ("none", lambda x: 0.5 * (1 + torch.erf(x / math.sqrt(2))) * x),
    ("none", lambda x: x * 0.5 * (torch.erf(x * (1 / math.sqrt(2))) + 1.0)),
    ("tanh", lambda x: 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))),
    ("tanh", lambda x: x * (1.0 + torch.tanh((x + x * x * x * 0.044715) * math.sqrt(2.0 / math.pi))) * 0.5),
]


@pytest.mark.parametrize("idx", range(len(GELUS)))
def test_hand_written_gelu_becomes_aten_gelu(caplog, infer_backend, idx):
    kind, fn = GELUS[idx]
    x = torch.randn(64, 32)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=infer_backend)(x)
    torch.testing.assert_close(got, fn(x), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(got, torch.nn.functional.gelu(x, approximate=kind), rtol=1e-5, atol=1e-6)
    assert "Pattern.Gelu changed graph" in caplog.text
    final = infer_backend.compiled_graphs[-1]
    calls = [n for n in final.graph.nodes if n.op == "call_function"]
    assert [str(n.target) for n in calls] == ["aten.gelu.default"]
    assert calls[0].kwargs.get("approximate", "none") == kind
    torch._dynamo.reset()


def test_near_gelu_is_left_alone(caplog, infer_backend):
    fns = [
        lambda x: 0.5 * (1 + torch.erf(x / 1.5)) * x,  # another divisor
        lambda x: 0.5 * (1 + torch.erf(x / math.sqrt(2))) * (x + 1),  # the gate multiplies something else
        lambda x: 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.05 * torch.pow(x, 3.0)))),  # another cubic weight
    ]
    with need_xpu_graph_logs():
        for fn in fns:
            run(infer_backend, fn, torch.randn(16, 8))
    assert "Pattern.Gelu changed graph" not in caplog.text


def test_recognised_gelu_becomes_the_dense_layers_activation():
    """On the mi355x target the dense pattern takes aten.gelu as its activation: a hand-written erf GELU behind a
    matmul + bias therefore ends in ONE dense call (the kernels refuse CPU tensors, so only the rewrite is checked)."""
    from xpu_graph_amd import OptLevel, Target

    def fn(x, w, b):
        z = torch.addmm(b, x, w)
        return 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(16, 64).to(bf), torch.randn(64, 128).to(bf), torch.randn(128).to(bf)]
    with pytest.raises(NotImplementedError), torch.no_grad():
        torch.compile(fn, backend=backend, dynamic=False)(*args)
    calls = [n for n in backend.compiled_graphs[-1].graph.nodes if n.op in ("call_module", "call_function")]
    assert [str(n.target) for n in calls] == ["custom_dense_layer_replacement"]
    assert calls[0].args[-1] == "gelu"
    torch._dynamo.reset()

