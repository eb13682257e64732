"""Graph rewrites that hand a sum or a copy to the kernel next to it (mi355x target, post-AOT stages), on fake
tensors: which nodes disappear, what the kernel call receives, and the cases that must be left alone."""
import operator

import torch
from torch._subclasses.fake_tensor import FakeTensorMode
from torch.fx.experimental.proxy_tensor import make_fx

import xpu_graph_amd.ops  # noqa: F401  (defines torch.ops.xpu_ops)
from xpu_graph_amd.passes.fake_prop import propagate_missing
from xpu_graph_amd.passes.patterns.targets.mi355x.sum_folds import FoldAddIntoDense, FoldAddIntoNormBackward, FoldCloneOfContiguous

bf16 = torch.bfloat16
xpu = torch.ops.xpu_ops
aten = torch.ops.aten


def trace(fn, *shapes_dtypes):
    mode = FakeTensorMode(allow_non_fake_inputs=True)
    with mode:
        args = [torch.empty(s, dtype=d) for s, d in shapes_dtypes]
    return make_fx(fn, tracing_mode="fake")(*args)


def to_fixed_point(pattern, gm):
    """As the pass manager does: fake values for the new nodes, then the pattern again, until nothing changes."""
    mode = next(n.meta["val"].fake_mode for n in gm.graph.nodes if n.op == "placeholder")
    while pattern.process(gm):
        propagate_missing(gm, mode)


def calls(gm, target):
    return [n for n in gm.graph.nodes if n.op == "call_function" and n.target is target]


def test_sum_of_three_projection_gradients_becomes_a_residual_chain():
    def fn(g1, g2, g3, w1, w2, w3):
        return xpu.dense(g1, w1, False, None, None, "none") + xpu.dense(g2, w2, False, None, None, "none") + xpu.dense(g3, w3, False, None, None, "none")

    gm = trace(fn, *[((64, 32), bf16)] * 3, *[((32, 48), bf16)] * 3)
    assert len(calls(gm, aten.add.Tensor)) == 2
    to_fixed_point(FoldAddIntoDense(), gm)
    gm.graph.lint()
    assert calls(gm, aten.add.Tensor) == []
    dense = calls(gm, xpu.dense.default)
    assert len(dense) == 3 and [d.args[4] is not None for d in dense] == [False, True, True]
    assert dense[2].args[4] is dense[1] and dense[1].args[4] is dense[0]


def test_residual_behind_a_reshape_and_on_either_side():
    def fn(h, x, w):
        y = xpu.dense(x.reshape(-1, 32), w, True, None, None, "none").reshape(2, 8, 48)
        return h + y

    gm = trace(fn, ((2, 8, 48), bf16), ((2, 8, 32), bf16), ((48, 32), bf16))
    assert FoldAddIntoDense().process(gm)
    gm.graph.lint()
    assert calls(gm, aten.add.Tensor) == []
    (dense,) = calls(gm, xpu.dense.default)
    res = dense.args[4]
    assert res.target is aten.reshape.default and res.args[1] == [16, 48]
    out = next(n for n in gm.graph.nodes if n.op == "output").args[0]
    assert out.target is aten.reshape.default and out.args[0] is dense


def test_dense_sum_is_kept_when_it_is_not_a_plain_residual():
    def act(h, x, w):
        return h + xpu.dense(x, w, False, None, None, "silu")  # the residual would go in before the activation

    def two_users(h, x, w):
        y = xpu.dense(x, w, False, None, None, "none")
        return h + y, y

    def broadcast(b, x, w):
        return xpu.dense(x, w, False, None, None, "none") + b

    def promoted(h, x, w):
        return h + xpu.dense(x, w, False, None, None, "none")

    for fn, first in ((act, ((16, 48), bf16)), (two_users, ((16, 48), bf16)), (broadcast, ((48,), bf16)), (promoted, ((16, 48), torch.float32))):
        gm = trace(fn, first, ((16, 32), bf16), ((32, 48), bf16))
        assert not FoldAddIntoDense().process(gm), fn.__name__


def test_gradient_sum_moves_into_the_norm_backward():
    def fn(x, w, gy, other):
        gx, gw = xpu.rms_norm_bwd(x, None, w, gy, None, 1e-6, True)
        return other + gx, gw

    gm = trace(fn, ((4, 8, 256), bf16), ((256,), bf16), ((4, 8, 256), bf16), ((4, 8, 256), bf16))
    assert FoldAddIntoNormBackward().process(gm)
    gm.graph.lint()
    assert calls(gm, aten.add.Tensor) == []
    (bwd,) = calls(gm, xpu.rms_norm_bwd.default)
    assert bwd.args[4].op == "placeholder" and bwd.args[4].name == "other_1"
    outs = next(n for n in gm.graph.nodes if n.op == "output").args[0]
    assert all(o.target is operator.getitem and o.args[0] is bwd for o in outs) and [o.args[1] for o in outs] == [0, 1]


def test_gradient_sum_moves_into_the_layer_norm_backward():
    def fn(x, w, gy, other):
        gx, gw, gb = xpu.layer_norm_bwd(x, None, w, gy, None, 1e-5, True, True)
        return gx + other, gw, gb

    gm = trace(fn, ((4, 8, 256), bf16), ((256,), bf16), ((4, 8, 256), bf16), ((4, 8, 256), bf16))
    assert FoldAddIntoNormBackward().process(gm)
    gm.graph.lint()
    assert calls(gm, aten.add.Tensor) == []
    (bwd,) = calls(gm, xpu.layer_norm_bwd.default)
    assert bwd.args[4].name == "other_1" and bwd.args[5:] == (1e-5, True, True)


def test_norm_backward_that_already_adds_a_gradient_is_left_alone():
    def fn(x, w, gy, gh, other):
        gx, _ = xpu.rms_norm_bwd(x, None, w, gy, gh, 1e-6, False)
        return other + gx

    gm = trace(fn, ((8, 256), bf16), ((256,), bf16), *[((8, 256), bf16)] * 3)
    assert not FoldAddIntoNormBackward().process(gm)


def test_copy_of_a_value_that_is_already_contiguous_is_dropped():
    def fn(x, w):
        y = xpu.dense(x, w, False, None, None, "none").reshape(2, 8, 4, 12)  # [B, S, H, D] storage
        t = y.transpose(1, 2)                                                   # what attention hands on
        return t.transpose(1, 2).clone(memory_format=torch.contiguous_format).reshape(16, 48) * 2

    gm = trace(fn, ((16, 32), bf16), ((32, 48), bf16))
    assert len(calls(gm, aten.clone.default)) == 1
    assert FoldCloneOfContiguous().process(gm)
    gm.graph.lint()
    assert calls(gm, aten.clone.default) == []


def test_copies_that_must_stay():
    def of_input(x):
        return x.clone() * 2  # the storage belongs to the caller

    def strided(x, w):
        return xpu.dense(x, w, False, None, None, "none").t().clone(memory_format=torch.contiguous_format)

    def both_returned(x, w):
        y = xpu.dense(x, w, False, None, None, "none")
        return y, y.clone()  # the caller may write into one of them

    gm = trace(of_input, ((16, 32), bf16))
    assert not FoldCloneOfContiguous().process(gm)
    for fn in (strided, both_returned):
        gm = trace(fn, ((16, 32), bf16), ((32, 48), bf16))
        assert not FoldCloneOfContiguous().process(gm), fn.__name__


def test_saved_activations_of_a_forward_graph_may_share_storage():
    def fn(x, w):
        y = xpu.dense(x, w, False, None, None, "none")
        c = y.clone()
        return c.sum(), y, c  # one result for the caller, two values saved for the backward

    gm = trace(fn, ((16, 32), bf16), ((32, 48), bf16))
    assert not FoldCloneOfContiguous().process(gm)  # without knowing which results the caller sees, every one counts
    gm.meta["xg_user_outputs"] = 1
    assert FoldCloneOfContiguous().process(gm)
    assert calls(gm, aten.clone.default) == []


def test_a_returned_copy_never_shares_storage_with_a_saved_activation():
    """The caller may write into a result between forward and backward (legal in eager): a copy it sees stays a copy
    when its source is saved for the backward, and the other way round."""

    def returned_copy(x, w):
        y = xpu.dense(x, w, False, None, None, "none")
        return y.clone(), y  # result for the caller, source saved

    def returned_source(x, w):
        y = xpu.dense(x, w, False, None, None, "none")
        return y, y.clone()  # source for the caller, copy saved

    for fn in (returned_copy, returned_source):
        gm = trace(fn, ((16, 32), bf16), ((32, 48), bf16))
        gm.meta["xg_user_outputs"] = 1
        assert not FoldCloneOfContiguous().process(gm), fn.__name__
        assert len(calls(gm, aten.clone.default)) == 1
