"""Graph rewriting for the mi355x target, checked on the CPU: which patterns
fire and what the rewritten graph calls.  The rewritten graphs are not run
here -- on CPU tensors the xpu_ops have no implementation and must raise."""
import math
import operator

import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig, mi355x_compiler
from xpu_graph_amd.test_utils import need_xpu_graph_logs

bf16 = torch.bfloat16


@pytest.fixture()
def backend():
    return mi355x_compiler()


def rewrite(backend, fn, *args, must_fail=True):
    """Compile fn for the mi355x target on CPU inputs; returns the rewritten graph."""
    with need_xpu_graph_logs():
        c = torch.compile(fn, backend=backend)
        if must_fail:
            with pytest.raises(NotImplementedError):  # no CPU fallback behind the custom ops
                c(*args)
        else:
            c(*args)
    return backend.compiled_graphs[-1]


def modules_called(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_module"]


def aten_ops(gm):
    return [str(n.target) for n in gm.graph.nodes if n.op == "call_function" and n.target is not operator.getitem]


def test_c1_rmsnorm_becomes_one_custom_call(caplog, backend):
    def fn(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

    gm = rewrite(backend, fn, torch.randn(8, 64), torch.randn(64))
    assert modules_called(gm) == ["custom_rms_norm"] and aten_ops(gm) == []
    assert "Pattern.CustomRMSNorm changed graph" in caplog.text


def test_unweighted_rmsnorm_stays_default(caplog, backend):
    def fn(x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)

    gm = rewrite(backend, fn, torch.randn(8, 64), must_fail=False)
    assert modules_called(gm) == ["fused_rms_norm"]  # CustomRMSNorm needs a weight


@pytest.mark.parametrize("form", ["library", "decomposed"])
def test_c2_add_layernorm_two_outputs(caplog, backend, form):
    def library(x, r, g, b):
        h = x + r
        return F.layer_norm(h, (h.shape[-1],), g, b, 1e-5), h

    def decomposed(x, r, g, b):
        h = x + r
        hf = h.float()
        n = ((hf - hf.mean(-1, keepdim=True)) * torch.rsqrt(hf.var(-1, unbiased=False, keepdim=True) + 1e-5)).to(h.dtype)
        return n * g + b, h

    args = (torch.randn(8, 64).to(bf16), torch.randn(8, 64).to(bf16), torch.randn(64).to(bf16), torch.randn(64).to(bf16))
    gm = rewrite(backend, {"library": library, "decomposed": decomposed}[form], *args)
    assert modules_called(gm) == ["mi355x_fused_add_norm"] and aten_ops(gm) == []
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert node.args[6] is True and node.args[7] == "layer_norm" and node.args[5] == 1e-5
    assert "Pattern.FusedAddLayerNorm changed graph" in caplog.text


def test_add_rmsnorm_single_output_when_sum_is_private(caplog, backend):
    def fn(x, r, w):
        h = (x + r).float()
        return (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype) * w

    args = (torch.randn(4, 32).to(bf16), torch.randn(4, 32).to(bf16), torch.randn(32).to(bf16))
    gm = rewrite(backend, fn, *args)
    assert modules_called(gm) == ["mi355x_fused_add_norm"]
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert node.args[6] is False and node.args[7] == "rms_norm"
    assert "Pattern.FusedAddRMSNorm changed graph" in caplog.text


def test_add_norm_sum_used_before_norm_keeps_topological_order(backend):
    def fn(x, r, g, b):
        h = x + r
        side = h * 2  # a user of the sum that precedes the norm in graph order
        return F.layer_norm(h, (h.shape[-1],), g, b, 1e-5), side

    args = (torch.randn(4, 32), torch.randn(4, 32), torch.randn(32), torch.randn(32))
    gm = rewrite(backend, fn, *args)
    gm.graph.lint()
    assert modules_called(gm) == ["mi355x_fused_add_norm"]


def test_c3_slice_cat_and_addn(caplog, backend):
    offs = [7, 100, 40, 200]

    def fn(src, *ts):
        cat = torch.cat([src[:, o : o + 8] for o in offs], dim=1)
        acc = ts[0]
        for t in ts[1:]:
            acc = acc + t
        return cat, acc

    ts = [torch.randn(6, 16) for _ in range(6)]
    gm = rewrite(backend, fn, torch.randn(6, 256), *ts)
    assert sorted(modules_called(gm)) == ["fuse_slice_cat", "mi355x_addn"]
    assert "aten.slice.Tensor" not in aten_ops(gm) and "aten.stack.default" not in aten_ops(gm)
    node = next(n for n in gm.graph.nodes if n.target == "fuse_slice_cat")
    assert node.args[1] == [(o, o + 8) for o in offs]
    for p in ("FusedCatSlice", "FusedAddN", "FusedStackSumToAddN", "FoldCat"):
        assert f"Pattern.{p} changed graph" in caplog.text, p


def test_slice_cat_mixed_inputs_int64max_and_negative_end(backend):
    def fn(src, other):
        return torch.cat([other, src[:, 3:9], src[:, 20:], src[:, 10:-200], other], dim=-1)

    gm = rewrite(backend, fn, torch.randn(4, 256), torch.randn(4, 5))
    node = next(n for n in gm.graph.nodes if n.target == "fuse_slice_cat")
    assert node.args[1] == [(3, 9), (20, 256), (10, 56)]
    cat = next(n for n in gm.graph.nodes if n.op == "call_function" and "cat" in str(n.target))
    assert len(cat.args[0]) == 3


def test_slice_cat_not_fused_along_rows_or_3d(caplog, backend):
    def rows(src):
        return torch.cat([src[0:2], src[4:6]], dim=0)

    def cube(src):
        return torch.cat([src[:, :, 0:2], src[:, :, 4:6]], dim=2)

    rewrite(backend, rows, torch.randn(8, 8), must_fail=False)
    rewrite(backend, cube, torch.randn(2, 8, 8), must_fail=False)
    assert "Pattern.FusedCatSlice changed graph" not in caplog.text


def test_fused_slice_groups_by_source_and_width(caplog, backend):
    """>= 3 equally wide last-dim slices of one source become one gather; the slabs are taken with select
    (reference tests/mlu/test_fuse_slice.py:24-33: two widths -> two modules)."""

    def fn(x):
        a = [x[:, s : s + 64] + 1 for s in (0, 64, 128, 192)]
        b = [x[:, s : s + 128] * 2 for s in (256, 384, 512)]
        return a + b + [x[:, 700:710] + 1]

    gm = rewrite(backend, fn, torch.randn(6, 1024))
    mods = modules_called(gm)
    assert mods == ["fused_slice_0", "fused_slice_1"]
    assert gm.get_submodule("fused_slice_0").slices_index == [0, 64, 128, 192]
    assert gm.get_submodule("fused_slice_1").slices_index == [256, 384, 512]
    calls = {n.target: n for n in gm.graph.nodes if n.op == "call_module"}
    assert calls["fused_slice_0"].args[1] == 64 and calls["fused_slice_1"].args[1] == 128
    assert tuple(calls["fused_slice_1"].meta["val"].shape) == (3, 6, 128)
    assert aten_ops(gm).count("aten.select.int") == 7 and aten_ops(gm).count("aten.slice.Tensor") == 1
    assert "Pattern.FusedSlice changed graph" in caplog.text


def test_fused_slice_3d_source_and_open_ends(backend):
    def fn(x):
        return [x[:, :, s:e] + 1 for s, e in ((0, 4), (-4, None), (10, 14), (20, -76))]

    gm = rewrite(backend, fn, torch.randn(2, 3, 100))
    (name,) = modules_called(gm)
    assert gm.get_submodule(name).slices_index == [0, 96, 10, 20]
    call = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert tuple(call.meta["val"].shape) == (4, 2, 3, 4)


def test_fused_slice_vetoes(caplog, backend):
    def two(x):  # fewer than three of one width
        return x[:, 0:8] + 1, x[:, 8:16] + 1, x[:, 16:32] + 1

    def views_only(x):  # slices that only feed the output stay views
        return x[:, 0:8], x[:, 8:16], x[:, 16:24]

    def rows(x):  # not the last dim
        return x[0:2] + 1, x[2:4] + 1, x[4:6] + 1

    def stepped(x):
        return x[:, 0:8:2] + 1, x[:, 8:16:2] + 1, x[:, 16:24:2] + 1

    for fn in (two, views_only, rows, stepped):
        rewrite(backend, fn, torch.randn(8, 64), must_fail=False)
    assert "Pattern.FusedSlice changed graph" not in caplog.text


def test_slice_sum_cat_run_inside_a_cat(caplog, backend):
    """>= 3 consecutive sum(dim 1) of row slices of one 3-D tensor among a cat's inputs become one call; the other
    inputs stay (reference tests/mlu/test_slice_sum_cat.py:13-41)."""
    params = [(0, 2), (0, 4), (0, 8), (0, 16)]

    def fn(x, other):
        sums = [torch.sum(x[:, a:b, :], dim=[1]) for a, b in params]
        return torch.cat([other] + sums + [other], dim=1)

    gm = rewrite(backend, fn, torch.randn(6, 32, 32), torch.randn(6, 32))
    (name,) = modules_called(gm)
    assert name == "mi355x_slice_sum_cat_0" and gm.get_submodule(name).slice_param == params
    call = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert tuple(call.meta["val"].shape) == (6, 4 * 32)
    cat = next(n for n in gm.graph.nodes if n.op == "call_function" and "cat" in str(n.target))
    assert len(cat.args[0]) == 3 and cat.args[0][1] is call
    assert "aten.sum.dim_IntList" not in aten_ops(gm) and "aten.slice.Tensor" not in aten_ops(gm)
    assert "Pattern.FusedCatSum changed graph" in caplog.text


def test_slice_sum_cat_alone_and_vetoes(caplog, backend):
    def whole(x):  # the run is the whole cat: no cat is left
        return torch.cat([x[:, a:b, :].sum(1) for a, b in ((1, 3), (0, 4), (2, 8))], dim=-1)

    gm = rewrite(backend, whole, torch.randn(5, 8, 16))
    assert modules_called(gm) == ["mi355x_slice_sum_cat_0"] and aten_ops(gm) == []
    assert gm.get_submodule("mi355x_slice_sum_cat_0").slice_param == [(1, 3), (0, 4), (2, 8)]
    caplog.clear()

    def two(x):
        return torch.cat([x[:, 0:2, :].sum(1), x[:, 0:4, :].sum(1)], dim=1)

    def keepdim(x):
        return torch.cat([x[:, 0:a, :].sum(1, keepdim=True) for a in (2, 4, 6)], dim=-1)

    def other_dim(x):
        return torch.cat([x[:, :, 0:a].sum(2) for a in (2, 4, 6)], dim=1)

    def shared(x):  # a slice with a second user must survive
        s = x[:, 0:2, :]
        return torch.cat([s.sum(1), x[:, 0:4, :].sum(1), x[:, 0:6, :].sum(1)], dim=1), s

    for fn in (two, keepdim, other_dim, shared):
        rewrite(backend, fn, torch.randn(5, 8, 16), must_fail=False)
    assert "Pattern.FusedCatSum changed graph" not in caplog.text


def test_multiple_slice_cats_share_one_multi_output_module(caplog, backend):
    def fn(src):
        a = torch.cat([src[:, 0:4], src[:, 8:12]], dim=1)
        b = torch.cat([src[:, 16:20], src[:, 4:8], src[:, 30:32]], dim=1)
        return a, b

    gm = rewrite(backend, fn, torch.randn(4, 64))
    mods = modules_called(gm)
    assert len(mods) == 1 and mods[0].startswith("fuse_slice_cat_v2")
    assert "Pattern.FusedMultipleSliceCat changed graph" in caplog.text
    sub = gm.get_submodule(mods[0])
    assert sub.many_slices == [[(0, 4), (8, 12)], [(16, 20), (4, 8), (30, 32)]]


def test_slice_stack_sum_and_combo_sum(caplog, backend):
    def fn(src):
        a = torch.stack([src[:, 0:8], src[:, 8:16], src[:, 32:40]], dim=0).sum(dim=0)
        b = torch.stack([src[:, 40:48], src[:, 16:24]], dim=0).sum(dim=0)
        return a, b

    gm = rewrite(backend, fn, torch.randn(4, 64))
    assert "Pattern.FusedSliceStackSum changed graph" in caplog.text
    assert "Pattern.ComboSum3dInp changed graph" in caplog.text
    assert "combo_sum" in modules_called(gm)


@pytest.mark.parametrize("form", ["mm_add", "linear", "nobias", "relu"])
def test_c4_dense(caplog, backend, form):
    x = torch.randn(16, 64).to(bf16)
    if form == "mm_add":
        fn, args = (lambda x, w, b: F.silu(x @ w + b)), (x, torch.randn(64, 32).to(bf16), torch.randn(32).to(bf16))
    elif form == "linear":
        fn, args = (lambda x, w, b: F.silu(F.linear(x, w, b))), (x, torch.randn(32, 64).to(bf16), torch.randn(32).to(bf16))
    elif form == "nobias":
        fn, args = (lambda x, w: x @ w), (x, torch.randn(64, 32).to(bf16))
    else:
        fn, args = (lambda x, w, b: F.relu(torch.addmm(b, x, w))), (x, torch.randn(64, 32).to(bf16), torch.randn(16, 32).to(bf16))
    gm = rewrite(backend, fn, *args)
    assert modules_called(gm) == ["custom_dense_layer_replacement"]
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert node.args[2] is (form == "linear")
    assert node.args[4] == {"mm_add": "silu", "linear": "silu", "nobias": "none", "relu": "relu"}[form]
    assert "Pattern.CustomDenseLayer changed graph" in caplog.text


def test_dense_constraint_vetoes_odd_sizes_and_takes_fp32(caplog, backend):
    """16-byte operand loads: K a multiple of 8 for 16-bit types and of 4 for fp32; N a multiple of 8.  fp32 layers
    (the dtype of the reference's dense-layer tests, tests/mlu/test_custom_denselayer.py:11) go to the fp32 MFMA kernel."""
    rewrite(backend, lambda x, w: x @ w, torch.randn(8, 12).to(bf16), torch.randn(12, 8).to(bf16), must_fail=False)
    rewrite(backend, lambda x, w: x @ w, torch.randn(8, 6), torch.randn(6, 8), must_fail=False)
    rewrite(backend, lambda x, w: x @ w, torch.randn(8, 16), torch.randn(16, 12), must_fail=False)
    rewrite(backend, lambda x, w: x @ w, torch.randn(8, 16, dtype=torch.float64), torch.randn(16, 8, dtype=torch.float64), must_fail=False)
    assert "Pattern.CustomDenseLayer changed graph" not in caplog.text
    gm = rewrite(backend, lambda x, w, b: torch.relu(x @ w + b), torch.randn(8, 12), torch.randn(12, 8), torch.randn(8))
    assert modules_called(gm) == ["custom_dense_layer_replacement"]
    assert "Pattern.CustomDenseLayer changed graph" in caplog.text


def test_swiglu_both_forms(caplog, backend):
    def halves(x):
        d = x.shape[-1] // 2
        return F.silu(x[..., :d]) * x[..., d:]

    def pair(a, b):
        return F.silu(a) * b

    gm = rewrite(backend, halves, torch.randn(4, 64).to(bf16))
    assert modules_called(gm) == ["mi355x_silu_mul"]
    gm = rewrite(backend, pair, torch.randn(4, 32).to(bf16), torch.randn(4, 32).to(bf16))
    assert modules_called(gm) == ["mi355x_silu_mul2"]
    assert "Pattern.FusedSwiGLU changed graph" in caplog.text


def _eager_causal_attention(q, k, v):
    S, D = q.shape[-2], q.shape[-1]
    w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(D)
    w = w + torch.full((S, S), float("-inf"), dtype=q.dtype).triu(1)
    w = torch.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(w, v)


def test_c5_causal_attention_recognised(caplog, backend):
    q, k, v = (torch.randn(2, 4, 32, 64).to(bf16) for _ in range(3))
    gm = rewrite(backend, _eager_causal_attention, q, k, v)
    assert "Pattern.FusedSDPA changed graph" in caplog.text
    assert "Pattern.FusedCausalSDPA changed graph" in caplog.text
    node = next(n for n in gm.graph.nodes if n.target == "mi355x_sdpa")
    assert node.args[3] is True and abs(node.args[4] - 1 / 8) < 1e-12
    # q, k, v reach the kernel as the caller's 4-D tensors: no clones, no mask, no softmax left
    assert all(a.op == "placeholder" for a in node.args[:3])
    assert not any(s in " ".join(aten_ops(gm)) for s in ("softmax", "full", "triu", "clone", "bmm"))


def test_library_sdpa_is_causal_flag(caplog, backend):
    q, k, v = (torch.randn(2, 4, 32, 64).to(bf16) for _ in range(3))
    gm = rewrite(backend, lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True), q, k, v)
    node = next(n for n in gm.graph.nodes if n.target == "mi355x_sdpa")
    assert node.args[3] is True


def test_arbitrary_mask_travels_as_an_operand_and_an_unusable_one_is_not_taken(caplog, backend):
    def fn(q, k, v, m):
        w = torch.matmul(q, k.transpose(2, 3)) / 8.0 + m
        return torch.matmul(torch.softmax(w, dim=-1), v)

    q, k, v = (torch.randn(2, 4, 32, 64).to(bf16) for _ in range(3))
    gm = rewrite(backend, fn, q, k, v, torch.randn(32, 32).to(bf16))  # a run-time mask: the kernel adds it
    assert modules_called(gm) == ["mi355x_sdpa_masked"]
    assert "aten.scaled_dot_product_attention.default" not in aten_ops(gm)
    # an integer bias is not an attention mask the fused op accepts: no attention call (the two products go to the
    # batched dense kernel instead)
    gm = rewrite(backend, fn, q, k, v, torch.randint(-3, 1, (32, 32)))
    assert not any(m.startswith("mi355x_sdpa") for m in modules_called(gm))
    assert "aten.scaled_dot_product_attention.default" not in aten_ops(gm)


def test_target_none_has_no_structure_patterns(caplog):
    be = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, target=Target.none))
    names = [str(p) for ps in be.get_pattern_manager()._patterns.values() for p in ps]
    assert "CustomRMSNorm" not in names and "FusedCatSlice" not in names and "FusedSwiGLU" not in names
    be2 = mi355x_compiler()
    names2 = [str(p) for ps in be2.get_pattern_manager()._patterns.values() for p in ps]
    for want in ("CustomRMSNorm", "CustomLayerNorm", "FusedCatSlice", "FusedMultipleSliceCat", "FusedSliceStackSum",
                 "ComboSum3dInp", "CustomDenseLayer", "FusedAddLayerNorm", "FusedAddRMSNorm", "FusedSwiGLU",
                 "FusedStackSumToAddN", "FusedCausalSDPA", "NativeNormToDefault"):
        assert want in names2, want


def _rope_fn(q, cos, sin):
    d = q.shape[-1] // 2
    return q * cos + torch.cat([-q[..., d:], q[..., :d]], dim=-1) * sin


def test_rope_rotate_half_becomes_one_call(caplog, backend):
    q = torch.randn(2, 16, 4, 64).to(bf16).transpose(1, 2)  # [B, H, S, D] view of [B, S, H, D] storage
    cos, sin = torch.randn(16, 64).to(bf16), torch.randn(16, 64).to(bf16)
    gm = rewrite(backend, _rope_fn, q, cos, sin)
    assert modules_called(gm) == ["mi355x_rope"] and aten_ops(gm) == []
    assert "Pattern.FusedRoPE changed graph" in caplog.text
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert node.meta["val"].stride() == q.stride()  # written in the layout it was read in


def test_rope_not_taken_for_other_rotations_or_mixed_dtypes(caplog, backend):
    q = torch.randn(2, 4, 16, 64).to(bf16)
    cos, sin = torch.randn(16, 64).to(bf16), torch.randn(16, 64).to(bf16)

    def quarter(q, cos, sin):  # rotates by a quarter of the head dim: not the rotate-half form
        return q * cos + torch.cat([-q[..., 16:], q[..., :16]], dim=-1) * sin

    def no_neg(q, cos, sin):
        return q * cos + torch.cat([q[..., 32:], q[..., :32]], dim=-1) * sin

    for fn, args in ((quarter, (q, cos, sin)), (no_neg, (q, cos, sin)), (_rope_fn, (q, cos.float(), sin.float())), (_rope_fn, (q, cos[None].expand(2, 16, 64)[:, None], sin[None].expand(2, 16, 64)[:, None]))):
        gm = rewrite(backend, fn, *args, must_fail=False)
        assert "mi355x_rope" not in modules_called(gm)


def test_llama_block_graph_has_no_layout_copies(backend):
    """q / k go through rope in the projection's own layout, attention writes [B, S, H, D], so the transposes
    around it are views and the contiguous() copy in front of the output projection disappears; the rotary
    tables are folded to constants."""
    from oracle import eager, inputs

    for batch in (1, 3):  # with a batch, the traced batched matmuls carry extra contiguous copies of q, k^T and v
        torch._dynamo.reset()  # a recompile for a new batch size would otherwise trace the batch as a symbol
        x, p = inputs.c5_llama_block(B=batch, S=32, hidden=512, inter=256, device="cpu")
        names = sorted(p)

        def fn(x, *ws):
            return eager.llama_block_eager(x, dict(zip(names, ws)), n_heads=8)

        gm = rewrite(mi355x_compiler(), fn, x, *[p[n] for n in names])
        mods = modules_called(gm)
        assert mods.count("mi355x_rope") == 2 and "mi355x_sdpa" in mods
        assert mods.count("mi355x_dense_glu") == 1 and "mi355x_silu_mul2" not in mods
        left = aten_ops(gm)
        assert not any(k in t for t in left for k in ("clone", "cat", "neg", "cos", "sin", "arange", "softmax", "aten.mm", "aten.bmm")), left


def test_activation_behind_the_reshape_of_a_linear_layer_joins_the_dense_call(backend):
    """A linear layer on [B, S, H] input is view -> addmm -> view; the activation that follows commutes with the view
    and goes into the dense epilogue."""

    def fn(x, w, b):
        return F.silu(F.linear(x, w, b)) + 1

    gm = rewrite(backend, fn, torch.randn(2, 8, 128).to(bf16), torch.randn(96, 128).to(bf16), torch.randn(96).to(bf16))
    assert modules_called(gm) == ["custom_dense_layer_replacement"]
    call = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert call.args[4] == "silu" and not any("silu" in t for t in aten_ops(gm))
    out = next(n for n in gm.graph.nodes if n.op == "output").args[0][0]
    assert tuple(out.meta["val"].shape) == (2, 8, 96)


def test_gate_and_up_projections_become_one_gated_dense(caplog, backend):
    def mlp(x, wg, wu):
        return F.silu(F.linear(x, wg)) * F.linear(x, wu)

    x = torch.randn(2, 8, 128).to(bf16)
    wg, wu = torch.randn(96, 128).to(bf16), torch.randn(96, 128).to(bf16)
    gm = rewrite(backend, mlp, x, wg, wu)
    assert modules_called(gm) == ["mi355x_dense_glu"]
    call = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert tuple(call.meta["val"].shape) == (16, 96)
    out = next(n for n in gm.graph.nodes if n.op == "output").args[0][0]
    assert tuple(out.meta["val"].shape) == (2, 8, 96)
    assert "Pattern.FusedDenseGLU changed graph" in caplog.text


def test_gated_dense_vetoes(caplog, backend):
    def k_not_slab(x, wg, wu):  # K = 96 is not a multiple of 64: no gated kernel for it
        return F.silu(F.linear(x, wg)) * F.linear(x, wu)

    def different_inputs(x, y, wg, wu):
        return F.silu(F.linear(x, wg)) * F.linear(y, wu)

    def shared_gate(x, wg, wu):  # the gate projection has a second user
        g = F.linear(x, wg)
        return F.silu(g) * F.linear(x, wu), g

    def kn_weights(x, wg, wu):  # [K, N] weights
        return F.silu(x @ wg) * (x @ wu)

    w = lambda *s: torch.randn(*s).to(bf16)  # noqa: E731
    rewrite(backend, k_not_slab, w(16, 96), w(32, 96), w(32, 96))
    rewrite(backend, different_inputs, w(16, 128), w(16, 128), w(32, 128), w(32, 128))
    rewrite(backend, shared_gate, w(16, 128), w(32, 128), w(32, 128))
    rewrite(backend, kn_weights, w(16, 128), w(128, 32), w(128, 32))
    assert "Pattern.FusedDenseGLU changed graph" not in caplog.text


def test_residual_add_moves_into_the_dense_epilogue(caplog, backend):
    def fn(x, w, r):
        return F.linear(x, w).view(2, 8, 32) + r  # output projection, reshaped, plus residual

    x, w, r = torch.randn(16, 64).to(bf16), torch.randn(32, 64).to(bf16), torch.randn(2, 8, 32).to(bf16)
    gm = rewrite(backend, fn, x, w, r)
    assert "Pattern.FusedDenseResidual changed graph" in caplog.text
    assert modules_called(gm) == ["custom_dense_layer_replacement"] and "aten.add.Tensor" not in aten_ops(gm)
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert tuple(node.args[3].meta["val"].shape) == (16, 32)  # the residual, viewed as [M, N]


def test_residual_not_fused_when_dense_has_other_users_or_an_activation(backend):
    def two_users(x, w, r):
        y = F.linear(x, w)
        return y + r, y

    def activated(x, w, r):
        return F.silu(F.linear(x, w)) + r

    x, w, r = torch.randn(16, 64).to(bf16), torch.randn(32, 64).to(bf16), torch.randn(16, 32).to(bf16)
    for fn in (two_users, activated):
        gm = rewrite(mi355x_compiler(), fn, x, w, r)
        assert "aten.add.Tensor" in aten_ops(gm)
        torch._dynamo.reset()


@pytest.mark.parametrize("form", ["bmm", "bmm_act", "bmm_bias", "baddbmm", "residual", "w_trans"])
def test_batch_dense_layer(caplog, backend, form):
    """bmm (+ bias | residual) (+ activation) -> one batched dense call
    (reference tests/mlu/test_custom_batchdenselayer.py; structure/custom_denselayer.py:102-128)."""
    B, M, K, N = 3, 16, 64, 32
    x = torch.randn(B, M, K).to(bf16)
    w = torch.randn(B, K, N).to(bf16)
    wt = torch.randn(B, N, K).to(bf16)
    bias = torch.randn(B, 1, N).to(bf16)
    res = torch.randn(B, M, N).to(bf16)
    fns = {
        "bmm": (lambda x, w: torch.bmm(x, w), (x, w), False, "none"),
        "bmm_act": (lambda x, w: F.gelu(torch.bmm(x, w)), (x, w), False, "gelu"),
        "bmm_bias": (lambda x, w, b: F.silu(torch.bmm(x, w) + b), (x, w, bias), False, "silu"),
        "baddbmm": (lambda x, w, b: torch.baddbmm(b, x, w), (x, w, bias), False, "none"),
        "residual": (lambda x, w, r: torch.bmm(x, w) + r, (x, w, res), False, "none"),
        "w_trans": (lambda x, w: torch.relu(torch.bmm(x, w.transpose(1, 2))), (x, wt), True, "relu"),
    }
    fn, args, trans, act = fns[form]
    gm = rewrite(backend, fn, *args)
    assert "Pattern.CustomBatchDenseLayer changed graph" in caplog.text
    assert modules_called(gm) == ["custom_batch_dense_layer_replacement"]
    assert not any(k in t for t in aten_ops(gm) for k in ("bmm", "gelu", "silu", "relu", "aten.add"))
    node = next(n for n in gm.graph.nodes if n.op == "call_module")
    assert node.args[2] is trans and node.args[4] == act
    assert (node.args[3] is None) == (len(args) == 2)


def test_batch_dense_layer_vetoes(backend):
    x32, w32 = torch.randn(2, 8, 16), torch.randn(2, 16, 8)
    gm = rewrite(mi355x_compiler(), lambda x, w: torch.bmm(x, w), x32, w32, must_fail=False)  # fp32 stays on Aten
    assert modules_called(gm) == []
    torch._dynamo.reset()
    x, w = torch.randn(2, 8, 12).to(bf16), torch.randn(2, 12, 8).to(bf16)  # K not a multiple of 8
    gm = rewrite(mi355x_compiler(), lambda x, w: torch.bmm(x, w), x, w, must_fail=False)
    assert modules_called(gm) == []
    torch._dynamo.reset()
    # a batch beyond one launch's grid (65535 entries) still fuses: the op wrapper sends it out in slices
    x, w = torch.randn(70000, 8, 8).to(bf16), torch.randn(70000, 8, 8).to(bf16)
    gm = rewrite(mi355x_compiler(), lambda x, w: torch.bmm(x, w), x, w)
    assert len(modules_called(gm)) == 1


def test_tanh_gelu_is_not_taken_for_the_erf_gelu_of_the_dense_kernel():
    """aten.gelu(approximate="tanh") behind a matmul stays an Aten op: the dense epilogue evaluates the erf form."""
    import torch.nn.functional as F

    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

    def fn(x, w, w2, b):
        return F.gelu(torch.addmm(b, x, w), approximate="tanh"), F.gelu(torch.addmm(b, x, w2))

    bf = torch.bfloat16
    backend = XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [torch.randn(16, 64).to(bf), torch.randn(64, 128).to(bf), torch.randn(64, 128).to(bf), torch.randn(128).to(bf)]
    with pytest.raises(NotImplementedError), torch.no_grad():
        torch.compile(fn, backend=backend, dynamic=False)(*args)
    calls = [n for n in backend.compiled_graphs[-1].graph.nodes if n.op in ("call_module", "call_function")]
    acts = sorted(n.args[-1] for n in calls if n.op == "call_module")
    assert acts == ["gelu", "none"]
    assert sum(1 for n in calls if "aten.gelu" in str(n.target)) == 1
    torch._dynamo.reset()


def test_slice_bounds_past_the_source_are_clamped_like_eager():
    """x[:, 5:10000] and x[:, -10000:3] are legal eager slices; the fused slice/cat must see the clamped ranges."""
    from xpu_graph_amd.passes.patterns.structure.slice_cat import slice_run_params

    def fn(x):
        return torch.cat([x[:, 5:10000], x[:, -10000:3], x[:, 7:7], x[:, 2:6]], dim=1)

    gm = torch.fx.experimental.proxy_tensor.make_fx(fn)(torch.randn(4, 16))
    slices = [n for n in gm.graph.nodes if n.op == "call_function" and n.target == torch.ops.aten.slice.Tensor and n.args[1] == 1]
    src, params = slice_run_params(slices)
    assert params == [(5, 16), (0, 3), (7, 7), (2, 6)]


def test_repeated_gather_index_becomes_a_broadcast_view(caplog):
    """reference tests/mlu/test_repeat_to_expand.py:8-38: arange -> expand -> unsqueeze -> repeat -> gather."""

    def fn(x, n):
        idx = torch.arange(n).reshape(1, -1).expand(x.shape[0], -1)
        idx = idx.unsqueeze(-1).repeat(1, 1, x.shape[2])
        return x.gather(index=idx, dim=1)

    def real_repeat(x, idx):
        return x.gather(index=idx.repeat(2, 1, 1), dim=1)  # copies along a real axis: must stay

    backend = XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level1, enable_cache=False))
    x = torch.randn(12, 40, 16)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend, dynamic=True)(x, 9)
    assert torch.equal(got, fn(x, 9))
    assert "Pattern.FusedGatherToCopy changed graph" in caplog.text
    assert not any("repeat" in str(n.target) for n in backend.compiled_graphs[-1].graph.nodes)
    caplog.clear()
    torch._dynamo.reset()
    idx = torch.randint(0, 40, (6, 5, 16))
    with need_xpu_graph_logs():
        got = torch.compile(real_repeat, backend=backend, dynamic=False)(x, idx)
    assert torch.equal(got, real_repeat(x, idx))
    assert "Pattern.FusedGatherToCopy changed graph" not in caplog.text
    torch._dynamo.reset()


def test_masked_and_tensor_scale_attention_become_the_masked_kernel_call(caplog, backend):
    """A non-causal additive mask and the wrapped tensor scale both end in `mi355x_sdpa_masked` (reference forms:
    tests/common/test_fuse_sdpa.py `_sdpa_pattern_*` with a mask, `_sdpa_pattern_tensor_scale`); a boolean mask
    stays on aten."""
    B, H, S, D = 2, 4, 64, 128

    def att_mask(q, k, v, m):
        return torch.softmax((q @ k.transpose(-2, -1) / math.sqrt(D)) + m, dim=-1) @ v

    def att_tscale(q, k, v, s):
        return torch.matmul(q, k.transpose(-2, -1)).div(s).softmax(dim=-1).matmul(v)

    q, k, v = (torch.randn(B, H, S, D).to(bf16) for _ in range(3))
    gm = rewrite(backend, att_mask, q, k, v, torch.randn(1, H, S, S).to(bf16))
    assert "mi355x_sdpa_masked" in modules_called(gm), (modules_called(gm), aten_ops(gm))
    assert not any("softmax" in t or "bmm" in t for t in aten_ops(gm))
    torch._dynamo.reset()
    gm = rewrite(backend, att_tscale, q, k, v, torch.tensor([math.sqrt(D)]))
    assert "mi355x_sdpa_masked" in modules_called(gm) and "fused_sdpa" not in modules_called(gm), (modules_called(gm), aten_ops(gm))


def test_library_attention_with_a_mask_or_grouped_heads_reaches_the_kernels(caplog, backend):
    """F.scaled_dot_product_attention with attn_mask arrives as a backend-specific op that carries the mask as its
    bias (a boolean mask already turned into 0 / -inf): it becomes the masked kernel call.  The pre-dispatch composite op with
    enable_gqa=True (fewer key/value heads, query head h reading key/value head h // (H / Hkv)) is what the kernels
    compute, so the pregrad stage takes it as it is."""
    import torch.nn.functional as F

    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

    B, H, S, D = 2, 4, 64, 128
    q, k, v = (torch.randn(B, H, S, D).to(bf16) for _ in range(3))
    gm = rewrite(backend, lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m) * 2.0, q, k, v, torch.randn(B, 1, S, S).to(bf16))
    assert modules_called(gm) == ["mi355x_sdpa_masked"], (modules_called(gm), aten_ops(gm))
    torch._dynamo.reset()
    # a boolean mask reaches the backend op as where(mask, 0, -inf): an additive mask like any other
    gm = rewrite(backend, lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m) * 2.0, q, k, v, torch.rand(B, 1, S, S) > 0.5)
    assert modules_called(gm) == ["mi355x_sdpa_masked"] and any("where" in t for t in aten_ops(gm)), (modules_called(gm), aten_ops(gm))
    torch._dynamo.reset()
    train = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    args = [t.clone().requires_grad_(True) for t in (q, k[:, :2], v[:, :2])]
    with need_xpu_graph_logs(), pytest.raises(NotImplementedError):
        torch.compile(lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True) * 2.0, backend=train)(*args)
    pregrad = train.compiled_graphs[-2]
    calls = [n for n in pregrad.graph.nodes if n.op == "call_module"]
    assert [n.target for n in calls] == ["mi355x_sdpa"] and calls[0].args[3] is True
    assert tuple(calls[0].args[1].meta["val"].shape) == (B, 2, S, D)  # the key/value heads go to the kernel unrepeated
    torch._dynamo.reset()


def test_repeated_key_value_heads_go_to_the_kernel_unrepeated(caplog, backend):
    """Grouped-query attention as decoders write it -- `repeat_kv` (index with None, expand, reshape) or
    repeat_interleave(n, dim=1) in front of the attention: the copies that repeat the heads disappear and the kernel
    call gets the [B, Hkv, S, D] tensors (query head h reads key/value head h // n).  Heads repeated in another order
    (`repeat`) stay as they are."""
    import torch.nn.functional as F

    B, H, Hkv, S, D = 2, 8, 2, 64, 128

    def repeat_kv(h, n):
        b, hk, s, d = h.shape
        return h[:, :, None, :, :].expand(b, hk, n, s, d).reshape(b, hk * n, s, d)

    q = torch.randn(B, H, S, D).to(bf16)
    k, v = (torch.randn(B, Hkv, S, D).to(bf16) for _ in range(2))
    for fn in (lambda q, k, v: F.scaled_dot_product_attention(q, repeat_kv(k, 4), repeat_kv(v, 4), is_causal=True) * 2.0,
               lambda q, k, v: F.scaled_dot_product_attention(q, k.repeat_interleave(4, dim=1), v.repeat_interleave(4, dim=1)) * 2.0):
        gm = rewrite(backend, fn, q, k, v)
        call = next(n for n in gm.graph.nodes if n.target == "mi355x_sdpa")
        assert tuple(call.args[1].meta["val"].shape) == (B, Hkv, S, D) and tuple(call.args[2].meta["val"].shape) == (B, Hkv, S, D)
        assert not any("expand" in t or "clone" in t for t in aten_ops(gm)), aten_ops(gm)
        torch._dynamo.reset()
    gm = rewrite(backend, lambda q, k, v: F.scaled_dot_product_attention(q, k.repeat(1, 4, 1, 1), v.repeat(1, 4, 1, 1)) * 2.0, q, k, v)
    call = next(n for n in gm.graph.nodes if n.target == "mi355x_sdpa")
    assert tuple(call.args[1].meta["val"].shape) == (B, H, S, D)  # head h reads key/value head h % Hkv there: not the kernels' rule
    torch._dynamo.reset()
