"""Symbolic shapes: with the batch dimension marked dynamic every pattern still fires (the kernels take the row
count at run time), and with every dimension symbolic (`dynamic=True`) nothing crashes -- what needs a static
width simply stays in Aten.  The reference runs most of its pattern tests in both modes
(e.g. tests/common/test_fuse_rmsnorm.py:125-157, tests/mlu/test_fuse_slice.py:167-178)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import eager, inputs
from xpu_graph_amd import mi355x_compiler

bf16 = torch.bfloat16


def _cases():
    x, p = inputs.c5_llama_block(B=2, S=32, hidden=256, inter=512)
    names = sorted(p)
    return {
        "rmsnorm": (lambda x, w: eager.rmsnorm_eager(x, w, 1e-6), (torch.randn(8, 64), torch.randn(64)), ["custom_rms_norm"]),
        "add_ln": (
            lambda x, r, g, b: eager.add_layernorm_eager(x, r, g, b, 1e-5),
            (torch.randn(8, 64).to(bf16), torch.randn(8, 64).to(bf16), torch.randn(64).to(bf16), torch.randn(64).to(bf16)),
            ["mi355x_fused_add_norm"],
        ),
        "slice_cat": (lambda s: torch.cat([s[:, o : o + 8] for o in (7, 100, 40, 200)], 1), (torch.randn(6, 256),), ["fuse_slice_cat"]),
        "addn": (lambda *ts: eager.addn_eager(list(ts)), tuple(torch.randn(6, 16) for _ in range(6)), ["mi355x_addn"]),
        "dense": (
            lambda x, W, b: F.silu(x @ W + b),
            (torch.randn(16, 64).to(bf16), torch.randn(64, 32).to(bf16), torch.randn(32).to(bf16)),
            ["custom_dense_layer_replacement"],
        ),
        "swiglu": (lambda x: eager.silu_mul_eager(x), (torch.randn(8, 64).to(bf16),), ["mi355x_silu_mul"]),
        "fused_slice": (lambda x: [x[:, s : s + 4] + 1 for s in (1, 9, 33)], (torch.randn(6, 64),), ["fused_slice_0"]),
        "slice_sum_cat": (lambda x: torch.cat([x[:, 0:a, :].sum(1) for a in (2, 4, 6)], 1), (torch.randn(5, 8, 16),), ["mi355x_slice_sum_cat_0"]),
        "sdpa": (
            lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True),
            tuple(torch.randn(2, 4, 32, 64).to(bf16) for _ in range(3)),
            ["mi355x_sdpa"],
        ),
        "llama": (
            lambda x, *ws: eager.llama_block_eager(x, dict(zip(names, ws)), n_heads=4),
            (x, *[p[n] for n in names]),
            ["custom_rms_norm", "custom_dense_layer_replacement", "custom_dense_layer_replacement", "custom_dense_layer_replacement",
             "mi355x_rope", "mi355x_rope", "mi355x_sdpa", "custom_dense_layer_replacement", "mi355x_fused_add_norm", "mi355x_dense_glu",
             "custom_dense_layer_replacement"],
        ),
    }


def _compile(fn, args, dynamic):
    backend = mi355x_compiler()
    torch._dynamo.reset()
    try:
        torch.compile(fn, backend=backend, dynamic=dynamic)(*args)
        reached = False
    except NotImplementedError:  # a custom op was asked to run on CPU tensors: the rewrite happened
        reached = True
    gm = backend.compiled_graphs[-1]
    return gm, reached


@pytest.mark.parametrize("name", list(_cases()))
def test_patterns_fire_with_a_symbolic_batch(name):
    fn, args, want = _cases()[name]
    lead = args[0].shape[0]
    for a in args:  # every operand that carries the batch
        if a.dim() >= 2 and a.shape[0] == lead and tuple(a.shape) != (lead, lead):
            torch._dynamo.mark_dynamic(a, 0)
    gm, reached = _compile(fn, args, dynamic=None)
    assert reached
    assert [n.target for n in gm.graph.nodes if n.op == "call_module"] == want
    shapes = [n.meta["val"].shape for n in gm.graph.nodes if n.op == "placeholder" and isinstance(n.meta.get("val"), torch.Tensor)]
    assert any(not isinstance(d, int) for s in shapes for d in s), "the batch was specialised"


@pytest.mark.parametrize("name", list(_cases()))
def test_fully_symbolic_graphs_do_not_crash(name):
    fn, args, _ = _cases()[name]
    gm, _ = _compile(fn, args, dynamic=True)
    gm.graph.lint()
