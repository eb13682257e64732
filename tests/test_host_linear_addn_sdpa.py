"""FusedAddMM, FusedAddN, FusedSDPA and the level-1 folds on the CPU default
path.  Cases follow tests/common/test_fuse_addmm.py:16-79,
test_fuse_addn.py:9-122 and test_fuse_sdpa.py:14-610 of the reference (their
eager forms re-typed here; unlike there, every numeric comparison is asserted)."""
import math

import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs


@pytest.fixture(scope="module")
def backend():
    return XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))


def run(backend, fn, *args, dynamic=False):
    with need_xpu_graph_logs():
        return torch.compile(fn, backend=backend, dynamic=dynamic)(*args)


# ---------------------------------------------------------------- addmm
@pytest.mark.parametrize(
    "bias_kind,fires",
    [("vector", True), ("matrix", True), ("row", True), ("scalar_tensor", True), ("python", True), ("column_broadcasts_out", False)],
)
def test_addmm(caplog, backend, bias_kind, fires):
    x, w = torch.randn(6, 8), torch.randn(8, 5)
    bias = {
        "vector": torch.randn(5),
        "matrix": torch.randn(6, 5),
        "row": torch.randn(1, 5),
        "scalar_tensor": torch.randn(()),
        "python": 0.25,
        "column_broadcasts_out": torch.randn(3, 6, 5),  # result is 3-d: not an addmm
    }[bias_kind]

    def fn(x, w, b):
        return torch.mm(x, w) + b

    got = run(backend, fn, x, w, bias)
    torch.testing.assert_close(got, fn(x, w, bias))
    assert ("Pattern.FusedAddMM changed graph" in caplog.text) == fires


def test_addmm_mm_with_second_user_not_fused(caplog, backend):
    def fn(x, w, b):
        m = torch.mm(x, w)
        return m + b, m

    x, w, b = torch.randn(4, 4), torch.randn(4, 4), torch.randn(4)
    a, m = run(backend, fn, x, w, b)
    torch.testing.assert_close(a, fn(x, w, b)[0])
    assert "Pattern.FusedAddMM changed graph" not in caplog.text


# ----------------------------------------------------------------- addn
def chain(*ts):
    acc = ts[0]
    for t in ts[1:]:
        acc = acc + t
    return acc


@pytest.mark.parametrize("n,fires", [(3, False), (4, True), (9, True), (32, True)])
def test_addn_chain_length(caplog, backend, n, fires):
    ts = [torch.randn(16, 8) for _ in range(n)]
    got = run(backend, chain, *ts)
    torch.testing.assert_close(got, chain(*ts), rtol=1e-5, atol=1e-5)
    assert ("Pattern.FusedAddN changed graph" in caplog.text) == fires


def test_addn_must_not_fuse(caplog, backend):
    def scalar_in_chain(a, b, c, d):
        return a + b + 1.0 + c + d  # the python scalar breaks the run of tensor adds

    def mixed_dtype(a, b, c, d):
        return a + b.half() + c + d

    def right_leaning(a, b, c, d):
        return a + (b + (c + d))  # only left operands are followed: order would change

    ts = [torch.randn(4, 4) for _ in range(4)]
    for fn in (scalar_in_chain, mixed_dtype, right_leaning):
        caplog.clear()
        torch._dynamo.reset()
        got = run(backend, fn, *ts)
        torch.testing.assert_close(got, fn(*ts))
        assert "Pattern.FusedAddN changed graph" not in caplog.text, fn.__name__


def test_addn_shared_partial_sum_kept(caplog, backend):
    def fn(a, b, c, d, e):
        p = a + b + c
        return p + d + e, p  # p has another user: the chain stops there

    ts = [torch.randn(4, 4) for _ in range(5)]
    out, p = run(backend, fn, *ts)
    torch.testing.assert_close(out, fn(*ts)[0])
    torch.testing.assert_close(p, fn(*ts)[1])


# ----------------------------------------------------------------- sdpa
B, H, S, D = 2, 4, 16, 8


def qkv(dtype=torch.float32, skv=S):
    g = torch.Generator().manual_seed(0)
    return (
        torch.randn(B, H, S, D, generator=g).to(dtype),
        torch.randn(B, H, skv, D, generator=g).to(dtype),
        torch.randn(B, H, skv, D, generator=g).to(dtype),
    )


def att_div(q, k, v, s):
    return torch.matmul(q, k.transpose(-2, -1)).div(s).softmax(dim=-1).matmul(v)


def att_mul(q, k, v, s):
    return torch.matmul(q, k.transpose(-2, -1)).mul(s).softmax(dim=-1).matmul(v)


def att_mask_add(q, k, v, m):
    return torch.softmax((q @ k.transpose(-2, -1) / math.sqrt(q.size(-1))) + m, dim=-1) @ v


def att_mask_sub(q, k, v, m):
    return torch.softmax((q @ k.transpose(-2, -1) * 0.3) - m, dim=-1) @ v


def att_noscale(q, k, v):
    return torch.softmax(q @ k.transpose(-2, -1), dim=-1) @ v


def att_fp32_softmax(q, k, v, m):
    w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(q.size(-1)) + m
    w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(w, v)


def att_baddbmm(q, k, v, m):
    q3, k3, v3 = (t.reshape(B * H, -1, D) for t in (q, k, v))
    w = torch.baddbmm(m, q3, k3.transpose(1, 2))
    return torch.bmm(torch.softmax(w, -1), v3).view(B, H, -1, D)


@pytest.mark.parametrize(
    "fn,extra",
    [
        (att_div, lambda: (math.sqrt(D),)),
        (att_mul, lambda: (1.0 / math.sqrt(D),)),
        (att_mask_add, lambda: (torch.randn(B, H, S, S),)),
        (att_mask_add, lambda: (torch.randn(S, S),)),
        (att_mask_add, lambda: (torch.randn(B, 1, 1, S),)),
        (att_mask_sub, lambda: (torch.randn(1, H, S, S),)),
        (att_noscale, lambda: ()),
        (att_fp32_softmax, lambda: (torch.randn(B, 1, S, S),)),
        (att_baddbmm, lambda: (torch.randn(B * H, S, S),)),
    ],
)
def test_sdpa_forms(caplog, backend, fn, extra):
    q, k, v = qkv()
    args = (q, k, v) + extra()
    got = run(backend, fn, *args)
    torch.testing.assert_close(got, fn(*args), rtol=1e-4, atol=1e-5)
    assert "Pattern.FusedSDPA changed graph" in caplog.text


def test_sdpa_cross_attention_lengths_and_half(caplog, backend):
    torch.manual_seed(0)  # bf16 results of two evaluation orders: keep the comparison reproducible
    q, k, v = qkv(torch.bfloat16, skv=24)
    m = torch.randn(B, H, S, 24).bfloat16()
    got = run(backend, att_fp32_softmax, q, k, v, m)
    assert is_similar(got.float(), att_fp32_softmax(q, k, v, m).float(), rtol=2e-2, atol=3e-2)
    assert "Pattern.FusedSDPA changed graph" in caplog.text


def test_sdpa_tensor_scale_is_unwrapped(caplog, backend):
    q, k, v = qkv()
    s = torch.tensor([math.sqrt(D)])
    got = run(backend, att_div, q, k, v, s)
    torch.testing.assert_close(got, att_div(q, k, v, s), rtol=1e-4, atol=1e-5)
    assert "Pattern.FusedSDPA changed graph" in caplog.text
    assert "Unwrap scale" in caplog.text


def test_sdpa_not_attention(caplog, backend):
    def fn(q, k, v):
        return torch.sigmoid(q @ k.transpose(-2, -1)) @ v  # no softmax

    q, k, v = qkv()
    got = run(backend, fn, q, k, v)
    torch.testing.assert_close(got, fn(q, k, v))
    assert "Pattern.FusedSDPA changed graph" not in caplog.text


# ---------------------------------------------------------------- folds
def test_level1_folds(caplog):
    be = XpuGraph(XpuGraphConfig(is_training=False))

    def fn(x):
        a = x.expand(4, 6)  # same shape
        b = a.view(4, 6)  # same shape
        c = b.view(2, 12).view(24)  # view of view
        d = torch.cat([c], dim=0)  # one-input cat
        e = d.clone().to(torch.float32)  # clone + same-dtype copy
        return e * 2

    x = torch.randn(4, 6)
    got = run(be, fn, x)
    assert torch.equal(got, fn(x))
    for name in ("FoldExpand", "FoldView0", "FoldView1", "FoldCat", "FoldClone"):
        assert f"Pattern.{name} changed graph" in caplog.text, name


def test_clone_feeding_output_is_kept():
    be = XpuGraph(XpuGraphConfig(is_training=False))

    def fn(x):
        return x.clone()

    x = torch.randn(3)
    y = torch.compile(fn, backend=be)(x)
    assert torch.equal(x, y) and y.data_ptr() != x.data_ptr()


def test_output_clone_of_private_intermediate_is_dropped():
    """Beyond the reference: the copy left over from cat([t]) of a fresh intermediate is removed even at a
    graph output, while clones that keep two outputs (or an output and an input) apart stay."""
    be = XpuGraph(XpuGraphConfig(is_training=False))
    x = torch.randn(4, 16)

    def single(x):
        return torch.cat([torch.cat([x[:, 0:4], x[:, 8:12]], dim=1)], dim=1)

    assert torch.equal(torch.compile(single, backend=be)(x), single(x))
    assert "aten.clone.default" not in [str(n.target) for n in be.compiled_graphs[-1].graph.nodes]

    def aliased(x):
        y = x + 1
        return y, y.clone(), x.clone(), x[:, :4].clone()

    got = torch.compile(aliased, backend=be)(x)
    for a, b in zip(got, aliased(x)):
        assert torch.equal(a, b)
    assert got[0].data_ptr() != got[1].data_ptr() and got[2].data_ptr() != x.data_ptr() and got[3].data_ptr() != x.data_ptr()


def test_matchers_respect_arguments_that_change_the_meaning(caplog):
    """add(mm, bias, alpha=2) is not addmm(bias); a softmax over the QUERY axis, or one that leaves in fp32, is not
    attention; a masked sum with alpha != 1 is not an additive mask."""
    import xpu_graph_amd
    from xpu_graph_amd.test_utils import need_xpu_graph_logs

    backend = xpu_graph_amd.XpuGraph(xpu_graph_amd.XpuGraphConfig(is_training=False, opt_level=xpu_graph_amd.OptLevel.level2, enable_cache=False))

    def scaled_bias(x, w, b):
        return torch.add(torch.mm(x, w), b, alpha=2.0)

    def softmax_over_queries(q, k, v):
        return torch.bmm(torch.softmax(torch.bmm(q, k.transpose(1, 2)) * 0.125, dim=1), v)

    def scaled_mask(q, k, v, m):
        return torch.bmm(torch.softmax(torch.add(torch.bmm(q, k.transpose(1, 2)) * 0.125, m, alpha=3.0), dim=-1), v)

    q, k, v = (torch.randn(4, 16, 64) for _ in range(3))
    m = torch.randn(4, 16, 16)
    with need_xpu_graph_logs():
        for fn, args in ((scaled_bias, (torch.randn(8, 16), torch.randn(16, 4), torch.randn(4))),
                         (softmax_over_queries, (q, k, v)), (scaled_mask, (q, k, v, m))):
            got = torch.compile(fn, backend=backend, dynamic=False)(*args)
            torch.testing.assert_close(got, fn(*args), rtol=1e-4, atol=1e-5)
            torch._dynamo.reset()
    assert "Pattern.FusedAddMM changed graph" not in caplog.text
    assert "Pattern.FusedSDPA changed graph" not in caplog.text


@pytest.mark.parametrize("is_training", [False, True])
@pytest.mark.parametrize(
    "in_dtype,bias_kind",
    [(torch.float32, torch.float32), (torch.float32, float), (torch.float32, None), (torch.bfloat16, torch.bfloat16),
     (torch.float16, torch.float16), (torch.bfloat16, torch.float32), (torch.float16, torch.bfloat16)],
)
def test_bmm_plus_bias_becomes_baddbmm(caplog, is_training, in_dtype, bias_kind):
    """The batched twin of mm + bias (reference tests/common/test_fuse_baddbmm.py:15-90): tensor, python-number and
    absent biases, biases of another type than the product."""
    import torch.nn.functional as F

    import xpu_graph_amd
    from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs

    def fn(x, w, bias=None):
        out = torch.bmm(x, w)
        out = out + bias if bias is not None else out
        return F.gelu(out)

    backend = xpu_graph_amd.XpuGraph(xpu_graph_amd.XpuGraphConfig(is_training=is_training, opt_level=xpu_graph_amd.OptLevel.level2, enable_cache=False))
    x = torch.randn(64, 37, 16, dtype=in_dtype)
    w = torch.randn(64, 16, 16, dtype=in_dtype, requires_grad=is_training)
    if bias_kind is float:
        bias = 3.0
    elif bias_kind is None:
        bias = None
    else:
        bias = torch.randn(16, dtype=bias_kind, requires_grad=is_training)
    want = fn(x, w, bias)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend, dynamic=is_training)(x, w, bias)
    assert got.dtype == want.dtype
    assert is_similar(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    assert ("Pattern.FusedBAddBMM changed graph" in caplog.text) == (bias is not None)
    torch._dynamo.reset()
