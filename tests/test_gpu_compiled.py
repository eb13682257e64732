"""End to end on the GPU: the five benchmark functions, written in plain eager
torch, go through torch.compile with the mi355x target and must (a) be
rewritten to the fused custom calls, (b) run on the HIP kernels, (c) agree
with eager at the stated tolerance (bit-exact for slice/cat, rtol 1e-5 fp32,
rtol 1.6e-2 bf16).  This is the reference's own test recipe
(compile, compare with eager, look at the graph), e.g.
tests/common/test_fuse_rmsnorm.py:52-77, tests/mlu/test_fuse_addlayernorm.py:57-84."""
import operator

import pytest
import torch

from oracle import eager, inputs
from xpu_graph_amd import mi355x_compiler

pytestmark = pytest.mark.gpu


def run(fn, *args):
    backend = mi355x_compiler()
    compiled = torch.compile(fn, backend=backend, dynamic=False)
    with torch.no_grad():
        out = compiled(*args)
    gm = backend.compiled_graphs[-1]
    mods = [n.target for n in gm.graph.nodes if n.op == "call_module"]
    rest = [str(n.target) for n in gm.graph.nodes if n.op == "call_function" and n.target is not operator.getitem]
    return out, mods, rest


def test_c1_rmsnorm(device):
    x, w = inputs.c1_rmsnorm(device=device)
    out, mods, rest = run(lambda x, w: eager.rmsnorm_eager(x, w, 1e-6), x, w)
    assert mods == ["custom_rms_norm"] and rest == []
    torch.testing.assert_close(out, eager.rmsnorm_eager(x, w, 1e-6), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("form", ["library", "decomposed"])
def test_c2_add_layernorm(device, form):
    x, r, g, b = inputs.c2_add_layernorm(device=device)
    fn = eager.add_layernorm_eager if form == "library" else eager.add_layernorm_decomposed_eager
    (y, h), mods, rest = run(lambda x, r, g, b: fn(x, r, g, b, 1e-5), x, r, g, b)
    assert mods == ["mi355x_fused_add_norm"] and rest == []
    y_ref, h_ref = eager.add_layernorm_eager(x, r, g, b, 1e-5)
    assert torch.equal(h, h_ref)
    torch.testing.assert_close(y, y_ref, rtol=1.6e-2, atol=1e-2)


def test_add_rmsnorm(device):
    x, r, g, _ = inputs.c2_add_layernorm(rows=1024, device=device)
    (y, h), mods, rest = run(lambda x, r, w: eager.add_rmsnorm_eager(x, r, w, 1e-6), x, r, g)
    assert mods == ["mi355x_fused_add_norm"] and rest == []
    y_ref, h_ref = eager.add_rmsnorm_eager(x, r, g, 1e-6)
    assert torch.equal(h, h_ref)
    torch.testing.assert_close(y, y_ref, rtol=1.6e-2, atol=1e-2)


def test_c3_slice_cat_bit_exact(device):
    src, slices = inputs.c3_slice_cat(device=device)
    out, mods, rest = run(lambda s: eager.slice_cat_eager(s, slices), src)
    assert len(mods) == 1 and rest == [], (mods, rest)
    assert torch.equal(out, eager.slice_cat_eager(src, slices))


def test_c3_sum_of_32(device):
    ts = inputs.c3_addn(device=device)
    out, mods, rest = run(lambda *t: eager.addn_eager(list(t)), *ts)
    assert len(mods) == 1 and rest == [], (mods, rest)
    torch.testing.assert_close(out, eager.addn_eager(ts), rtol=1e-5, atol=1e-5)


def test_c3_slice_stack_sum_becomes_combo_sum(device):
    """Groups of column slices stacked and summed: one gather call + one combo-sum call
    (the graph of the reference's tests/mlu/test_slice_stack_sum.py)."""
    src = torch.randn(1024, 512, generator=torch.Generator().manual_seed(0)).to(device)

    def fn(src):
        a = torch.stack([src[:, 0:32], src[:, 64:96], src[:, 200:232], src[:, 300:332]], dim=0).sum(dim=0)
        b = torch.stack([src[:, 100:132], src[:, 400:432]], dim=0).sum(dim=0)
        return a, b

    outs, mods, rest = run(fn, src)
    assert "combo_sum" in mods and not any("aten.sum" in t or "aten.stack" in t or "aten.cat" in t for t in rest), (mods, rest)
    for o, ref in zip(outs, fn(src)):
        torch.testing.assert_close(o, ref, rtol=1e-5, atol=1e-5)


def test_c4_dense_silu(device):
    x, W, b = inputs.c4_dense(device=device)
    out, mods, rest = run(eager.dense_silu_eager, x, W, b)
    assert len(mods) == 1 and rest == [], (mods, rest)
    Wf, bf = W.float(), b.float()
    for r0 in range(0, 8192, 1024):  # every row against the fp32 evaluation
        want = torch.nn.functional.silu(x[r0 : r0 + 1024].float() @ Wf + bf)
        torch.testing.assert_close(out[r0 : r0 + 1024].float(), want, rtol=1.6e-2, atol=2e-2)
    torch.testing.assert_close(out, eager.dense_silu_eager(x, W, b), rtol=1.6e-2, atol=2e-2)


@pytest.mark.parametrize("form", ["mm", "mm_t_bias_sigmoid"])
def test_fp32_dense_layer_of_the_reference_tests(device, form):
    """The reference's dense-layer tests are fp32 (tests/mlu/test_custom_denselayer.py:11, 109-119: inputs
    [4096, 768], weight [768, 16] or [16, 768], bias [16]); compiled for the mi355x target they run on the fp32 MFMA
    kernel and agree with float64."""
    x = torch.randn(4096, 768, device=device)
    b = torch.randn(16, device=device)
    if form == "mm":
        w = torch.randn(768, 16, device=device)
        fn = lambda x, w: torch.matmul(x, w).reshape(128, 32, 16)  # noqa: E731
        args, want = (x, w), (x.double() @ w.double()).reshape(128, 32, 16)
        noise = want.abs().max().item() * 768**0.5 * 2.0**-24  # fp32 accumulation of 768 terms
    else:
        w = torch.randn(16, 768, device=device)
        fn = lambda x, w, b: torch.sigmoid(torch.matmul(x, w.transpose(0, 1)) + b)  # noqa: E731
        z = x.double() @ w.double().t() + b.double()
        args, want = (x, w, b), torch.sigmoid(z)
        noise = 0.25 * z.abs().max().item() * 768**0.5 * 2.0**-24  # the same noise through the sigmoid's largest slope
    out, mods, rest = run(fn, *args)
    assert mods == ["custom_dense_layer_replacement"], (mods, rest)
    assert not any("aten.mm" in t or "addmm" in t or "sigmoid" in t for t in rest), rest
    torch.testing.assert_close(out.double(), want, rtol=1e-5, atol=noise)


def test_swiglu(device):
    x = torch.randn(512, 2 * 1408, device=device).bfloat16()
    out, mods, rest = run(eager.silu_mul_eager, x)
    assert len(mods) == 1 and rest == [], (mods, rest)
    torch.testing.assert_close(out, eager.silu_mul_eager(x), rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("B,S", [(1, 256), (4, 2048)])
def test_c5_llama_block(device, B, S):
    x, p = inputs.c5_llama_block(B=B, S=S, device=device)
    names = sorted(p)

    def fn(x, *ws):
        return eager.llama_block_eager(x, dict(zip(names, ws)), n_heads=32)

    out, mods, rest = run(fn, x, *[p[n] for n in names])
    print("llama block modules:", mods)
    print("llama block remaining aten:", rest)
    assert "mi355x_sdpa" in mods and mods.count("mi355x_rope") == 2
    assert "mi355x_dense_glu" in mods and "mi355x_silu_mul2" not in mods  # gate and up projections share one kernel
    assert not any(k in t for t in rest for k in ("clone", "aten.cat", "aten.neg")), rest  # no layout copies, no unfused rotary math
    heavy = [t for t in rest if any(k in t for k in ("aten.mm", "aten.bmm", "aten.addmm", "softmax", "aten.matmul"))]
    assert heavy == [], heavy  # every matmul and the softmax went to custom kernels
    # A block is a chain of some twenty bf16 roundings; eager and fused round at different places, so both are
    # measured against the same block evaluated in fp32 from the same bf16 weights.  The fused path must be within
    # rtol 1.6e-2 of it, with an absolute floor equal to the eager bf16 path's OWN worst deviation from fp32, and
    # its mean error must not exceed eager's.
    with torch.no_grad():
        want_bf16 = fn(x, *[p[n] for n in names])
        want_f32 = eager.llama_block_eager(x.float(), {n: w.float() for n, w in p.items()}, n_heads=32)
    err_eager = (want_bf16.float() - want_f32).abs()
    err_fused = (out.float() - want_f32).abs()
    print(f"llama block B{B} S{S}: mean |err| fused {err_fused.mean().item():.4g} eager {err_eager.mean().item():.4g}; max fused {err_fused.max().item():.4g} eager {err_eager.max().item():.4g}")
    assert err_fused.mean().item() <= 1.05 * err_eager.mean().item()
    torch.testing.assert_close(out.float(), want_f32, rtol=1.6e-2, atol=err_eager.max().item())


@pytest.mark.parametrize("B,S", [(1, 700), (8, 2048)])
def test_c5_llama_block_decode_step(device, B, S):
    # One new token per sequence against S cached positions: every projection is a few rows against a whole weight
    # matrix, the rotary table is one row, and attention has one query row per head.
    H, D = 32, 128
    x, p = inputs.c5_llama_block(B=B, S=1, device=device)
    names = sorted(p)
    g = torch.Generator().manual_seed(11)
    kc = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(device)
    vc = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(device)
    ang = torch.rand(D // 2, generator=g) * 6.283
    cos = torch.cat([ang.cos(), ang.cos()]).to(torch.bfloat16).to(device)
    sin = torch.cat([ang.sin(), ang.sin()]).to(torch.bfloat16).to(device)

    def fn(x, kc, vc, cos, sin, *ws):
        return eager.llama_block_decode_eager(x, dict(zip(names, ws)), kc, vc, cos, sin, n_heads=H)

    (out, k_new, v_new), mods, rest = run(fn, x, kc, vc, cos, sin, *[p[n] for n in names])
    print("decode step modules:", mods)
    print("decode step remaining aten:", rest)
    assert "mi355x_sdpa" in mods and mods.count("mi355x_rope") == 2 and "mi355x_dense_glu" in mods
    heavy = [t for t in rest if any(k in t for k in ("aten.mm", "aten.bmm", "aten.addmm", "softmax", "aten.matmul"))]
    assert heavy == [], heavy
    with torch.no_grad():
        want_bf16 = fn(x, kc, vc, cos, sin, *[p[n] for n in names])
        want_f32 = eager.llama_block_decode_eager(
            x.float(), {n: w.float() for n, w in p.items()}, kc.float(), vc.float(), cos.float(), sin.float(), n_heads=H
        )
    for got, eb, ef, what in zip((out, k_new, v_new), want_bf16, want_f32, ("out", "k_new", "v_new")):
        err_eager = (eb.float() - ef).abs()
        err_fused = (got.float() - ef).abs()
        print(f"decode step B{B} S{S} {what}: mean |err| fused {err_fused.mean().item():.4g} eager {err_eager.mean().item():.4g}")
        assert err_fused.mean().item() <= 1.05 * err_eager.mean().item() + 1e-6
        torch.testing.assert_close(got.float(), ef, rtol=1.6e-2, atol=max(err_eager.max().item(), 1e-3))


@pytest.mark.parametrize("rank", [2, 3])
def test_fused_slice_compiled(device, rank):
    """Equally wide slices of one tensor, each with a consumer (reference tests/mlu/test_fuse_slice.py:43-60, 128-147):
    one gather per width, results bit-identical to eager."""
    starts = [12573, 11984, 11562, 9782, 9727, 9745, 9763, 9773, 9805, 9822, 10283, 10736]

    def fn(x):
        return [x[..., s : s + 4] + 1 for s in starts] + [x[..., s : s + 32] * 2 for s in starts[:5]]

    x = torch.randn(*((64, 43106) if rank == 2 else (10, 12, 43106)), device=device)
    out, mods, rest = run(fn, x)
    assert mods == ["fused_slice_0", "fused_slice_1"] and "aten.slice.Tensor" not in rest
    for got, want in zip(out, fn(x)):
        assert torch.equal(got, want)


@pytest.mark.parametrize("form", ["alone", "between", "with_other_sum"])
def test_slice_sum_cat_compiled(device, form):
    """tests/mlu/test_slice_sum_cat.py:13-58 (fn0, fn2, fn3) on the mi355x target."""
    params = [(0, 2), (0, 4), (0, 8), (0, 16)]
    x = torch.rand(86, 32, 32, device=device).half()
    other2 = torch.rand(86, 32, device=device).half()
    other3 = torch.rand(86, 32, 32, device=device).half()

    def fn(x, other):
        sums = [torch.sum(x[:, a:b, :], dim=[1]) for a, b in params]
        if form == "between":
            sums = [other] + sums + [other]
        elif form == "with_other_sum":
            sums = sums + [torch.sum(other, dim=[1])]
        return torch.cat(sums, dim=1)

    other = other3 if form == "with_other_sum" else other2
    out, mods, rest = run(fn, x, other)
    assert mods == ["mi355x_slice_sum_cat_0"] and "aten.slice.Tensor" not in rest
    torch.testing.assert_close(out, fn(x, other), rtol=1.6e-2, atol=1e-3)


def test_compile_cache_round_trip_runs_the_kernels(device, tmp_path, caplog):
    """What the artifact cache hands back after a reload still calls the HIP kernels and computes the same
    (reference tests/common/test_cache.py:14-55, here on the mi355x target)."""
    from xpu_graph_amd.test_utils import need_xpu_graph_logs

    src, slices = inputs.c3_slice_cat(rows=512, device=device)
    x, r, g, b = inputs.c2_add_layernorm(rows=512, device=device)

    def fn(src, x, r, g, b):
        y, h = eager.add_layernorm_eager(x, r, g, b, 1e-5)
        return eager.slice_cat_eager(src, slices), y, h

    backend = mi355x_compiler(cache=tmp_path)
    outs = []
    with need_xpu_graph_logs(), torch.no_grad():
        for _ in range(2):
            outs.append(torch.compile(fn, backend=backend, dynamic=False)(src, x, r, g, b))
            torch._dynamo.reset()
    assert caplog.text.count("Save cache in location") == 1 and caplog.text.count("Use cache in location") == 1
    mods = [n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"]
    assert sorted(mods) == ["fuse_slice_cat", "mi355x_fused_add_norm"]
    for a, c in zip(outs[0], outs[1]):
        assert torch.equal(a, c)
    assert torch.equal(outs[1][0], eager.slice_cat_eager(src, slices))


def test_interceptor_on_the_mi355x_target(device, caplog, tmp_path, monkeypatch):
    """The run-time guard compares the HIP path with the Dynamo graph on every call: silent at the bf16 tolerance,
    loud when the tolerance is set far below bf16 rounding."""
    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig
    from xpu_graph_amd.test_utils import need_xpu_graph_logs

    monkeypatch.setattr("xpu_graph_amd.config._dump_dir", str(tmp_path))
    x, W, b = inputs.c4_dense(512, 1024, 768, device=device)

    def run_with(tol):
        cfg = XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False, enable_interceptor=tol)
        backend = XpuGraph(cfg)
        with torch.no_grad():
            out = torch.compile(eager.dense_silu_eager, backend=backend, dynamic=False)(x, W, b)
        mods = [n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"]
        assert mods == ["custom_dense_layer_replacement"]
        return out

    with need_xpu_graph_logs():
        out = run_with("rtol=1.6e-2,atol=2e-2")
        assert "Monitored inference" in caplog.text and "diverges" not in caplog.text
        torch.testing.assert_close(out, eager.dense_silu_eager(x, W, b), rtol=1.6e-2, atol=2e-2)
        run_with("rtol=0,atol=1e-7")  # the fused epilogue rounds once, eager three times: not bit-identical
    assert "The inference pass diverges" in caplog.text


def test_dynamic_batch_one_compile_many_sizes(device):
    """The batch dimension marked dynamic: one compile serves several batch sizes, every fused kernel takes the row
    count at run time, results follow eager (reference tests compile most patterns with dynamic=True as well)."""
    import torch.nn.functional as F

    torch._dynamo.reset()
    offs = [7, 100, 40, 200]
    g = torch.Generator().manual_seed(3)
    w_norm = torch.randn(256, generator=g).to(device)
    W = (torch.randn(256, 128, generator=g) / 16).bfloat16().to(device)
    b = torch.randn(128, generator=g).bfloat16().to(device)

    def fn(src, x):
        cat = torch.cat([src[:, o : o + 8] for o in offs], dim=1)
        h = eager.rmsnorm_eager(x, w_norm, 1e-6)
        y = F.silu(h.bfloat16() @ W + b)
        return cat, h, y

    backend = mi355x_compiler()
    compiled = torch.compile(fn, backend=backend, dynamic=None)
    n_graphs = 0
    for rows in (48, 200, 7):
        src = torch.randn(rows, 512, generator=g).to(device)
        x = torch.randn(rows, 256, generator=g).to(device)
        torch._dynamo.mark_dynamic(src, 0)
        torch._dynamo.mark_dynamic(x, 0)
        with torch.no_grad():
            cat, h, y = compiled(src, x)
            cat_e, h_e, y_e = fn(src, x)
        if n_graphs == 0:
            n_graphs = len(backend.compiled_graphs)
            mods = sorted(n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module")
            assert mods == ["custom_dense_layer_replacement", "custom_rms_norm", "fuse_slice_cat"]
        assert torch.equal(cat, cat_e)
        torch.testing.assert_close(h, h_e, rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(y, y_e, rtol=1.6e-2, atol=2e-2)
    assert len(backend.compiled_graphs) == n_graphs  # no recompilation for the other batch sizes


@pytest.mark.parametrize("freeze", [False, True])
@pytest.mark.parametrize("name", ["Linear1", "RotateHalves", "InplaceAfterClone", "DataDependentScatter", "WithDropout"])
def test_model_zoo_on_the_mi355x_target(device, name, freeze):
    """The small-module zoo of tests/test_host_models.py (reference tests/common/test_models.py) on the GPU with the
    mi355x target, dynamic shapes, fp16: in-place updates, data-dependent shapes and dropout survive the rewrite;
    the linear layers run on the dense kernel."""
    import test_host_models as zoo

    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

    cls = getattr(zoo, name)
    golden, compiled = cls().to(device).half().eval(), cls().to(device).half().eval()
    compiled.load_state_dict(golden.state_dict())
    backend = XpuGraph(XpuGraphConfig(is_training=False, target=Target.mi355x, opt_level=OptLevel.level2, freeze=freeze, enable_cache=False))
    compiled.forward = torch.compile(compiled.forward, backend=backend, dynamic=True)
    x = torch.randn(80, zoo.DIM, device=device).half()
    keep = x.clone()
    with torch.inference_mode():
        with torch.random.fork_rng(device_type="cuda"):
            want = golden(keep)
        got = compiled(x)
    assert torch.equal(x, keep)
    assert got.shape == want.shape
    torch.testing.assert_close(got.float(), want.float(), rtol=1.6e-2, atol=2e-2)
    torch._dynamo.reset()


def _naive_layer_norm(x, w, b):
    dt = x.dtype
    x = x.to(torch.float32)
    mean = torch.mean(x, dim=-1, keepdim=True)
    var = torch.var(x, dim=-1, keepdim=True, unbiased=False)
    return (w * ((x - mean) / ((var + 1e-6) ** 0.5)) + b).to(dt)


def _layer_norm_between_pointwise(x, w, b):
    a = x * torch.sigmoid(x) * 0.1
    n = _naive_layer_norm(a, w, b)
    return n * n + 1e-6


@pytest.mark.parametrize("act_dtype,param_dtype", [(torch.float32, torch.float32), (torch.float32, torch.float16),
                                                   (torch.float16, torch.float16), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("fn", [_naive_layer_norm, _layer_norm_between_pointwise])
def test_layer_norm_with_mixed_activation_and_parameter_types(device, caplog, fn, act_dtype, param_dtype):
    """Activations and affine parameters of different types (reference tests/mlu/test_mixedtype_layernorm.py:19-92):
    the matcher fires and the kernel takes the mix."""
    from xpu_graph_amd.test_utils import need_xpu_graph_logs

    backend = mi355x_compiler()
    x = torch.randn(8, 1024, device=device, dtype=act_dtype)
    w = torch.randn(1024, device=device, dtype=param_dtype)
    b = torch.randn(1024, device=device, dtype=param_dtype)
    with need_xpu_graph_logs(), torch.no_grad():
        got = torch.compile(fn, backend=backend, dynamic=False)(x, w, b)
    assert "Pattern.FusedLayerNorm changed graph" in caplog.text
    mods = [str(n.target) for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"]
    assert any("norm" in m for m in mods), mods
    want = fn(x, w, b)
    assert got.dtype == want.dtype
    torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2)
    torch._dynamo.reset()


@pytest.mark.parametrize("param_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fn", [_naive_layer_norm, _layer_norm_between_pointwise])
def test_layer_norm_mixed_types_loss_and_grad(device, caplog, fn, param_dtype):
    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig
    from xpu_graph_amd.test_utils import need_xpu_graph_logs

    backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
    x = torch.randn(8, 1024, device=device, requires_grad=True)
    w = torch.randn(1024, device=device, dtype=param_dtype, requires_grad=True)
    b = torch.randn(1024, device=device, dtype=param_dtype, requires_grad=True)
    dy = torch.randn(8, 1024, device=device)
    with need_xpu_graph_logs():
        y0 = torch.compile(fn, backend=backend, dynamic=False)(x, w, b)
        g0 = torch.autograd.grad((y0,), (x, w, b), (dy,), allow_unused=True)
    assert "Pattern.FusedLayerNorm changed graph" in caplog.text
    y1 = fn(x, w, b)
    g1 = torch.autograd.grad((y1,), (x, w, b), (dy,), allow_unused=True)
    torch.testing.assert_close(y0.float(), y1.float(), rtol=1e-2, atol=1e-2)
    for a, c in zip(g0, g1):
        assert (a is None) == (c is None)
        if a is not None:
            assert a.dtype == c.dtype
            torch.testing.assert_close(a.float(), c.float(), rtol=2e-2, atol=2e-2 * max(1.0, c.float().abs().mean().item()))
    torch._dynamo.reset()


@pytest.mark.parametrize("form", ["erf", "tanh"])
def test_hand_written_gelu_runs_in_the_dense_epilogue_or_as_aten_gelu(device, form):
    """A GELU written out in elementary ops behind matmul + bias: the erf form becomes the dense kernel's activation
    (one launch); the tanh form becomes aten.gelu(approximate="tanh") behind a plain dense launch."""
    import math

    def fn(x, w, b):
        z = torch.addmm(b, x, w)
        if form == "erf":
            return 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))
        return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * torch.pow(z, 3.0))))

    g = torch.Generator().manual_seed(4)
    bf = torch.bfloat16
    x = torch.randn(384, 256, generator=g).to(bf).to(device)
    w = (torch.randn(256, 512, generator=g) / 16).to(bf).to(device)
    b = torch.randn(512, generator=g).to(bf).to(device)
    backend = mi355x_compiler()
    with torch.no_grad():
        got = torch.compile(fn, backend=backend, dynamic=False)(x, w, b)
    want = torch.nn.functional.gelu(torch.addmm(b.float(), x.float(), w.float()), approximate="none" if form == "erf" else "tanh")
    torch.testing.assert_close(got.float(), want, rtol=1.6e-2, atol=2e-2)
    calls = [str(n.target) for n in backend.compiled_graphs[-1].graph.nodes if n.op in ("call_module", "call_function")]
    if form == "erf":
        assert calls == ["custom_dense_layer_replacement"], calls
    else:
        assert calls == ["custom_dense_layer_replacement", "aten.gelu.default"], calls
    torch._dynamo.reset()


def test_sdpa_with_a_tensor_scale_runs_the_kernel_without_a_host_read(device):
    """The reference's tensor-scale form (tests/common/test_fuse_sdpa.py:608-610, `_sdpa_pattern_tensor_scale`):
    FusedSDPA wraps it in xpu_graph::sdpa_wrapped_scale, which reads the scale with .item(); on this target the
    kernel reads the one-element tensor itself."""
    import math

    from tests.tolerance import assert_close_16bit, attention_floor

    def att_div(q, k, v, s):
        return torch.matmul(q, k.transpose(-2, -1)).div(s).softmax(dim=-1).matmul(v)

    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 4, 256, 128, generator=g).bfloat16().to(device) for _ in range(3))
    s = torch.tensor([math.sqrt(128.0)], device=device)
    out, mods, rest = run(att_div, q, k, v, s)
    assert "mi355x_sdpa_masked" in mods and "fused_sdpa" not in mods, (mods, rest)
    assert not any("softmax" in t or "bmm" in t or "matmul" in t for t in rest), rest
    want = att_div(q.float(), k.float(), v.float(), s)
    assert_close_16bit(out, want, attention_floor(want, out.dtype), "sdpa tensor-scale compiled")


@pytest.mark.parametrize("mask_kind", ["per_head", "rows_f32", "padding"])
def test_sdpa_with_an_additive_mask_runs_the_kernel(device, mask_kind):
    """Masked attention written out in eager (the reference's `_sdpa_pattern_*` forms with a mask): FusedSDPA emits
    aten.scaled_dot_product_attention(attn_mask=...), the target hands the mask to the kernel."""
    import math

    from tests.tolerance import assert_close_16bit, attention_floor

    def att(q, k, v, m):
        return torch.softmax((q @ k.transpose(-2, -1) / math.sqrt(q.size(-1))) + m, dim=-1) @ v

    g = torch.Generator().manual_seed(1)
    B, H, S, D = 2, 4, 192, 128
    q, k, v = (torch.randn(B, H, S, D, generator=g).bfloat16().to(device) for _ in range(3))
    if mask_kind == "per_head":
        m = torch.randn(1, H, S, S, generator=g).bfloat16().to(device)
    elif mask_kind == "rows_f32":
        m = torch.randn(S, S, generator=g).to(device)
    else:
        m = torch.zeros(B, 1, S, S)
        m[0, :, :, 150:] = float("-inf")
        m[1, :, :, 100:] = float("-inf")
        m = m.bfloat16().to(device)
    out, mods, rest = run(att, q, k, v, m)
    assert "mi355x_sdpa_masked" in mods, (mods, rest)
    assert not any("softmax" in t or "bmm" in t for t in rest), rest
    want = att(q.float(), k.float(), v.float(), m.float())
    assert_close_16bit(out.to(torch.bfloat16) if out.dtype != torch.bfloat16 else out, want, attention_floor(want, torch.bfloat16), f"sdpa masked compiled {mask_kind}")


@pytest.mark.parametrize("mask_kind", ["additive", "boolean"])
@pytest.mark.parametrize("Sq,Skv", [(192, 192), (1, 1536), (8, 1024)])
def test_library_attention_with_a_mask_runs_the_kernel(device, mask_kind, Sq, Skv):
    """F.scaled_dot_product_attention(attn_mask=...) itself -- a float mask, or a boolean one that torch turns into
    0 / -inf -- at a prefill shape and at decode shapes (the key-split kernel): the graph calls the masked attention
    module and the result follows fp32 attention."""
    import torch.nn.functional as F

    from tests.test_gpu_sdpa import ref32_masked
    from tests.tolerance import assert_close_16bit, attention_floor

    g = torch.Generator().manual_seed(Sq + Skv)
    B, H, D = 2, 8, 128
    q = torch.randn(B, H, Sq, D, generator=g).bfloat16().to(device)
    k, v = (torch.randn(B, H, Skv, D, generator=g).bfloat16().to(device) for _ in range(2))
    if mask_kind == "additive":
        m = torch.randn(B, 1, Sq, Skv, generator=g).bfloat16().to(device)
        add = m
    else:
        m = torch.rand(B, 1, Sq, Skv, generator=g) < 0.8
        m[..., 0] = True  # every row sees key 0
        m = m.to(device)
        add = torch.zeros(B, 1, Sq, Skv, device=device).masked_fill(~m, float("-inf"))
    out, mods, rest = run(lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m), q, k, v, m)
    assert "mi355x_sdpa_masked" in mods, (mods, rest)
    want = ref32_masked(q, k, v, add, False, 1.0 / D**0.5)
    assert_close_16bit(out, want, attention_floor(want, torch.bfloat16), f"sdpa library mask {mask_kind} {Sq}x{Skv}")


@pytest.mark.parametrize("Sq,Skv,causal", [(256, 256, True), (1, 2048, False)])
def test_grouped_query_attention_of_a_decoder_runs_unrepeated(device, Sq, Skv, causal):
    """`repeat_kv` in front of the attention (the HF decoders' grouped-query form), prefill and decode: the kernel gets the
    [B, Hkv, S, D] keys and values, no repeated copy is made, and the result follows fp32 attention over the repeated heads."""
    import torch.nn.functional as F

    from tests.test_gpu_sdpa import ref32
    from tests.tolerance import assert_close_16bit, attention_floor

    def repeat_kv(h, n):
        b, hk, s, d = h.shape
        return h[:, :, None, :, :].expand(b, hk, n, s, d).reshape(b, hk * n, s, d)

    def att(q, k, v):
        return F.scaled_dot_product_attention(q, repeat_kv(k, 4), repeat_kv(v, 4), is_causal=causal)

    g = torch.Generator().manual_seed(Sq + Skv)
    q = torch.randn(2, 8, Sq, 128, generator=g).bfloat16().to(device)
    k, v = (torch.randn(2, 2, Skv, 128, generator=g).bfloat16().to(device) for _ in range(2))
    out, mods, rest = run(att, q, k, v)
    assert mods == ["mi355x_sdpa"] and not any("expand" in t or "clone" in t for t in rest), (mods, rest)
    want = ref32(q, k, v, causal, 128**-0.5)
    assert_close_16bit(out, want, attention_floor(want, torch.bfloat16), f"sdpa grouped compiled {Sq}x{Skv}")


@pytest.mark.parametrize("form", ["permuted_fp32_softmax", "permuted_prescaled_query", "permuted_divide", "decoder_output_transposed"])
def test_permuted_input_sdpa_forms_reach_the_kernel(device, form):
    """The reference's attention forms whose operands arrive as [B, S, H, E] and are permuted inside the function
    (tests/common/test_fuse_sdpa.py:166-262, `_sdpa_pattern_7` .. `_12`), and the decoder form that hands its result
    on transposed and contiguous (`_sdpa_pattern_transformer_1`, :490-506): each is rewritten to the HIP attention
    kernel, reads the permuted storage in place, and follows the fp32 evaluation of the same function."""
    from tests.test_host_sdpa_reference_forms import decoder, permuted_divide, permuted_fp32_softmax, permuted_prescaled_query
    from tests.tolerance import assert_close_16bit, attention_floor

    g = torch.Generator().manual_seed(7)
    B, S, H, D = 2, 320, 8, 128
    bf = torch.bfloat16
    if form == "decoder_output_transposed":
        q, k, v = (torch.randn(B, H, S, D, generator=g).to(bf).to(device) for _ in range(3))
        fn, args = decoder, (q, k, v)
    else:
        q, k, v = (torch.randn(B, S, H, D, generator=g).to(bf).to(device) for _ in range(3))
        fn = {"permuted_fp32_softmax": permuted_fp32_softmax, "permuted_prescaled_query": permuted_prescaled_query, "permuted_divide": permuted_divide}[form]
        args = (q, k, v, D**0.5) if form == "permuted_divide" else (q, k, v)
    out, mods, rest = run(fn, *args)
    assert any(m.startswith("mi355x_sdpa") for m in mods), (mods, rest)
    assert not any("softmax" in t or "bmm" in t or "matmul" in t for t in rest), rest
    want = fn(*(a.float() if torch.is_tensor(a) else a for a in args))
    assert out.shape == want.shape and out.dtype == bf
    assert_close_16bit(out, want, attention_floor(want, bf), f"sdpa compiled {form}")
