"""GPU parity of the attention backward kernels (torch.ops.xpu_ops.sdpa_lse / sdpa_bwd -> xg_sdpa_lse,
xg_sdpa_backward).

Reference: autograd of softmax(q k^T * scale + causal mask) v evaluated in fp32 on the SAME bf16 / fp16 inputs, with
the same upstream gradient.  Tolerance: rtol 1.6e-2 plus the gradient floor of tests/tolerance.py.  The reference
project's bar for training graphs is that compiled and eager gradients agree (tests/common/test_training.py:30-80);
the cases are those of the forward tests: self and cross attention, ragged tails, causal masking, grouped heads,
strided views.
"""
import math

import pytest
import torch

from tests.test_gpu_sdpa import make, ref32, ref32_masked
from tests.tolerance import assert_close_16bit, attention_floor, attention_grad_floor

pytestmark = pytest.mark.gpu


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def ref_grads(q, k, v, g, causal, scale):
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    out = ref32(qf, kf, vf, causal, scale)
    return (out.detach(), *torch.autograd.grad(out, (qf, kf, vf), g.float()))


def ref_lse(q, k, causal, scale):
    rep = q.shape[1] // k.shape[1]
    s = torch.matmul(q.float(), k.float().repeat_interleave(rep, dim=1).transpose(-1, -2)) * scale
    if causal:
        s = s + torch.full(s.shape[-2:], float("-inf"), device=q.device).triu(1)
    return torch.logsumexp(s, dim=-1)


def cancel_noise(q, k, v, g, scale):
    """dq and dk are sums of P (dP - delta) terms, and dP - delta cancels exactly where a row's softmax is
    saturated (one visible key): there the fp32 reference gives 0 and the kernel, which adds the same products in
    another order, gives fp32 rounding noise.  Bound: 2^-20 of |g| |v| D |scale| max(|q|, |k|)."""
    D = q.shape[-1]
    return 2.0**-20 * (g.abs().max() * v.abs().max() * D * abs(scale) * max(q.abs().max(), k.abs().max())).item()


def close_grad(got, want, what, noise=0.0):
    floor = attention_grad_floor(want, got.dtype) + noise
    assert_close_16bit(got, want, floor, f"sdpa_bwd {what} {tuple(got.shape)} {got.dtype}")


def run_backward(q, k, v, g, causal, scale):
    out, lse = _ops().sdpa_lse(q, k, v, causal, scale)
    return (out, lse, *_ops().sdpa_bwd(q, k, v, out, g, lse, causal, scale))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Sq,Skv", [(256, 256), (128, 64), (1, 1), (1, 300), (129, 65), (200, 333), (333, 200), (64, 1000), (640, 512), (16, 640)])
def test_backward_shapes(device, dtype, D, causal, Sq, Skv):
    q, k, v = make(2, 3, 3, Sq, Skv, D, dtype, device, seed=Sq + Skv + D)
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(7)).to(dtype).to(device)
    scale = 1.0 / math.sqrt(D)
    out, lse, dq, dk, dv = run_backward(q, k, v, g, causal, scale)
    assert torch.equal(out, _ops().sdpa(q, k, v, causal, scale))  # the same kernel with one more store
    torch.testing.assert_close(lse, ref_lse(q, k, causal, scale), rtol=1e-4, atol=1e-4)
    want_out, wq, wk, wv = ref_grads(q, k, v, g, causal, scale)
    assert_close_16bit(out, want_out, attention_floor(want_out, dtype), f"sdpa {tuple(out.shape)} {dtype}")
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape and dq.dtype == dtype
    noise = cancel_noise(q, k, v, g, scale)
    close_grad(dq, wq, "dq", noise)
    close_grad(dk, wk, "dk", noise)
    close_grad(dv, wv, "dv")


def test_backward_grouped_heads_and_strided_views(device):
    """Four query heads per key/value head (their gradients are summed inside the kernel); q, k, v, and the upstream
    gradient are [B, S, H, D] storage viewed as [B, H, S, D], as a llama block hands them over."""
    B, H, Hkv, S, D = 2, 8, 2, 320, 128
    gen = torch.Generator().manual_seed(3)
    q = torch.randn(B, S, H, D, generator=gen).bfloat16().to(device).transpose(1, 2)
    k = torch.randn(B, S, Hkv, D, generator=gen).bfloat16().to(device).transpose(1, 2)
    v = torch.randn(B, S, Hkv, D, generator=gen).bfloat16().to(device).transpose(1, 2)
    g = torch.randn(B, S, H, D, generator=gen).bfloat16().to(device).transpose(1, 2)
    for causal in (True, False):
        out, lse, dq, dk, dv = run_backward(q, k, v, g, causal, 0.09)
        _, wq, wk, wv = ref_grads(q, k, v, g, causal, 0.09)
        assert dq.stride() == q.stride() and dk.stride() == k.stride() and dv.stride() == v.stride()  # written in place of the layouts they came in
        close_grad(dq, wq, "dq gqa")
        close_grad(dk, wk, "dk gqa")
        close_grad(dv, wv, "dv gqa")
        again = _ops().sdpa_bwd(q, k, v, out, g, lse, causal, 0.09)
        assert all(torch.equal(a, b) for a, b in zip(again, (dq, dk, dv)))  # no atomics: run to run identical


@pytest.mark.parametrize("scale", [-0.2, 0.0, 1.0])
def test_backward_scale_sign_and_zero(device, scale):
    q, k, v = make(1, 2, 2, 150, 170, 64, torch.float16, device, seed=11)
    q, k = q * 0.3, k * 0.3
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(5)).half().to(device)
    _, _, dq, dk, dv = run_backward(q, k, v, g, True, scale)
    _, wq, wk, wv = ref_grads(q, k, v, g, True, scale)
    close_grad(dq, wq, "dq scale", cancel_noise(q, k, v, g, scale))
    close_grad(dk, wk, "dk scale", cancel_noise(q, k, v, g, scale))
    close_grad(dv, wv, "dv scale")


def test_autograd_runs_the_backward_kernels(device):
    """loss.backward() through the plain op (which recomputes the row statistics) and through the op that saved them
    gives the kernels' gradients, bit for bit."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    q, k, v = make(2, 4, 2, 192, 192, 128, torch.bfloat16, device, seed=21)
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(9)).bfloat16().to(device)
    _, _, dq, dk, dv = run_backward(q, k, v, g, True, 0.1)
    for op in ("sdpa", "sdpa_lse"):
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        out = getattr(_ops(), op)(*leaves, True, 0.1)
        out = out[0] if op == "sdpa_lse" else out
        out.backward(g)
        for leaf, want in zip(leaves, (dq, dk, dv)):
            assert torch.equal(leaf.grad, want), op


def ref_grads_masked(q, k, v, g, mask, causal, scale):
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    out = ref32_masked(qf, kf, vf, mask, causal, scale)
    return (out.detach(), *torch.autograd.grad(out, (qf, kf, vf), g.float()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("mask_shape,mask_dtype", [("full", "same"), ("rows", "f32"), ("per_batch", "same"), ("per_head", "f32")])
@pytest.mark.parametrize("Sq,Skv", [(256, 256), (130, 77), (1, 300), (200, 333), (320, 512)])
def test_backward_with_an_additive_mask(device, dtype, D, mask_shape, mask_dtype, Sq, Skv):
    """Gradients of the attn_mask form (reference passes/patterns/common/fuse_scaled_dot_product_attention.py:184-234
    in a training graph): the backward kernels add the mask to the recomputed scores.  Masks broadcast over batch and /
    or heads, in the tensors' dtype or fp32, with -inf entries (padded keys; key 0 stays visible so that no row is
    empty), odd sizes, grouped heads, and a causal flag on top where the problem is square."""
    B, H, Hkv = 2, 4, 2
    q, k, v = make(B, H, Hkv, Sq, Skv, D, dtype, device, seed=Sq * 5 + Skv + D)
    gen = torch.Generator().manual_seed(Sq + 2 * Skv)
    shape = {"full": (B, H, Sq, Skv), "rows": (Sq, Skv), "per_batch": (B, 1, Sq, Skv), "per_head": (1, H, Sq, Skv)}[mask_shape]
    mask = torch.randn(shape, generator=gen)
    pad = torch.rand(shape[:-2] + (1, Skv), generator=gen) < 0.2
    pad[..., 0] = False
    mask = mask.masked_fill(pad.expand(shape), float("-inf")).to(dtype if mask_dtype == "same" else torch.float32).to(device)
    g = torch.randn(q.shape, generator=gen).to(dtype).to(device)
    scale = 1.0 / math.sqrt(D)
    for causal in ((False, True) if Sq == Skv else (False,)):
        out, lse = _ops().sdpa_masked_lse(q, k, v, mask, None, causal, scale)
        assert torch.equal(out, _ops().sdpa_masked(q, k, v, mask, None, causal, scale))
        dq, dk, dv = _ops().sdpa_masked_bwd(q, k, v, out, g, lse, mask, None, causal, scale)
        want_out, wq, wk, wv = ref_grads_masked(q, k, v, g, mask, causal, scale)
        assert_close_16bit(out, want_out, attention_floor(want_out, dtype), f"sdpa masked {tuple(out.shape)} {dtype}")
        noise = cancel_noise(q, k, v, g, scale)
        close_grad(dq, wq, f"dq mask {mask_shape}", noise)
        close_grad(dk, wk, f"dk mask {mask_shape}", noise)
        close_grad(dv, wv, f"dv mask {mask_shape}")


def test_backward_with_the_scale_in_a_device_tensor(device):
    """The tensor-scale form (reference passes/patterns/utils/default_replacements.py:39-55): the backward kernels read
    the scale on the device too; without a mask the gradients equal the by-value call's bit for bit, with one they
    match fp32 autograd."""
    q, k, v = make(2, 4, 2, 200, 264, 128, torch.bfloat16, device, seed=31)
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(3)).bfloat16().to(device)
    t = torch.tensor([0.07], device=device)
    out, lse = _ops().sdpa_masked_lse(q, k, v, None, t, False, 123.0)  # the by-value scale is ignored
    got = _ops().sdpa_masked_bwd(q, k, v, out, g, lse, None, t, False, 123.0)
    _, _, dq, dk, dv = run_backward(q, k, v, g, False, t.item())
    for a, b in zip(got, (dq, dk, dv)):
        assert torch.equal(a, b)
    mask = torch.randn(2, 1, 200, 264, generator=torch.Generator().manual_seed(5)).to(device)
    out, lse = _ops().sdpa_masked_lse(q, k, v, mask, t, False, 123.0)
    dq, dk, dv = _ops().sdpa_masked_bwd(q, k, v, out, g, lse, mask, t, False, 123.0)
    _, wq, wk, wv = ref_grads_masked(q, k, v, g, mask, False, 0.07)
    noise = cancel_noise(q, k, v, g, 0.07)
    close_grad(dq, wq, "dq mask + tensor scale", noise)
    close_grad(dk, wk, "dk mask + tensor scale", noise)
    close_grad(dv, wv, "dv mask + tensor scale")


def test_autograd_of_the_masked_op(device):
    """loss.backward() through sdpa_masked (which recomputes the row statistics) and sdpa_masked_lse gives the
    kernels' gradients bit for bit; a mask or a scale tensor that wants a gradient is refused, not ignored."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    q, k, v = make(2, 4, 4, 192, 160, 64, torch.float16, device, seed=23)
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(9)).half().to(device)
    mask = torch.randn(1, 4, 192, 160, generator=torch.Generator().manual_seed(2)).to(device)
    out, lse = _ops().sdpa_masked_lse(q, k, v, mask, None, False, 0.1)
    want = _ops().sdpa_masked_bwd(q, k, v, out, g, lse, mask, None, False, 0.1)
    for op in ("sdpa_masked", "sdpa_masked_lse"):
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        res = getattr(_ops(), op)(*leaves, mask, None, False, 0.1)
        res = res[0] if op == "sdpa_masked_lse" else res
        res.backward(g)
        for leaf, w in zip(leaves, want):
            assert torch.equal(leaf.grad, w), op
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
    learned = mask.clone().requires_grad_(True)
    with pytest.raises(NotImplementedError):
        _ops().sdpa_masked(*leaves, learned, None, False, 0.1).backward(g)


def test_backward_c5_full_size_holds_no_score_matrix(device):
    """B4 H32 S2048 D128 causal: peak memory stays far below one [B, H, S, S] matrix (1 GiB in bf16), and two
    (batch, head) pairs are checked against fp32 autograd."""
    B, H, S, D = 4, 32, 2048, 128
    q, k, v = make(B, H, H, S, S, D, torch.bfloat16, device, seed=2)
    g = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(4)).bfloat16().to(device)
    scale = 1.0 / math.sqrt(D)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    out, lse, dq, dk, dv = run_backward(q, k, v, g, True, scale)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - before
    tensors = 4 * B * H * S * D * 2 + 2 * B * H * S * 4  # out, dq, dk, dv + lse, delta
    assert extra <= tensors + (8 << 20), (extra, tensors)
    for b, h in ((0, 0), (3, 31)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        _, wq, wk, wv = ref_grads(q[sl], k[sl], v[sl], g[sl], True, scale)
        close_grad(dq[sl], wq, "dq c5")
        close_grad(dk[sl], wk, "dk c5")
        close_grad(dv[sl], wv, "dv c5")
