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

from tests.test_gpu_sdpa import make, ref32
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
@pytest.mark.parametrize("Sq,Skv", [(256, 256), (128, 64), (1, 1), (1, 300), (129, 65), (200, 333), (333, 200), (64, 1000), (640, 512)])
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
