"""GPU parity of the attention kernel (torch.ops.xpu_ops.sdpa -> xg_sdpa).

Reference: softmax(q k^T * scale + mask) v evaluated in fp32 on the SAME bf16 /
fp16 inputs (the oracle's formula with no intermediate rounding), tolerance
rtol 1.6e-2 with the attention floor of tests/tolerance.py (2^-9 of the largest
output for bf16: the probabilities are rounded to the storage type); the
oracle itself (which rounds the scores and probabilities to the storage dtype,
as the HF eager form does) is compared at the same tolerance.  Cases follow the
reference's tests/common/test_fuse_sdpa.py:14-610: self and cross attention,
unequal lengths, half precision, plus what the kernel adds: causal masking by
index, grouped heads, strided [B, S, H, D] views, ragged tails.
"""
import math

import pytest
import torch

from oracle import eager
from tests.tolerance import assert_close_16bit, attention_floor

pytestmark = pytest.mark.gpu


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def ref32(q, k, v, causal, scale):
    qf, kf, vf = q.float(), k.float(), v.float()
    rep = q.shape[1] // k.shape[1]
    if rep > 1:
        kf = kf.repeat_interleave(rep, dim=1)
        vf = vf.repeat_interleave(rep, dim=1)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if causal:
        Sq, Sk = q.shape[-2], k.shape[-2]
        s = s + torch.full((Sq, Sk), float("-inf"), device=q.device).triu(1)
    return torch.matmul(torch.softmax(s, dim=-1), vf)


def close(got, want):
    assert_close_16bit(got, want, attention_floor(want, got.dtype), f"sdpa {tuple(got.shape)} {got.dtype}")


def make(B, H, Hkv, Sq, Skv, D, dtype, device, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype).to(device)
    k = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype).to(device)
    v = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype).to(device)
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Sq,Skv", [(256, 256), (128, 64), (1, 1), (1, 300), (129, 65), (200, 333), (333, 200), (64, 1000)])
def test_sdpa_shapes(device, dtype, D, causal, Sq, Skv):
    q, k, v = make(2, 3, 3, Sq, Skv, D, dtype, device, seed=Sq + Skv + D)
    scale = 1.0 / math.sqrt(D)
    got = _ops().sdpa(q, k, v, causal, scale)
    assert got.shape == q.shape and got.dtype == dtype
    close(got, ref32(q, k, v, causal, scale))


def test_sdpa_and_rope_take_misaligned_views(device):
    """q / k / v cut out of a wider buffer at an offset that is not a multiple of 16 bytes (eager takes any view): the
    wrapper copies what the kernels' 16-byte loads cannot read in place."""
    big = torch.randn(2, 4, 96, 140, device=device).bfloat16()
    q, k, v = big[..., 3:131], big[..., 4:132], big[..., 7:135]
    scale = 1.0 / math.sqrt(128)
    close(_ops().sdpa(q, k, v, True, scale), ref32(q, k, v, True, scale))
    cos = torch.cos(torch.arange(96 * 128, device=device).reshape(96, 128) * 1e-3)
    sin = torch.sin(torch.arange(96 * 128, device=device).reshape(96, 128) * 1e-3)
    got = _ops().rope(q, cos, sin)
    qf = q.float()
    want = qf * cos + torch.cat([-qf[..., 64:], qf[..., :64]], -1) * sin
    torch.testing.assert_close(got.float(), want, rtol=1.6e-2, atol=2.0**-7 * want.abs().max().item())


def ref32_masked(q, k, v, mask, causal, scale):
    qf, kf, vf = q.float(), k.float(), v.float()
    rep = q.shape[1] // k.shape[1]
    if rep > 1:
        kf, vf = kf.repeat_interleave(rep, dim=1), vf.repeat_interleave(rep, dim=1)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if mask is not None:
        s = s + mask.float()
    if causal:
        s = s + torch.full(s.shape[-2:], float("-inf"), device=q.device).triu(1)
    return torch.matmul(torch.softmax(s, dim=-1), vf)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("mask_shape,mask_dtype", [("full", "same"), ("rows", "f32"), ("per_batch", "same"), ("per_head", "f32")])
@pytest.mark.parametrize("Sq,Skv", [(256, 256), (130, 77), (1, 300), (200, 333)])
def test_sdpa_additive_mask(device, dtype, D, mask_shape, mask_dtype, Sq, Skv):
    """attn_mask of the FusedSDPA form (reference tests/common/test_fuse_sdpa.py: `_sdpa_pattern_*` with a mask
    operand): any floating-point additive mask, broadcast over batch and / or heads, odd sizes (rows the kernel must
    read element by element), -inf entries (padding) and a causal flag on top."""
    B, H, Hkv = 2, 4, 2
    q, k, v = make(B, H, Hkv, Sq, Skv, D, dtype, device, seed=Sq * 3 + Skv + D)
    g = torch.Generator().manual_seed(Sq + Skv)
    shape = {"full": (B, H, Sq, Skv), "rows": (Sq, Skv), "per_batch": (B, 1, Sq, Skv), "per_head": (1, H, Sq, Skv)}[mask_shape]
    mask = torch.randn(shape, generator=g)
    pad = torch.rand(shape[:-2] + (1, Skv), generator=g) < 0.2  # padded keys, at least key 0 stays visible
    pad[..., 0] = False
    mask = mask.masked_fill(pad.expand(shape), float("-inf")).to(dtype if mask_dtype == "same" else torch.float32).to(device)
    scale = 1.0 / math.sqrt(D)
    got = _ops().sdpa_masked(q, k, v, mask, None, False, scale)
    assert got.shape == q.shape and got.dtype == dtype
    close(got, ref32_masked(q, k, v, mask, False, scale))
    if Sq == Skv:
        close(_ops().sdpa_masked(q, k, v, mask, None, True, scale), ref32_masked(q, k, v, mask, True, scale))


def test_sdpa_scale_from_a_device_tensor(device):
    """The scale arrives as a one-element tensor (the reference's sdpa_wrapped_scale reads it with .item()): the kernel
    reads it on the device, and the result equals the by-value call bit for bit."""
    q, k, v = make(2, 4, 4, 192, 160, 128, torch.bfloat16, device, seed=9)
    for value, dt in ((0.07, torch.float32), (1.0 / math.sqrt(128), torch.bfloat16)):
        t = torch.tensor([value], dtype=dt, device=device)
        got = _ops().sdpa_masked(q, k, v, None, t, False, 123.0)  # the by-value scale is ignored
        assert torch.equal(got, _ops().sdpa(q, k, v, False, t.float().item()))
    # a fully masked row is NaN, as in eager
    mask = torch.zeros(192, 160, device=device)
    mask[5] = float("-inf")
    out = _ops().sdpa_masked(q, k, v, mask, None, False, 0.1)
    assert torch.isnan(out[:, :, 5]).all() and not torch.isnan(out[:, :, 4]).any()
    with pytest.raises(ValueError):
        _ops().sdpa_masked(q, k, v, torch.zeros(3, 192, 160, device=device), None, False, 0.1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Hkv,Sq,Skv,D", [
    (1, 32, 32, 1, 2048, 128),   # one query row per head
    (2, 8, 2, 1, 1000, 128),     # four query heads share a key/value head and a workgroup; ragged last tile
    (2, 8, 2, 4, 513, 64),       # 16 packed rows, one key in the last tile
    (1, 8, 1, 5, 4100, 128),     # 40 rows do not fit one tile: one query head per workgroup
    (3, 4, 4, 32, 777, 64),      # the most rows a workgroup holds
    (1, 2, 1, 16, 640, 128),     # 32 packed rows exactly
    (1, 4, 4, 3, 8192, 128),     # long context: many key ranges per head
])
def test_sdpa_decode_sizes_split_the_keys(device, dtype, B, H, Hkv, Sq, Skv, D):
    """A decode step (at most 32 query rows per head, no causal flag) runs on the key-split kernel: against the fp32
    anchor, with the log-sum-exp of every row, on K / V held as [B, S, H, D] (a cache layout) as well, and through the
    C ABI with no workspace (one key range) and with the preferred one."""
    import ctypes

    from xpu_graph_amd import _lib

    q, k, v = make(B, H, Hkv, Sq, Skv, D, dtype, device, seed=Sq + Skv + D + H)
    scale = 1.0 / math.sqrt(D)
    want = ref32(q, k, v, False, scale)
    got = _ops().sdpa(q, k, v, False, scale)
    assert got.shape == q.shape and got.dtype == dtype
    close(got, want)
    out, lse = _ops().sdpa_lse(q, k, v, False, scale)
    assert torch.equal(out, got)
    rep = H // Hkv
    s = torch.matmul(q.float(), k.float().repeat_interleave(rep, dim=1).transpose(-1, -2)) * scale
    torch.testing.assert_close(lse, torch.logsumexp(s, dim=-1), rtol=1e-4, atol=1e-4)
    kc, vc = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (k, v))  # [B, S, Hkv, D] storage
    assert torch.equal(_ops().sdpa(q, kc, vc, False, scale), got)
    S3 = ctypes.c_int64 * 3
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    st = lambda t: S3(*t.stride()[:3])  # noqa: E731
    lib = _lib.lib()
    n_ws = lib.xg_sdpa_decode_workspace_floats(B, H, Hkv, Sq, Skv, D)
    code = 2 if dtype == torch.bfloat16 else 1
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for ws_floats in sorted({0, n_ws}):
        ws = torch.empty(max(ws_floats, 1), device=device)
        o = torch.full_like(q, float("nan"))
        rc = lib.xg_sdpa_decode(P(q), P(k), P(v), P(o), None, None, None, code, None, P(ws) if ws_floats else None, ws_floats, B, H, Hkv, Sq, Skv,
                                D, st(q), st(k), st(v), st(o), scale, code, stream)
        assert rc == 0
        close(o, want)
        if ws_floats == n_ws:
            assert torch.equal(o, got)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mask_shape,mask_dtype", [("full", "same"), ("rows", "f32"), ("per_batch", "same"), ("per_head", "f32")])
@pytest.mark.parametrize("H,Hkv,Sq,Skv,D", [(8, 8, 1, 1024, 128), (8, 2, 3, 777, 64), (4, 4, 32, 2050, 128)])
def test_sdpa_decode_sizes_with_a_mask_and_a_tensor_scale(device, dtype, mask_shape, mask_dtype, H, Hkv, Sq, Skv, D):
    """The attn_mask form at decode shapes (padding masks of batched decoding: [B, 1, 1 | Sq, Skv]) and the scale in a
    device tensor run on the key-split kernel as well; keys hidden with -inf, whole 32-key blocks of them included; a
    row hidden completely is NaN, as in eager."""
    B = 2
    q, k, v = make(B, H, Hkv, Sq, Skv, D, dtype, device, seed=Sq * 7 + Skv + D)
    g = torch.Generator().manual_seed(Sq + Skv)
    shape = {"full": (B, H, Sq, Skv), "rows": (Sq, Skv), "per_batch": (B, 1, Sq, Skv), "per_head": (1, H, Sq, Skv)}[mask_shape]
    mask = torch.randn(shape, generator=g)
    pad = torch.rand(shape[:-2] + (1, Skv), generator=g) < 0.2
    pad[..., 0] = False
    pad[..., 200:300] = True  # whole blocks of hidden keys
    mask = mask.masked_fill(pad.expand(shape), float("-inf")).to(dtype if mask_dtype == "same" else torch.float32).to(device)
    scale = 1.0 / math.sqrt(D)
    got = _ops().sdpa_masked(q, k, v, mask, None, False, scale)
    close(got, ref32_masked(q, k, v, mask, False, scale))
    t = torch.tensor([0.05], device=device)
    close(_ops().sdpa_masked(q, k, v, mask, t, False, 123.0), ref32_masked(q, k, v, mask, False, 0.05))
    assert torch.equal(_ops().sdpa_masked(q, k, v, None, t, False, 123.0), _ops().sdpa(q, k, v, False, t.item()))
    out, lse = _ops().sdpa_masked_lse(q, k, v, mask, None, False, scale)
    assert torch.equal(out, got)
    rep = H // Hkv
    s = torch.matmul(q.float(), k.float().repeat_interleave(rep, dim=1).transpose(-1, -2)) * scale + mask.float()
    torch.testing.assert_close(lse, torch.logsumexp(s, dim=-1), rtol=1e-4, atol=1e-4)
    if mask_shape == "rows":
        hidden = mask.clone()
        hidden[0] = float("-inf")
        out = _ops().sdpa_masked(q, k, v, hidden, None, False, scale)
        assert torch.isnan(out[:, :, 0]).all() and (Sq == 1 or not torch.isnan(out[:, :, 1:]).any())


def test_sdpa_matches_oracle_causal(device):
    q, k, v = make(1, 4, 4, 512, 512, 128, torch.bfloat16, device, seed=5)
    got = _ops().sdpa(q, k, v, True, 1.0 / math.sqrt(128))
    # the eager form rounds scores and probabilities to bf16 (up to one ulp of |out| <= 4), hence the wider floor
    torch.testing.assert_close(got.float(), eager.causal_sdpa_eager(q, k, v).float(), rtol=1.6e-2, atol=2e-2)


def test_sdpa_grouped_heads_and_strided_views(device):
    B, S, H, Hkv, D = 2, 320, 8, 2, 128
    g = torch.Generator().manual_seed(11)
    # [B, S, H, D] storage viewed as [B, H, S, D], as a projection followed by view + transpose leaves it
    q = torch.randn(B, S, H, D, generator=g).bfloat16().to(device).transpose(1, 2)
    k = torch.randn(B, S, Hkv, D, generator=g).bfloat16().to(device).transpose(1, 2)
    v = torch.randn(B, S, Hkv, D, generator=g).bfloat16().to(device).transpose(1, 2)
    assert not q.is_contiguous()
    for causal in (True, False):
        close(_ops().sdpa(q, k, v, causal, 0.1), ref32(q, k, v, causal, 0.1))


@pytest.mark.parametrize("scale", [-0.2, 0.0, 1.0])
def test_sdpa_scale_sign_and_zero(device, scale):
    q, k, v = make(1, 2, 2, 192, 192, 64, torch.bfloat16, device, seed=3)
    q = q * 0.3
    for causal in (True, False):
        close(_ops().sdpa(q, k, v, causal, scale), ref32(q, k, v, causal, scale))


def test_sdpa_invariants(device):
    """What the mathematics fixes regardless of size: rows of the softmax sum to one (v = const gives const);
    causal row 0 returns v[0]; one-hot attention (huge aligned scores) returns the selected value row exactly."""
    B, H, S, D = 1, 2, 384, 128
    q, k, v = make(B, H, H, S, S, D, torch.bfloat16, device, seed=9)
    ones = torch.full_like(v, 0.75)
    for causal in (True, False):
        out = _ops().sdpa(q, k, ones, causal, 0.09)
        assert torch.equal(out, ones)
    out = _ops().sdpa(q, k, v, True, 0.09)
    assert torch.equal(out[:, :, 0], v[:, :, 0])
    # keys = +-1 codes of their index; query i = 16 * code(i): score(i, i) = 16 * D, every other score is lower by
    # at least 32, so after the softmax only key i survives in bf16
    idx = torch.arange(S, device=device)
    bits = ((idx[:, None] >> torch.arange(9, device=device)[None, :]) & 1).float() * 2 - 1  # [S, 9]
    code = bits.repeat(1, D // 9 + 1)[:, :D]
    kk = code.bfloat16().expand(B, H, S, D).contiguous()
    qq = (16 * code).bfloat16().expand(B, H, S, D).contiguous()
    for causal in (True, False):
        out = _ops().sdpa(qq, kk, v, causal, 1.0)
        assert torch.equal(out, v)


def test_sdpa_c5_full_size(device):
    """The attention of benchmark config 5: B 4, 32 heads, S 2048, D 128, causal, bf16."""
    B, H, S, D = 4, 32, 2048, 128
    q, k, v = make(B, H, H, S, S, D, torch.bfloat16, device, seed=1)
    scale = 1.0 / math.sqrt(D)
    got = _ops().sdpa(q, k, v, True, scale)
    for b in range(B):  # reference one batch at a time: 32 x 2048 x 2048 fp32 scores = 512 MiB
        close(got[b : b + 1], ref32(q[b : b + 1], k[b : b + 1], v[b : b + 1], True, scale))
    ones = torch.ones_like(v)
    assert torch.equal(_ops().sdpa(q, k, ones, True, scale), ones)


def test_sdpa_c5_full_size_permutation_and_prefix_properties(device):
    """At the full C5 shape: heads and batches are independent problems, so permuting them permutes the output bit
    for bit (whatever workgroup order or XCD a head lands on); under the causal mask the first n query rows do not
    depend on later keys, so a prefix of the sequence gives the same first rows bit for bit; the same holds through
    strided [B, S, H, D] storage."""
    B, H, S, D = 4, 32, 2048, 128
    q, k, v = make(B, H, H, S, S, D, torch.bfloat16, device, seed=5)
    scale = 1.0 / math.sqrt(D)
    ops = _ops()
    base = ops.sdpa(q, k, v, True, scale)
    g = torch.Generator().manual_seed(3)
    ph = torch.randperm(H, generator=g).to(device)
    pb = torch.randperm(B, generator=g).to(device)
    got = ops.sdpa(q[pb][:, ph].contiguous(), k[pb][:, ph].contiguous(), v[pb][:, ph].contiguous(), True, scale)
    assert torch.equal(got, base[pb][:, ph])
    n = 1280  # ten query blocks; keys 1280.. are never visible to them
    pre = ops.sdpa(q[:, :, :n].contiguous(), k[:, :, :n].contiguous(), v[:, :, :n].contiguous(), True, scale)
    assert torch.equal(pre, base[:, :, :n])
    qs, ks, vs = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))  # [B, S, H, D] storage
    assert torch.equal(ops.sdpa(qs, ks, vs, True, scale), base)


def test_sdpa_rejects_what_the_kernel_cannot_take(device):
    q, k, v = make(1, 2, 2, 64, 64, 128, torch.bfloat16, device)
    with pytest.raises(Exception):
        _ops().sdpa(q.float(), k.float(), v.float(), False, 1.0)  # fp32 has no kernel
    q96, k96, v96 = make(1, 2, 2, 64, 64, 96, torch.bfloat16, device)
    with pytest.raises(Exception):
        _ops().sdpa(q96, k96, v96, False, 1.0)  # head dim 96
    with pytest.raises(Exception):
        _ops().sdpa(q, k[:, :1], v, False, 1.0)  # k / v disagree
    empty = _ops().sdpa(q[:, :, :0], k, v, False, 1.0)
    assert empty.shape == (1, 2, 0, 128)
