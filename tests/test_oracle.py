"""Pins the eager oracle (oracle/eager.py) with checks that do not repeat its
formulas: float64 numpy closed forms written independently, torch library
routines, invariants, brute force on tiny inputs, and the committed golden
fixtures.  A dropped eps, a wrong axis, a transposed operand or a mis-ordered
sum fails at least one of these."""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import eager, inputs

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def np64(t):
    return t.detach().double().numpy()


def test_rmsnorm_against_numpy_and_library():
    x, w = inputs.c1_rmsnorm(16, 256)
    X, W = np64(x), np64(w)
    want = X / np.sqrt((X * X).sum(axis=1, keepdims=True) / X.shape[1] + 1e-6) * W
    np.testing.assert_allclose(np64(eager.rmsnorm_eager(x, w, 1e-6)), want, rtol=2e-6, atol=1e-6)
    np.testing.assert_allclose(np64(eager.default_rms_norm(x, w, 1e-6)), want, rtol=2e-6, atol=1e-6)
    torch.testing.assert_close(eager.default_rms_norm(x, w, 1e-6), F.rms_norm(x, (256,), w, 1e-6))
    # eps matters (a dropped eps fails here): all-zero rows must give 0, not nan
    z = torch.zeros(2, 8)
    assert torch.equal(eager.rmsnorm_eager(z, torch.ones(8), 1e-6), z)
    # scale invariance: rmsnorm(c*x) == rmsnorm(x) for c > 0 when eps is negligible
    torch.testing.assert_close(eager.default_rms_norm(3 * x, w, 1e-12), eager.default_rms_norm(x, w, 1e-12), rtol=1e-5, atol=1e-6)


def test_layernorm_against_numpy_and_library():
    x, r, g, b = inputs.c2_add_layernorm(8, 128, dtype=torch.float32)
    X, G, Bv = np64(x), np64(g), np64(b)
    mu = X.mean(axis=1, keepdims=True)
    var = ((X - mu) ** 2).mean(axis=1, keepdims=True)  # population variance
    want = (X - mu) / np.sqrt(var + 1e-5) * G + Bv
    np.testing.assert_allclose(np64(eager.default_layer_norm(x, g, b, 1e-5)), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(eager.default_layer_norm(x, g, b, 1e-5), F.layer_norm(x, (128,), g, b, 1e-5), rtol=1e-5, atol=1e-5)
    # invariants: unit affine -> mean 0, variance 1 per row; shift invariance
    u = eager.default_layer_norm(x, None, None, 1e-12)
    np.testing.assert_allclose(np64(u).mean(axis=1), 0, atol=1e-6)
    np.testing.assert_allclose(np64(u).var(axis=1), 1, rtol=1e-4)
    torch.testing.assert_close(eager.default_layer_norm(x + 5.0, g, b, 1e-5), eager.default_layer_norm(x, g, b, 1e-5), rtol=1e-4, atol=1e-4)


def test_add_layernorm_rounds_the_sum_first():
    x, r, g, b = inputs.c2_add_layernorm(8, 128)
    y, h = eager.add_layernorm_eager(x, r, g, b, 1e-5)
    assert h.dtype == torch.bfloat16 and torch.equal(h, (x.float() + r.float()).bfloat16())
    H = np64(h)
    mu = H.mean(axis=1, keepdims=True)
    want = (H - mu) / np.sqrt(((H - mu) ** 2).mean(axis=1, keepdims=True) + 1e-5) * np64(g) + np64(b)
    np.testing.assert_allclose(np64(y), want, rtol=1.6e-2, atol=1e-2)
    y2, h2 = eager.add_layernorm_decomposed_eager(x, r, g, b, 1e-5)
    assert torch.equal(h2, h)
    np.testing.assert_allclose(np64(y2), want, rtol=1.6e-2, atol=4e-2)
    y3, h3 = eager.add_rmsnorm_eager(x, r, g, 1e-6)
    want3 = H / np.sqrt((H * H).mean(axis=1, keepdims=True) + 1e-6) * np64(g)
    assert torch.equal(h3, h)
    np.testing.assert_allclose(np64(y3), want3, rtol=1.6e-2, atol=1e-2)


def test_slice_cat_brute_force_and_fixture():
    src = torch.arange(5 * 40, dtype=torch.float32).reshape(5, 40)
    slices = [(3, 7), (0, 2), (39, 40), (10, 10), (20, 31)]
    got = eager.slice_cat_eager(src, slices)
    want = [[float(src[r, c]) for s, e in slices for c in range(s, e)] for r in range(5)]
    assert got.tolist() == want
    starts = inputs.c3_slice_offsets()
    fixture = json.load(open(os.path.join(GOLDEN, "c3_slice_offsets.json")))
    assert starts == fixture["starts"] == inputs.make_slice_offsets(64, 32, 8192, seed=0)
    assert len(starts) == 64 and len(set(starts)) == 64
    ivals = sorted((s, s + 32) for s in starts)
    assert all(a[1] <= b[0] for a, b in zip(ivals, ivals[1:])) and ivals[-1][1] <= 8192  # non-overlapping, in range
    assert any(s % 32 for s in starts) and any(s % 4 for s in starts)  # genuinely unaligned
    assert starts != sorted(starts)  # shuffled order


def test_addn_is_left_to_right_fp32():
    ts = inputs.c3_addn(32, 8, 16)
    got = eager.addn_eager(ts)
    acc = ts[0].numpy().copy()
    for t in ts[1:]:
        acc = (acc + t.numpy()).astype(np.float32)  # same association, one fp32 rounding per step
    assert np.array_equal(got.numpy(), acc)
    np.testing.assert_allclose(np64(got), sum(np64(t) for t in ts), rtol=1e-5, atol=1e-5)
    for o, t in zip(eager.combo_sum_eager([ts[0].reshape(8, 4, 4)], 1), [ts[0].reshape(8, 4, 4)]):
        np.testing.assert_allclose(np64(o), np64(t).sum(axis=1), rtol=1e-6)


def test_fused_slice_and_slice_sum_cat_brute_force():
    src = torch.arange(3 * 4 * 50, dtype=torch.float32).reshape(3, 4, 50)
    starts = [7, 0, 46, 13]
    got = eager.fused_slice_eager(src, starts, 4)
    assert got.shape == (4, 3, 4, 4)
    for k, s0 in enumerate(starts):
        for a in range(3):
            for b in range(4):
                assert got[k, a, b].tolist() == [float(a * 200 + b * 50 + s0 + c) for c in range(4)]
    x = torch.arange(2 * 6 * 3, dtype=torch.float32).reshape(2, 6, 3)
    params = [(0, 2), (0, 6), (3, 4), (2, 2)]
    out = eager.slice_sum_cat_eager(x, params)
    want = [[sum(float(x[b, r, c]) for r in range(a, e)) for a, e in params for c in range(3)] for b in range(2)]
    assert out.tolist() == want
    # prefix sums telescope: the slice (a, e) is the difference of two slices that start at row 0
    y = torch.randn(4, 16, 8, dtype=torch.float64)
    full = eager.slice_sum_cat_eager(y, [(0, 5), (0, 12), (5, 12)])
    np.testing.assert_allclose(full[:, 16:24].numpy(), (full[:, 8:16] - full[:, 0:8]).numpy(), rtol=1e-12, atol=1e-12)


def test_dense_against_numpy_and_identity():
    x, W, b = inputs.c4_dense(16, 32, 24, dtype=torch.float32)
    z = np64(x) @ np64(W) + np64(b)
    np.testing.assert_allclose(np64(eager.dense_silu_eager(x, W, b)), z / (1 + np.exp(-z)), rtol=1e-4, atol=1e-5)
    eye = torch.eye(32)
    torch.testing.assert_close(eager.dense_eager(x, eye, False, None, "none"), x)  # W = I returns x
    torch.testing.assert_close(eager.dense_eager(x, W.t().contiguous(), True, b, "relu"), torch.relu(x @ W + b))
    res = torch.randn(16, 24)
    torch.testing.assert_close(eager.dense_eager(x, W, False, res, "none"), x @ W + res)  # 2-D bias acts as a residual


def test_fp8_quantiser_known_answers():
    kat = json.load(open(os.path.join(GOLDEN, "fp8_e4m3fn_kat.json")))
    q = torch.tensor(kat["inputs"], dtype=torch.float32).to(torch.float8_e4m3fn)
    assert q.view(torch.uint8).tolist() == kat["codes"]
    assert q.float().tolist() == kat["decoded"]
    # spot values fixed by the format itself: 1.0 = 0x38, max finite 448 = 0x7e, ties to even
    assert kat["codes"][1] == 0x38 and kat["codes"][11] == 0x7E and kat["decoded"][2] == 1.0 and kat["decoded"][3] == 1.25
    x, W, b = inputs.c4_dense(8, 64, 16, dtype=torch.float32)
    xq, sx = eager.quantize_fp8_per_tensor(x)
    Wq, sw = eager.quantize_fp8_per_out_channel(W)
    assert sx.shape == (1,) and sw.shape == (16,)
    assert float(xq.float().abs().max()) == 448.0 and torch.all(Wq.float().abs().amax(0) == 448.0)  # absmax scaling hits the top code
    deq = (xq.float() * sx) @ (Wq.float() * sw)
    torch.testing.assert_close(deq, x @ W, rtol=0.1, atol=0.02)  # e4m3 has 3 mantissa bits
    z = np64(xq.float()) @ np64(Wq.float()) * float(sx) * np64(sw) + np64(b)
    np.testing.assert_allclose(np64(eager.dense_fp8_silu_eager(xq, Wq, sx, sw, b)), z / (1 + np.exp(-z)), rtol=1e-4, atol=1e-5)


def test_causal_sdpa_against_library_and_invariants():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 3, 16, 8, generator=g) for _ in range(3))
    got = eager.causal_sdpa_eager(q, k, v)
    torch.testing.assert_close(got, F.scaled_dot_product_attention(q, k, v, is_causal=True), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(got[:, :, 0], v[:, :, 0])  # the first query sees only the first key
    # brute force for one (batch, head)
    Q, K, V = np64(q[0, 0]), np64(k[0, 0]), np64(v[0, 0])
    out = np.zeros_like(Q)
    for i in range(16):
        s = Q[i] @ K[: i + 1].T / math.sqrt(8)
        p = np.exp(s - s.max())
        out[i] = (p / p.sum()) @ V[: i + 1]
    np.testing.assert_allclose(np64(got[0, 0]), out, rtol=1e-5, atol=1e-6)


def test_sdpa_against_library_brute_force_and_special_cases():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(2, 4, 3, 8, generator=g)
    k, v = (torch.randn(2, 2, 20, 8, generator=g) for _ in range(2))  # two query heads per key/value head
    mask = torch.randn(2, 1, 3, 20, generator=g)
    mask[0, 0, :, 5:9] = float("-inf")
    got = eager.sdpa_eager(q, k, v, mask, 0.3)
    kr, vr = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    torch.testing.assert_close(got, F.scaled_dot_product_attention(q, kr, vr, attn_mask=mask, scale=0.3), rtol=1e-5, atol=1e-6)
    # brute force, float64: query head 3 of batch 0 reads key/value head 1
    Q, K, V, M = np64(q[0, 3]), np64(k[0, 1]), np64(v[0, 1]), np64(mask[0, 0])
    out = np.zeros_like(Q)
    for i in range(3):
        sc = Q[i] @ K.T * 0.3 + M[i]
        pr = np.exp(sc - sc.max())
        out[i] = (pr / pr.sum()) @ V
    np.testing.assert_allclose(np64(got[0, 3]), out, rtol=1e-5, atol=1e-6)
    # one key: the output is that key's value row; a zero query: the mean of the values; default scale 1 / sqrt(D)
    torch.testing.assert_close(eager.sdpa_eager(q, k[:, :, :1], v[:, :, :1]), vr[:, :, :1].expand(2, 4, 3, 8))
    torch.testing.assert_close(eager.sdpa_eager(torch.zeros_like(q), k, v), vr.mean(dim=2, keepdim=True).expand(2, 4, 3, 8), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(eager.sdpa_eager(q, k, v), eager.sdpa_eager(q, k, v, None, 1 / math.sqrt(8)))


def test_silu_mul_and_rope_closed_forms():
    x = torch.randn(4, 32)
    a, b = np64(x[:, :16]), np64(x[:, 16:])
    np.testing.assert_allclose(np64(eager.silu_mul_eager(x)), a / (1 + np.exp(-a)) * b, rtol=1e-5, atol=1e-6)
    cos, sin = eager.rope_tables(8, 16)
    np.testing.assert_allclose(np64(cos) ** 2 + np64(sin) ** 2, 1.0, rtol=1e-6)
    assert torch.equal(cos[0], torch.ones(16)) and torch.equal(sin[0], torch.zeros(16))
    assert abs(float(cos[1, 0]) - math.cos(1.0)) < 1e-6 and abs(float(cos[1, 7]) - math.cos(10000.0 ** (-14 / 16))) < 1e-6


def test_llama_block_against_module_composition():
    """The block oracle against an independent composition from torch library modules."""
    x, p = inputs.c5_llama_block(B=1, S=16, hidden=64, inter=96, dtype=torch.float32)
    H = 4
    got = eager.llama_block_eager(x, p, n_heads=H)
    D = 64 // H
    h = F.rms_norm(x, (64,), p["ln1"], 1e-6)
    q, k, v = (F.linear(h, p[n]).view(1, 16, H, D).transpose(1, 2) for n in ("wq", "wk", "wv"))
    pos = torch.arange(16, dtype=torch.float32)
    inv = 10000.0 ** (-torch.arange(0, D, 2, dtype=torch.float32) / D)
    ang = pos[:, None] * inv[None, :]

    def rope(t):  # rotate pairs (i, i + D/2) by ang
        t1, t2 = t[..., : D // 2], t[..., D // 2 :]
        return torch.cat([t1 * ang.cos() - t2 * ang.sin(), t2 * ang.cos() + t1 * ang.sin()], dim=-1)

    o = F.scaled_dot_product_attention(rope(q), rope(k), v, is_causal=True).transpose(1, 2).reshape(1, 16, 64)
    x1 = x + F.linear(o, p["wo"])
    h2 = F.rms_norm(x1, (64,), p["ln2"], 1e-6)
    want = x1 + F.linear(F.silu(F.linear(h2, p["wg"])) * F.linear(h2, p["wu"]), p["wd"])
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)


def test_llama_block_decode_step_equals_the_last_position_of_the_whole_block():
    """Incremental decoding of the block: keys and values of earlier calls stored in the caches, then the step for the
    last token gives what the whole block gives at that position (the causal mask hides nothing from the last row)."""
    S, H, hidden = 9, 4, 64
    x, p = inputs.c5_llama_block(B=2, S=S, hidden=hidden, inter=96, dtype=torch.float32)
    D = hidden // H
    want = eager.llama_block_eager(x, p, n_heads=H)[:, S - 1 :]
    cos, sin = eager.rope_tables(S, D)
    k_cache, v_cache = torch.zeros(2, H, S, D), torch.zeros(2, H, S, D)
    empty = torch.zeros(2, H, 1, D)
    for t in range(S):
        _, k_new, v_new = eager.llama_block_decode_eager(x[:, t : t + 1], p, empty, empty, cos[t], sin[t], n_heads=H)
        k_cache[:, :, t : t + 1], v_cache[:, :, t : t + 1] = k_new, v_new
    got, _, _ = eager.llama_block_decode_eager(x[:, S - 1 :], p, k_cache, v_cache, cos[S - 1], sin[S - 1], n_heads=H)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    # and a middle position, against the block run on the prefix that ends there
    t = 4
    want_t = eager.llama_block_eager(x[:, : t + 1], p, n_heads=H)[:, t:]
    got_t, _, _ = eager.llama_block_decode_eager(x[:, t : t + 1], p, k_cache[:, :, : t + 1], v_cache[:, :, : t + 1], cos[t], sin[t], n_heads=H)
    torch.testing.assert_close(got_t, want_t, rtol=1e-5, atol=1e-5)
